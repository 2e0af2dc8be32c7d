"""Weights by tensor name, checked against what the assembled model declares.

The reference's Gemma exporter walks the same names by attribute path
(model/export_gemma.py:60-73) and its torch-free exporter by string with the
tied-head fallback (model/export_safetensors.py:201-216); truncation there is a
panic (runtime/src/lib.rs:1113-1133).  Here every problem of a folder is found
before anything is uploaded and reported in one error.

Tensors keep their stored width on the way in: bf16 stays bf16, a tensor stored in
32 bits stays so, integer tables become int32.  Parts convert what their kernels
need when they bind (a float32 engine widens bf16 exactly; norm gains are always
formed in fp32).
"""
import torch

from .safetensors_io import WeightFolder


class WeightError(ValueError):
    """A model folder does not hold the tensors the model needs.  Lists everything that is wrong."""

    def __init__(self, folder, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.folder = folder
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"weights in '{folder}' do not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n}: expected {list(e)}, found {list(f)}" for n, e, f in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong dtypes ({len(self.wrong_dtype)}): " + "; ".join(
                f"{n}: expected {e}, found {f}" for n, e, f in self.wrong_dtype))
        super().__init__("\n".join(lines))


_FLOATS = (torch.bfloat16, torch.float16, torch.float32, torch.float64)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


def check_source(source, layout, folder="<memory>"):
    """Compare what `source` holds with the model's tensor layout; raise WeightError on any difference."""
    have = set(source.names())
    need = set(layout)
    missing = sorted(need - have)
    unexpected = sorted(have - need)
    wrong_shape, wrong_dtype = [], []
    for name in sorted(need & have):
        ts = layout[name]
        if tuple(source.shape(name)) != tuple(ts.shape):
            wrong_shape.append((name, tuple(ts.shape), tuple(source.shape(name))))
        dt = source.dtype(name)
        if ts.dtype == "float" and dt not in _FLOATS:
            wrong_dtype.append((name, "a floating-point type", str(dt)))
        if ts.dtype == "int" and dt not in _INTS:
            wrong_dtype.append((name, "an integer type", str(dt)))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(folder, missing, unexpected, wrong_shape, wrong_dtype)


def stored_to_device(t, device):
    """Keep the stored width: bf16 and fp32 as they are, fp16/fp64 to fp32, integers to int32."""
    if t.dtype in (torch.float16, torch.float64):
        t = t.to(torch.float32)
    elif t.dtype in _INTS and t.dtype != torch.int32:
        t = t.to(torch.int32)
    return t.to(device, copy=True)


def load_into(model, source, folder="<memory>"):
    """Check `source` (a WeightFolder or anything with names/shape/dtype/tensor) and bind the model to it."""
    check_source(source, model.tensor_layout(), folder)
    model.bind(lambda name: stored_to_device(source.tensor(name), model.rt.device))


def load_folder(model, folder):
    source = WeightFolder(folder)
    try:
        load_into(model, source, folder)
    finally:
        source.close()
