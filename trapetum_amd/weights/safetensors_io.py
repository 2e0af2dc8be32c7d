"""Reading and writing safetensors files without a helper package.

Format as the reference's torch-free exporter reads it
(model/export_safetensors.py:24-48): 8 bytes little-endian header length, a JSON
header {name: {dtype, shape, data_offsets}} (offsets relative to the end of the
header, "__metadata__" skipped), then the raw little-endian data.  Sharded
folders carry model.safetensors.index.json with a weight_map (:51-60).
Tensors are memory-mapped and handed out as torch views, so a 50 GB model is
never held twice.
"""
import json
import mmap
import os
import struct

import torch


class WeightFileError(ValueError):
    """A weights file is missing, truncated or malformed."""


_DTYPES = {
    "BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafeTensorsFile:
    """One memory-mapped .safetensors file."""

    def __init__(self, path):
        self.path = path
        if not os.path.isfile(path):
            raise FileNotFoundError(f"no weights file '{path}'")
        size = os.path.getsize(path)
        if size < 8:
            raise WeightFileError(f"{path}: {size} bytes is too short for a safetensors header")
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_COPY)
        n = struct.unpack("<Q", self._mm[:8])[0]
        if 8 + n > size:
            raise WeightFileError(f"{path}: header of {n} bytes runs past the end of the file ({size} bytes)")
        try:
            header = json.loads(self._mm[8:8 + n].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{path}: header is not JSON: {e}") from None
        self._base = 8 + n
        self.entries = {}
        for name, meta in header.items():
            if name == "__metadata__":
                continue
            try:
                dt, shape, (s, e) = meta["dtype"], tuple(meta["shape"]), meta["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise WeightFileError(f"{path}: entry '{name}' lacks dtype, shape or data_offsets") from None
            if dt not in _DTYPES:
                raise WeightFileError(f"{path}: tensor '{name}' has unsupported dtype {dt}")
            count = 1
            for d in shape:
                count *= d
            want = count * torch.empty((), dtype=_DTYPES[dt]).element_size()
            if e - s != want or s < 0 or self._base + e > size:
                raise WeightFileError(
                    f"{path}: tensor '{name}' {dt}{list(shape)} needs {want} bytes, header gives "
                    f"[{s}, {e}) in a data section of {size - self._base} bytes")
            self.entries[name] = (_DTYPES[dt], shape, s, e)

    def names(self):
        return list(self.entries)

    def shape(self, name):
        return self.entries[name][1]

    def dtype(self, name):
        return self.entries[name][0]

    def tensor(self, name):
        """A read-only CPU view of the mapped bytes (copy it before the file is closed)."""
        dt, shape, s, e = self.entries[name]
        if e == s:
            return torch.empty(shape, dtype=dt)
        buf = memoryview(self._mm)[self._base + s:self._base + e]
        return torch.frombuffer(buf, dtype=dt).reshape(shape)

    def close(self):
        try:
            self._mm.close()
        except BufferError:         # views still alive; the map goes with them
            pass
        self._f.close()


class WeightFolder:
    """All tensors of a model folder: model.safetensors, or the shards its index names."""

    def __init__(self, folder):
        self.folder = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        if os.path.isfile(index):
            with open(index) as f:
                try:
                    files = sorted(set(json.load(f)["weight_map"].values()))
                except (json.JSONDecodeError, KeyError, AttributeError):
                    raise WeightFileError(f"{index} has no weight_map") from None
        elif os.path.isfile(single):
            files = ["model.safetensors"]
        else:
            raise FileNotFoundError(f"no model.safetensors (or model.safetensors.index.json) in '{folder}'")
        self.files = [SafeTensorsFile(os.path.join(folder, f)) for f in files]
        self._where = {}
        for sf in self.files:
            for name in sf.names():
                self._where[name] = sf

    def names(self):
        return list(self._where)

    def __contains__(self, name):
        return name in self._where

    def shape(self, name):
        return self._where[name].shape(name)

    def dtype(self, name):
        return self._where[name].dtype(name)

    def tensor(self, name):
        return self._where[name].tensor(name)

    def close(self):
        for sf in self.files:
            sf.close()


def write_safetensors(path, tensors, metadata=None):
    """Write {name: CPU tensor} in the order given."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().contiguous().cpu()
        if t.dtype not in _NAMES:
            raise WeightFileError(f"tensor '{name}' has dtype {t.dtype}, which safetensors cannot hold")
        raw = t.view(torch.uint8).reshape(-1).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hj += b" " * ((8 - len(hj) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for raw in blobs:
            f.write(raw)


def write_safetensors_streamed(path, layout, produce, metadata=None):
    """Write tensors one at a time: `layout` = {name: (torch dtype, shape)}, `produce(name)` -> CPU tensor.

    Only one tensor is alive at a time, so a folder larger than memory can be written."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, (dt, shape) in layout.items():
        if dt not in _NAMES:
            raise WeightFileError(f"tensor '{name}' has dtype {dt}, which safetensors cannot hold")
        count = 1
        for d in shape:
            count *= d
        n = count * torch.empty((), dtype=dt).element_size()
        header[name] = {"dtype": _NAMES[dt], "shape": list(shape), "data_offsets": [offset, offset + n]}
        offset += n
    hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hj += b" " * ((8 - len(hj) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for name, (dt, shape) in layout.items():
            t = produce(name).detach().contiguous().cpu()
            if t.dtype != dt or tuple(t.shape) != tuple(shape):
                raise WeightFileError(f"tensor '{name}': produced {t.dtype}{list(t.shape)}, layout says {dt}{list(shape)}")
            if t.numel():
                f.write(t.view(torch.uint8).reshape(-1).numpy().tobytes())
