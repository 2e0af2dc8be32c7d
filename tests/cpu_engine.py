"""The engine's host logic on the CPU: the product's model, cache and step function with the plain
torch kernels of tests/ref_ops.py in the HIP library's place."""
import types

from trapetum_amd.engine.model import Model
from trapetum_amd.engine.runtime import Runtime
from trapetum_amd.registry import config_from_folder
from trapetum_amd.weights import load_folder

from . import ref_ops


def ref_ops_namespace():
    return types.SimpleNamespace(**{k: getattr(ref_ops, k) for k in dir(ref_ops) if not k.startswith("_")})


def load_cpu_model(folder, dtype="float32"):
    arch, cfg = config_from_folder(folder)
    rt = Runtime(dtype=dtype, device="cpu", ops=ref_ops_namespace())
    model = Model(arch.build_spec(cfg), rt)
    load_folder(model, folder)
    return model, cfg
