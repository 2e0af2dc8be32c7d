"""Loading a model folder onto the GPU through the product's own path."""
import torch

from trapetum_amd.engine.model import Model
from trapetum_amd.engine.runtime import Runtime
from trapetum_amd.registry import config_from_folder
from trapetum_amd.weights import load_folder


def load_gpu_model(folder, dtype):
    arch, cfg = config_from_folder(folder)
    rt = Runtime(dtype=dtype, device="cuda:0")
    model = Model(arch.build_spec(cfg), rt)
    load_folder(model, folder)
    return model, cfg
