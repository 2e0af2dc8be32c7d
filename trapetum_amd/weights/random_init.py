"""Random weights from a configuration and a seed.

Every tensor the assembled model declares is drawn on its own generator keyed by
(seed, tensor name), so values do not depend on the order of generation:
matrices and the embedding ~ N(0, sigma), norm weights ~ N(0, sigma_norm) (the
effective gain of a (1 + w) norm is then 1 +- sigma_norm, like the reference's test
models: runtime/src/bin/model.rs:158-176).  Values are rounded to bfloat16, the
width a model folder stores.  `write_model_folder` writes config.json and
model.safetensors that load like any other model folder.
"""
import hashlib
import json
import os

import torch

from .safetensors_io import write_safetensors_streamed


def _seed_for(seed, name):
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


class RandomWeights:
    """A weight source (names / shape / dtype / tensor) that draws each tensor when asked."""

    def __init__(self, layout, seed, sigma=0.02, sigma_norm=0.1, store_dtype=torch.bfloat16, draw_on=None):
        """draw_on: a device to draw on instead of the CPU (faster for large models; other values than the
        CPU's for the same seed, so not what `write_model_folder` writes)."""
        self.draw_on = draw_on
        self.layout = layout
        self.seed = seed
        self.sigma = sigma
        self.sigma_norm = sigma_norm
        self.store_dtype = store_dtype

    def names(self):
        return list(self.layout)

    def shape(self, name):
        return tuple(self.layout[name].shape)

    def dtype(self, name):
        return torch.int32 if self.layout[name].dtype == "int" else self.store_dtype

    def tensor(self, name):
        ts = self.layout[name]
        g = torch.Generator().manual_seed(_seed_for(self.seed, name))
        if ts.dtype == "int":
            return torch.zeros(ts.shape, dtype=torch.int32)
        if ts.init == "zeros":
            return torch.zeros(ts.shape, dtype=self.store_dtype)
        if ts.init == "ones":
            return torch.ones(ts.shape, dtype=self.store_dtype)
        sigma = self.sigma_norm if ts.init == "norm" else self.sigma
        if self.draw_on is not None:
            gd = torch.Generator(device=self.draw_on).manual_seed(_seed_for(self.seed, name))
            t = torch.empty(ts.shape, dtype=torch.float32, device=self.draw_on).normal_(0.0, 1.0, generator=gd)
            return (t * sigma).to(self.store_dtype)
        t = torch.empty(ts.shape, dtype=torch.float32).normal_(0.0, 1.0, generator=g)
        return (t * sigma).to(self.store_dtype)


def write_model_folder(config, folder, seed, sigma=0.02, sigma_norm=0.1, store_dtype="bfloat16"):
    """Write config.json and model.safetensors of a randomly initialised model of `config`.  store_dtype
    "bfloat16" rounds the drawn values to bfloat16; "float32" stores them as drawn (and the engine keeps them so)."""
    from ..engine.model import Model
    from ..registry import architecture
    widths = {"bfloat16": torch.bfloat16, "float32": torch.float32}
    if store_dtype not in widths:
        raise ValueError(f"store_dtype '{store_dtype}' must be bfloat16 or float32")
    arch = architecture(config.architecture)
    layout = Model(arch.build_spec(config), rt=None).tensor_layout()
    source = RandomWeights(layout, seed, sigma, sigma_norm, store_dtype=widths[store_dtype])
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
    write_safetensors_streamed(
        os.path.join(folder, "model.safetensors"),
        {n: (source.dtype(n), source.shape(n)) for n in source.names()},
        source.tensor, metadata={"format": "pt", "seed": seed})
    return folder
