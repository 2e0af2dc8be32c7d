"""trapetum_amd: Gemma-2 generation on one AMD MI355X, assembled from registered parts.

    from trapetum_amd import load_model
    engine = load_model("path/to/model", dtype="bfloat16")
    ids = engine.generate([[2, 651, 6037]], max_tokens=24)
"""
from .config import ConfigError, Gemma2Config   # noqa: F401
from .registry import (architecture, architectures, config_from_folder, register_architecture,   # noqa: F401
                       register_part)


def load_model(folder, **kw):
    from .engine import load_model as _load
    return _load(folder, **kw)


def __getattr__(name):
    if name in ("Engine", "Model", "Runtime", "generate"):
        from . import engine
        return getattr(engine, name)
    if name in ("SamplingParams",):
        from . import sampling
        return getattr(sampling, name)
    raise AttributeError(name)
