"""One registry from names to what they build.

Architectures: config.json["architectures"][0] -> (configuration class, function
from a configuration to a ModelSpec).  Parts: kind of part ("mixer",
"feed_forward", "norm", "position", "block", "embedding", "head") and a name
-> the class that implements it.  The reference dispatches by file magic to
one loader and one binary per architecture (runtime/src/lib.rs:1060-1062,
:4567); here a model is described as data and assembled from registered parts,
so adding an architecture is a registration, not new engine code.
"""
from .config.base import ConfigError, architecture_name, read_config_json

_ARCHITECTURES = {}
_PARTS = {}

PART_KINDS = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")


class Architecture:
    def __init__(self, name, config_cls, build_spec):
        self.name = name
        self.config_cls = config_cls
        self.build_spec = build_spec


def register_architecture(name, config_cls, build_spec):
    """`build_spec(config) -> ModelSpec`.  Registering a name again replaces it."""
    _ARCHITECTURES[name] = Architecture(name, config_cls, build_spec)


def architecture(name):
    _load_builtin()
    if name not in _ARCHITECTURES:
        known = ", ".join(sorted(_ARCHITECTURES)) or "none"
        raise ConfigError(f"unsupported architecture '{name}' (registered: {known})")
    return _ARCHITECTURES[name]


def architectures():
    _load_builtin()
    return sorted(_ARCHITECTURES)


def register_part(kind, name, cls):
    if kind not in PART_KINDS:
        raise ValueError(f"unknown kind of part '{kind}' (one of {', '.join(PART_KINDS)})")
    _PARTS[(kind, name)] = cls


def part_class(kind, name):
    _load_builtin()
    if (kind, name) not in _PARTS:
        known = ", ".join(sorted(n for k, n in _PARTS if k == kind)) or "none"
        raise ConfigError(f"no {kind} named '{name}' is registered (registered: {known})")
    return _PARTS[(kind, name)]


def build_part(kind, spec):
    """spec = (name, params dict) -> an instance."""
    name, params = spec
    return part_class(kind, name)(**params)


def config_from_folder(folder):
    d = read_config_json(folder)
    arch = architecture(architecture_name(d))
    return arch, arch.config_cls.from_dict(d)


_loaded = False


def _load_builtin():
    global _loaded
    if _loaded:
        return
    _loaded = True
    from . import parts      # noqa: F401  registers the built-in parts
    from . import models     # noqa: F401  registers the built-in architectures
