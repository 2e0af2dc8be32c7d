"""Typed configurations read from a model folder's config.json.

A configuration class names the config.json keys it needs; nothing that
config.json gives is repeated as a constant in code.  The reference has no
run-time configuration (its exporter reads the same keys from the checkpoint's
config and bakes them into a file header: model/export_gemma.py:40-46,
model/export_safetensors.py:171-183).
"""
import dataclasses
import json
import os


class ConfigError(ValueError):
    """config.json is missing a key, has a value of the wrong kind, or names sizes that do not fit together."""


_MISSING = object()


def key(name, kind, default=_MISSING, doc=""):
    """A dataclass field bound to the config.json key `name`."""
    meta = {"key": name, "kind": kind, "doc": doc, "required": default is _MISSING}
    if default is _MISSING:
        return dataclasses.field(metadata=meta)
    return dataclasses.field(default=default, metadata=meta)


def _coerce(name, kind, value):
    if kind == "int":
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value == int(value):
                return int(value)
            raise ConfigError(f"config key '{name}' must be an integer, found {value!r}")
        return int(value)
    if kind == "float":
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"config key '{name}' must be a number, found {value!r}")
        return float(value)
    if kind == "opt_float":                      # null or absent switches the feature off
        if value is None:
            return None
        return _coerce(name, "float", value)
    if kind == "opt_int":
        if value is None:
            return None
        return _coerce(name, "int", value)
    if kind == "bool":
        if not isinstance(value, bool):
            raise ConfigError(f"config key '{name}' must be true or false, found {value!r}")
        return value
    if kind == "str":
        if not isinstance(value, str):
            raise ConfigError(f"config key '{name}' must be a string, found {value!r}")
        return value
    if kind == "int_list":                       # a number or a list of numbers (eos_token_id is either:
        if value is None:                        # runtime/src/bin/serve.rs:88-101)
            return ()
        if isinstance(value, int) and not isinstance(value, bool):
            return (int(value),)
        if isinstance(value, (list, tuple)) and all(isinstance(v, int) and not isinstance(v, bool) for v in value):
            return tuple(int(v) for v in value)
        raise ConfigError(f"config key '{name}' must be an integer or a list of integers, found {value!r}")
    if kind == "str_list":
        if value is None:
            return None
        if isinstance(value, (list, tuple)) and all(isinstance(v, str) for v in value):
            return tuple(value)
        raise ConfigError(f"config key '{name}' must be a list of strings, found {value!r}")
    raise AssertionError(kind)


@dataclasses.dataclass
class ModelConfig:
    """Base of every architecture's configuration."""

    architecture = None          # the string in config.json["architectures"][0]; set by subclasses

    @classmethod
    def from_dict(cls, d):
        if not isinstance(d, dict):
            raise ConfigError("config.json must hold a JSON object")
        values = {}
        for f in dataclasses.fields(cls):
            m = f.metadata
            if "key" not in m:
                continue
            if m["key"] in d:
                values[f.name] = _coerce(m["key"], m["kind"], d[m["key"]])
            elif m["required"]:
                raise ConfigError(f"config.json has no '{m['key']}' ({cls.__name__} needs it: {m['doc']})")
        cfg = cls(**values)
        cfg.validate()
        return cfg

    @classmethod
    def from_kwargs(cls, **kw):
        """Build from config.json keys given as keyword arguments."""
        return cls.from_dict(kw)

    def to_dict(self):
        """The config.json object that reads back as this configuration."""
        d = {"architectures": [self.architecture]}
        for f in dataclasses.fields(self):
            m = f.metadata
            if "key" not in m:
                continue
            v = getattr(self, f.name)
            if isinstance(v, tuple):
                v = list(v)
            d[m["key"]] = v
        return d

    def validate(self):
        """Raise ConfigError when sizes do not fit together."""


def read_config_json(folder):
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"no config.json in model folder '{folder}'")
    with open(path) as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path} must hold a JSON object")
    return d


def architecture_name(d):
    archs = d.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json has no 'architectures' list naming the model class")
    return archs[0]
