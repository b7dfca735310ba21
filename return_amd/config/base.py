"""Typed model configuration and the one registry from architecture name to model.

The reference has no configuration class of its own: it reads HF config objects
(rollout/engine_actor.py:14-21) and picks the model class by a substring of
``config.model_type`` (rollout/engine_actor.py:24-32). Here a configuration is a
frozen dataclass filled from the keys of the architecture's own config.json, and
the registry maps ``architectures[0]`` to (configuration class, spec builder).
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, Callable, Dict, Tuple


class ConfigError(ValueError):
    """A config.json that this engine cannot run, with the key and the reason."""


_MISSING = object()


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    """Base of all architecture configurations.

    Subclasses declare their config.json keys as dataclass fields (a field without a
    default is required), may rename keys through ``KEY_ALIASES`` and check
    combinations in ``validate``. Keys that the class does not declare are kept in
    ``extra`` and ignored.
    """

    architecture: str

    KEY_ALIASES = {}          # field name -> config.json key, where they differ
    IGNORED_KEYS = ()         # keys known to be harmless (informational)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ModelConfig":
        raw = dict(raw)
        arch = raw.get("architectures") or [raw.get("architecture")]
        if not arch or not arch[0]:
            raise ConfigError("config.json has no 'architectures' entry")
        values = {"architecture": arch[0]}
        missing = []
        for f in dataclasses.fields(cls):
            if f.name == "architecture":
                continue
            key = cls.KEY_ALIASES.get(f.name, f.name)
            got = raw.get(key, _MISSING)
            if got is _MISSING or got is None:
                if f.default is dataclasses.MISSING and f.default_factory is dataclasses.MISSING:
                    if got is None and f.metadata.get("nullable"):
                        values[f.name] = None
                    else:
                        missing.append(key)
                continue
            values[f.name] = got
        if missing:
            raise ConfigError(f"{arch[0]}: config.json lacks required key(s): {', '.join(missing)}")
        cfg = cls(**values)
        cfg._coerce()
        cfg.validate(raw)
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "ModelConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def _coerce(self):
        """Bring JSON numbers to the declared field types (1e6 read as float for an int field, ...)."""
        for f in dataclasses.fields(self):
            v = getattr(self, f.name)
            if v is None:
                continue
            if f.type in ("int", int):
                if isinstance(v, bool) or float(v) != int(v):
                    raise ConfigError(f"{self.architecture}: {f.name} must be an integer, got {v!r}")
                object.__setattr__(self, f.name, int(v))
            elif f.type in ("float", float):
                object.__setattr__(self, f.name, float(v))
            elif f.type in ("bool", bool):
                if not isinstance(v, bool):
                    raise ConfigError(f"{self.architecture}: {f.name} must be true or false, got {v!r}")

    def validate(self, raw: Dict[str, Any]) -> None:  # pragma: no cover - overridden
        pass

    def to_dict(self) -> Dict[str, Any]:
        """The config.json this configuration is read back from."""
        out = {"architectures": [self.architecture]}
        for f in dataclasses.fields(self):
            if f.name == "architecture":
                continue
            out[self.KEY_ALIASES.get(f.name, f.name)] = getattr(self, f.name)
        return out

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=2)


# architecture name -> (configuration class, function(config) -> ModelSpec)
_ARCHITECTURES: Dict[str, Tuple[type, Callable]] = {}


def register_architecture(name: str, config_cls: type, build_spec: Callable) -> None:
    """Make ``name`` (the value of config.json's architectures[0]) loadable.

    ``build_spec(config)`` returns a ``return_amd.parts.spec.ModelSpec``: the parts of
    every block, the order the blocks run in, and the tensor names of their weights.
    """
    _ARCHITECTURES[name] = (config_cls, build_spec)


def lookup_architecture(name: str) -> Tuple[type, Callable]:
    if name not in _ARCHITECTURES:
        known = ", ".join(sorted(_ARCHITECTURES)) or "(none)"
        raise ConfigError(f"unknown architecture {name!r}; registered: {known}")
    return _ARCHITECTURES[name]


def registered_architectures():
    return sorted(_ARCHITECTURES)


def load_config(path: str) -> ModelConfig:
    """Read config.json (a file or a model folder) with the class its architecture names."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.exists(path):
        raise ConfigError(f"no config.json at {path}")
    with open(path) as f:
        raw = json.load(f)
    arch = raw.get("architectures") or [None]
    if not arch[0]:
        raise ConfigError(f"{path}: no 'architectures' entry")
    cls, _ = lookup_architecture(arch[0])
    return cls.from_dict(raw)
