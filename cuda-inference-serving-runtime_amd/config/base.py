"""Typed configurations and the one registry from an architecture's name to
its configuration class and model builder.

config.json names its architecture twice: ``architectures[0]`` (a class name)
and ``model_type``.  Both are registered; lookup prefers the first.  The
reference has no registry, only a ``model_type == 'llama'`` check
(runtime/checkpoint.py:12).
"""
import json
from dataclasses import dataclass
from pathlib import Path


class ConfigError(ValueError):
    pass


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: type
    build: object  # callable(config, dtype, device) -> Model


_REGISTRY = {}


def register_architecture(names, config_cls, build):
    """Register `build(config, ...)` and `config_cls.from_dict` under each name."""
    if isinstance(names, str):
        names = [names]
    arch = Architecture(names[0], config_cls, build)
    for name in names:
        if name in _REGISTRY:
            raise ConfigError(f"architecture {name!r} is already registered")
        _REGISTRY[name] = arch
    return arch


def unregister_architecture(name):
    _REGISTRY.pop(name, None)


def registered_architectures():
    return sorted(_REGISTRY)


def architecture_of(raw):
    """The registry entry for a config.json dict."""
    candidates = list(raw.get("architectures") or []) + [raw.get("model_type")]
    for name in candidates:
        if name in _REGISTRY:
            return _REGISTRY[name]
    raise ConfigError(f"no registered architecture among {candidates}; known: {registered_architectures()}")


def read_config_json(folder):
    path = Path(folder) / "config.json"
    if not path.exists():
        raise ConfigError(f"{path} not found")
    return json.loads(path.read_text())


def config_from_folder(folder):
    raw = read_config_json(folder)
    arch = architecture_of(raw)
    return arch, arch.config_cls.from_dict(raw)
