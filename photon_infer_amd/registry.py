"""The one registry from an architecture's name to its configuration and model.

The reference constructs ``LLaMAModel`` directly (demo/llama_infer.cpp:209) and has no
registry; here ``config.json``'s ``architectures[0]`` selects an entry everywhere a
model folder is opened (engine, command line, trace replay, random-weights writer).

An entry provides
  * ``config_cls.from_dict(raw) -> config``  (typed, validated),
  * ``build(config) -> ModelSpec``           (the layer list and run order; no tensors),
which is all that the loader, the cache manager and the step function need.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict

from .config.base import architecture_name, read_config_json
from .errors import UnsupportedModelError


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Any
    build: Callable[[Any], Any]


_ARCHITECTURES: Dict[str, Architecture] = {}
_BUILTINS_LOADED = False


def register_architecture(name: str, config_cls: Any, build: Callable[[Any], Any]) -> Architecture:
    """Add (or replace) the entry for ``name``.  ``build(config)`` returns a ModelSpec."""
    entry = Architecture(name, config_cls, build)
    _ARCHITECTURES[name] = entry
    return entry


def _load_builtins() -> None:
    global _BUILTINS_LOADED
    if not _BUILTINS_LOADED:
        _BUILTINS_LOADED = True
        from . import models  # noqa: F401  (registers on import)


def get_architecture(name: str) -> Architecture:
    _load_builtins()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        known = ", ".join(sorted(_ARCHITECTURES)) or "<none>"
        raise UnsupportedModelError(
            f"architecture '{name}' is not registered (registered: {known})"
        ) from None


def registered_architectures() -> tuple:
    _load_builtins()
    return tuple(sorted(_ARCHITECTURES))


def config_from_dict(raw: dict, where: str = "config.json"):
    arch = get_architecture(architecture_name(raw, where))
    return arch.config_cls.from_dict(raw, where)


def load_config(model_dir: str):
    """Read ``model_dir/config.json`` into the typed config of its architecture."""
    raw = read_config_json(model_dir)
    return config_from_dict(raw, f"{model_dir}/config.json")


def build_model_spec(config):
    return get_architecture(config.architecture).build(config)
