"""One registry from an architecture's name to how its model is made.

The reference matches the checkpoint's architecture string against the one it
supports and reports anything else as unsupported (rocml/src/model.rs:30-46,
rocml/src/error.rs:21).  Here the string is ``architectures[0]`` of config.json
and the table can hold more than one entry; an unknown name lists the known ones.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict

from ..errors import ConfigError, UnsupportedArchitectureError
from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    """What the library needs to know about one architecture.

    ``read_config`` turns config.json's dictionary into the typed configuration;
    ``to_spec`` turns that into parts; ``checkpoint_names`` maps the library's
    parameter names to the checkpoint's tensor names."""
    name: str
    read_config: Callable[[Dict], Any]
    to_spec: Callable[[Any], ModelSpec]
    checkpoint_names: Callable[[ModelSpec], Dict[str, str]]


_ARCHITECTURES: Dict[str, Architecture] = {}
_plugins_loaded = False

PLUGINS_ENV = "ROCML_AMD_PLUGINS"


def load_plugins() -> None:
    """Imports the modules named in the environment variable ``ROCML_AMD_PLUGINS`` (separated by
    commas), once.  A module that brings another architecture, parts or catalog entries registers
    them when it is imported; this is how the command line and the replay program, which build
    their model from config.json alone, learn of it without a change to this package."""
    global _plugins_loaded
    if _plugins_loaded:
        return
    _plugins_loaded = True
    import importlib
    for name in os.environ.get(PLUGINS_ENV, "").split(","):
        name = name.strip()
        if not name:
            continue
        try:
            importlib.import_module(name)
        except ImportError as e:
            raise ConfigError(f"{PLUGINS_ENV} names the module {name!r}, which cannot be imported: {e}") from e


def register_architecture(arch: Architecture) -> None:
    _ARCHITECTURES[arch.name] = arch


def known_architectures():
    load_plugins()
    return sorted(_ARCHITECTURES)


def architecture(name: str) -> Architecture:
    load_plugins()
    if name not in _ARCHITECTURES:
        raise UnsupportedArchitectureError(
            f"architecture {name!r} is not registered; known: {', '.join(known_architectures())}")
    return _ARCHITECTURES[name]


def read_config_json(path: str) -> Dict:
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json at {path}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            return json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from e


def architecture_of(raw: Dict) -> Architecture:
    archs = raw.get("architectures")
    if not isinstance(archs, (list, tuple)) or not archs:
        raise ConfigError("config.json lacks the key 'architectures'")
    return architecture(archs[0])


def _register_builtin() -> None:
    from . import qwen3
    register_architecture(Architecture(
        name=qwen3.ARCHITECTURE,
        read_config=qwen3.Qwen3Config.from_dict,
        to_spec=lambda cfg: cfg.to_model_spec(),
        checkpoint_names=qwen3.checkpoint_names))


_register_builtin()
