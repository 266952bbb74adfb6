"""One registry from an architecture's name (config.json "architectures"[0]) to
its configuration class; the configuration's ``plan()`` is its model recipe.

The reference imports its model class directly (model/inference_paged.py:47) and
picks engines from a dict (model/server.py:79-85); here the model folder's own
config.json decides, everywhere in the framework.
"""

from __future__ import annotations

import json
from pathlib import Path

from .qwen3 import ConfigError, Qwen3Config

_ARCHITECTURES = {}


def register_architecture(name: str, config_cls) -> None:
    """``config_cls`` needs ``from_dict(dict)``, ``to_dict()`` and ``plan() -> ModelPlan``."""
    _ARCHITECTURES[name] = config_cls


def known_architectures():
    return sorted(_ARCHITECTURES)


_plugins_loaded = False


def _load_plugins() -> None:
    """Import the modules that SOCRATES_AMD_PLUGINS names, once."""
    global _plugins_loaded
    if _plugins_loaded:
        return
    _plugins_loaded = True
    import importlib
    import os
    for module in filter(None, (m.strip() for m in os.environ.get("SOCRATES_AMD_PLUGINS", "").split(","))):
        try:
            importlib.import_module(module)
        except ImportError as e:
            raise ConfigError(f"SOCRATES_AMD_PLUGINS names {module!r}, which cannot be imported: {e}") from e


def config_class_for(name: str):
    if name not in _ARCHITECTURES:
        _load_plugins()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f"unknown architecture {name!r}; known: {known_architectures()}") from None


def load_config(folder):
    """Read ``folder/config.json`` and return the typed configuration it names."""
    path = Path(folder) / "config.json"
    if not path.is_file():
        raise ConfigError(f"{path} not found")
    raw = json.loads(path.read_text())
    archs = raw.get("architectures")
    if not archs:
        raise ConfigError(f"{path} has no 'architectures' entry; known: {known_architectures()}")
    return config_class_for(archs[0]).from_dict(raw)


_PRESETS = Path(__file__).resolve().parent / "presets"


def known_presets():
    """Names of the configuration files that come with the package (``presets/*.json``):
    the two tiny test shapes and Qwen3-4B, -8B and -32B sizes."""
    return sorted(p.stem for p in _PRESETS.glob("*.json"))


def preset_path(name: str) -> Path:
    path = _PRESETS / f"{name}.json"
    if not path.is_file():
        raise ConfigError(f"unknown preset {name!r}; known: {known_presets()}")
    return path


def load_preset(name: str):
    """The typed configuration of a preset; which class reads it is decided by its own
    ``architectures`` entry, as for a model folder."""
    raw = json.loads(preset_path(name).read_text())
    return config_class_for(raw["architectures"][0]).from_dict(raw)


register_architecture("Qwen3ForCausalLM", Qwen3Config)
