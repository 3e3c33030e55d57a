"""One registry from an architecture's name (config.json ``architectures[0]``)
to its typed configuration and the function that turns it into a ModelSpec.

The reference keeps a table of repository ids that all map to "qwen2"
(shrike/config.py:21-25) and never dispatches on it; here the name in
config.json chooses the model everywhere (engine, replay, command line).
"""

from __future__ import annotations

import importlib
import json
import os
from dataclasses import dataclass
from pathlib import Path
from typing import Callable

from .specs import ModelSpec


class ConfigError(ValueError):
    """config.json is absent, names no known architecture, or holds a bad value."""


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: type
    build_spec: Callable[[object], ModelSpec]
    model_types: tuple[str, ...] = ()


_ARCHITECTURES: dict[str, Architecture] = {}
_MODEL_TYPES: dict[str, str] = {}

#: Default model folder of the command line, as the reference's
#: DEFAULT_MODEL_DIR with its SHRIKE_MODEL_DIR override (shrike/config.py:29).
DEFAULT_MODEL_DIR: str = os.environ.get("SHRIKE_MODEL_DIR", "models_cache/qwen2.5-0.5b-instruct")


def register_architecture(
    name: str, config_cls: type, build_spec: Callable, model_types: tuple[str, ...] = ()
) -> None:
    """``config_cls.from_dict(raw) -> cfg``; ``build_spec(cfg) -> ModelSpec``."""
    _ARCHITECTURES[name] = Architecture(name, config_cls, build_spec, tuple(model_types))
    for mt in model_types:
        _MODEL_TYPES[mt] = name


def architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


_plugins_loaded = False


def load_plugins() -> None:
    """Imports what the environment variable SHRIKE_AMD_PLUGINS names, once:
    comma-separated `module` or `module:function` entries.  A module registers
    its architectures and parts when it is imported, or when `function()` is
    called; that is how the command-line programs come to know an architecture
    that is not part of the package."""
    global _plugins_loaded
    if _plugins_loaded:
        return
    _plugins_loaded = True
    for entry in filter(None, (e.strip() for e in os.environ.get("SHRIKE_AMD_PLUGINS", "").split(","))):
        module_name, _, function = entry.partition(":")
        try:
            module = importlib.import_module(module_name)
            if function:
                getattr(module, function)()
        except Exception as e:
            raise ConfigError(f"SHRIKE_AMD_PLUGINS: cannot load {entry!r}: {type(e).__name__}: {e}") from e


def get_architecture(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        load_plugins()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(architectures()) or 'none'}"
        ) from None


def read_config_json(model_dir: str | Path) -> dict:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(
            f"no config.json under {str(model_dir)!r}; give a model folder with config.json and "
            "model.safetensors (python -m shrike_amd.weights.random_init writes one), "
            "or set SHRIKE_MODEL_DIR"
        )
    try:
        raw = json.loads(path.read_text())
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return raw


def architecture_name(raw: dict) -> str:
    archs = raw.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        return str(archs[0])
    mt = raw.get("model_type")
    if mt in _MODEL_TYPES:
        return _MODEL_TYPES[mt]
    raise ConfigError(
        "config.json names no architecture: expected \"architectures\": [name] "
        f"(registered: {', '.join(architectures())})"
    )


def load_model_config(model_dir: str | Path):
    """-> (typed config, ModelSpec) of the architecture that config.json names."""
    raw = read_config_json(model_dir)
    arch = get_architecture(architecture_name(raw))
    cfg = arch.config_cls.from_dict(raw)
    return cfg, arch.build_spec(cfg)
