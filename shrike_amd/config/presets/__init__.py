"""config.json files of published sizes of the architectures this package runs, as
data: for runs with random weights where no model folder is at hand
(`python -m shrike_amd --random-config qwen2.5-7b`, bench.py)."""

from __future__ import annotations

import json
from pathlib import Path

_HERE = Path(__file__).resolve().parent


def preset_names() -> list[str]:
    return sorted(p.stem for p in _HERE.glob("*.json"))


def load_preset(name: str) -> dict:
    """The config.json of the preset `name` (case-insensitive), as a dict."""
    path = _HERE / f"{name.lower()}.json"
    if not path.is_file():
        raise KeyError(f"no preset {name!r}; there are: {', '.join(preset_names())}")
    with open(path) as f:
        return json.load(f)
