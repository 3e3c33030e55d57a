"""Reads a model folder's safetensors files and binds every tensor the model
declares, by name.

Reference: shrike/models/qwen.py:202-214 reads every *.safetensors file of the
folder in sorted order, casts everything to the model dtype and binds by exact
name with a strict check.  Here the check comes first and reports everything
that is wrong at once.
"""

from __future__ import annotations

from pathlib import Path

import torch
from safetensors import safe_open

from ..parts.base import ParamSpec


class WeightError(RuntimeError):
    """The weight files do not hold what the model declares."""

    def __init__(self, message, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def shard_files(model_dir: str | Path) -> list[Path]:
    shards = sorted(Path(model_dir).glob("*.safetensors"))
    if not shards:
        raise FileNotFoundError(
            f"no *.safetensors file under {str(model_dir)!r}; a model folder holds config.json "
            "and model.safetensors"
        )
    return shards


def _index(shards: list[Path]) -> dict[str, tuple[Path, tuple[int, ...]]]:
    """name -> (file, shape) from the headers alone; a later file overrides an earlier one."""
    found: dict[str, tuple[Path, tuple[int, ...]]] = {}
    for shard in shards:
        with safe_open(str(shard), framework="pt") as f:
            for name in f.keys():
                found[name] = (shard, tuple(f.get_slice(name).get_shape()))
    return found


def check_names(found: dict, params: list[ParamSpec]) -> None:
    expected = {p.name: p for p in params}
    missing = sorted(n for n, p in expected.items() if n not in found and not p.optional)
    unexpected = sorted(n for n in found if n not in expected)
    wrong = sorted(
        (n, found[n][1], tuple(p.shape))
        for n, p in expected.items()
        if n in found and tuple(found[n][1]) != tuple(p.shape)
    )
    if not (missing or unexpected or wrong):
        return
    lines = ["the weight files do not match the model that config.json describes:"]
    if missing:
        lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(
            f"  wrong shape ({len(wrong)}): "
            + ", ".join(f"{n} is {list(got)}, expected {list(want)}" for n, got, want in wrong)
        )
    raise WeightError("\n".join(lines), missing, unexpected, wrong)


def convert(t: torch.Tensor, p: ParamSpec, dtype: torch.dtype) -> torch.Tensor:
    """Held dtype of a tensor: integer tables as int32; vectors that enter
    float32 arithmetic as float32 (a tensor stored in 32-bit stays so, one
    stored in bfloat16 widens exactly); everything else in the compute dtype."""
    if not t.dtype.is_floating_point:
        return t.to(torch.int32)
    return t.to(torch.float32 if p.keep_float32 else dtype)


def load_weights(model_dir, params: list[ParamSpec], dtype: torch.dtype, device) -> dict:
    """name -> device tensor for every declared tensor that the files hold."""
    shards = shard_files(model_dir)
    found = _index(shards)
    check_names(found, params)
    out: dict[str, torch.Tensor] = {}
    by_file: dict[Path, list[ParamSpec]] = {}
    for p in params:
        if p.name in found:
            by_file.setdefault(found[p.name][0], []).append(p)
    for shard, plist in by_file.items():
        with safe_open(str(shard), framework="pt") as f:
            for p in plist:
                out[p.name] = convert(f.get_tensor(p.name).to(device), p, dtype).contiguous()
    return out
