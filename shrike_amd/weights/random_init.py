"""Random weights from a configuration and a seed: as tensors for a model, or
written out as a model folder (config.json, model.safetensors) that the
ordinary loader reads back.

Matrices and biases are N(0, 0.02), norm weights 1 + N(0, 0.1).  Every tensor
has a generator of its own, seeded from the seed and the tensor's name, so a
tensor's values do not depend on which other tensors exist.
"""

from __future__ import annotations

import argparse
import hashlib
import json
from pathlib import Path

import torch
from safetensors.torch import save_file

from ..parts.base import ParamSpec

_STD = {"matrix": 0.02, "embedding": 0.02, "bias": 0.02, "norm": 0.1}

#: "reference": the distributions above.  "unit": matrices N(0, 1/fan_in) (the
#: embedding table N(0, 1)), biases N(0, 0.1): every part's output is as large
#: as its input, so attention scores spread and each layer moves the logits.
INIT_MODES = ("reference", "unit")


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(p: ParamSpec, seed: int, dtype: torch.dtype, device="cpu",
                  mode: str = "reference") -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, p.name))
    try:
        std = _STD[p.init]
    except KeyError:
        raise ValueError(f"{p.name}: unknown init {p.init!r}") from None
    if mode == "unit":
        if p.init == "matrix":
            std = float(p.shape[-1]) ** -0.5
        elif p.init == "embedding":
            std = 1.0
        elif p.init == "bias":
            std = 0.1
    elif mode != "reference":
        raise ValueError(f"init mode must be one of {INIT_MODES}, got {mode!r}")
    t = torch.empty(p.shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen)
    if p.init == "norm":
        t += 1.0
    return t.to(dtype)


def random_tensors(params: list[ParamSpec], seed: int, dtype: torch.dtype, device="cpu",
                   skip_optional: bool = True, mode: str = "reference") -> dict[str, torch.Tensor]:
    """Every declared tensor, drawn on `device` (large models: draw on the GPU)."""
    out = {}
    for p in params:
        if p.optional and skip_optional:
            continue
        t = random_tensor(p, seed, torch.float32 if p.keep_float32 else dtype, device, mode)
        out[p.name] = t
    return out


def write_model_folder(config: dict, path, seed: int = 0, dtype: str | None = None,
                       mode: str = "reference") -> Path:
    """Writes config.json and model.safetensors for the architecture that
    `config` (the content of a config.json) names.  `dtype` overrides the
    stored dtype (config["torch_dtype"])."""
    from ..config.registry import architecture_name, get_architecture
    from ..models import DecoderModel

    config = dict(config)
    if dtype is not None:
        config["torch_dtype"] = dtype
    arch = get_architecture(architecture_name(config))
    cfg = arch.config_cls.from_dict(config)
    spec = arch.build_spec(cfg)
    model = DecoderModel(spec)
    stored = getattr(torch, spec.stored_dtype)
    tensors = {}
    for p in model.params():
        if p.optional:
            continue
        tensors[p.name] = random_tensor(p, seed, stored, mode=mode).contiguous()
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(config, indent=2) + "\n")
    save_file(tensors, str(path / "model.safetensors"))
    return path


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(
        description="Write a model folder with random weights from a config.json"
    )
    ap.add_argument("--config", required=True, help="a config.json (file) to take the sizes from")
    ap.add_argument("--out", required=True, help="folder to write")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default=None)
    ap.add_argument("--init", choices=INIT_MODES, default="reference")
    args = ap.parse_args(argv)
    config = json.loads(Path(args.config).read_text())
    print(write_model_folder(config, args.out, args.seed, args.dtype, args.init))


if __name__ == "__main__":
    main()
