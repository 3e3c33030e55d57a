"""From a model folder (or a spec and a seed) to a model that is ready to step."""

from __future__ import annotations

import torch

from ..config.registry import load_model_config
from ..config.specs import ModelSpec
from ..models import DecoderModel
from ..weights import load_weights, random_tensors
from .runtime import Runtime

_TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def require_gpu(device) -> None:
    if not torch.cuda.is_available():
        raise RuntimeError(
            "no GPU is visible: shrike_amd runs its HIP kernels on an MI355X (gfx950) and has no "
            "CPU path"
        )
    name = torch.cuda.get_device_properties(torch.device(device)).gcnArchName
    if not name.startswith("gfx950"):
        raise RuntimeError(f"the kernels are built for gfx950, but {device} is {name}")


def load_model(model_dir, dtype: str | None = None, device="cuda:0"):
    """-> (model, runtime, typed config).  `dtype` None takes the stored dtype."""
    require_gpu(device)
    cfg, spec = load_model_config(model_dir)
    runtime = Runtime(device, _TORCH_DTYPES[dtype or spec.stored_dtype])
    model = DecoderModel(spec)
    tensors = load_weights(model_dir, model.params(), runtime.dtype, runtime.device)
    model.load(tensors, runtime)
    return model, runtime, cfg


def random_model(spec: ModelSpec, seed: int = 0, dtype: str = "bfloat16", device="cuda:0"):
    """A model with random weights drawn on the device (no files involved)."""
    require_gpu(device)
    runtime = Runtime(device, _TORCH_DTYPES[dtype])
    model = DecoderModel(spec)
    tensors = random_tensors(model.params(), seed, runtime.dtype, runtime.device)
    model.load(tensors, runtime)
    return model, runtime
