"""Options of the engine, named as the reference's LLMEngine keyword arguments
(shrike/engine/engine.py:42-53) where it has them."""

from __future__ import annotations

from dataclasses import dataclass

_DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32"}


def canonical_dtype(name: str) -> str:
    try:
        return _DTYPES[str(name).replace("torch.", "")]
    except KeyError:
        raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}") from None


@dataclass
class EngineConfig:
    """block_size, gpu_mem_util, max_tokens_per_step, max_running and
    enable_prefix_caching mean what they mean in the reference.

    num_kv_blocks: pages of every cache group; None sizes the pool from free
        device memory times gpu_mem_util (shrike/engine/model_runner.py:165-174).
    dtype: "bfloat16" (serving kernels) or "float32" (every kernel in true
        32-bit arithmetic); None takes the dtype the model folder was stored in.
    graphs: replay decode-only steps from HIP graphs.
    overlap_steps: launch the next decode step before the host has read the
        tokens of this one (they pass from the sampler to the next step on the
        device); a request that turns out to have ended is dropped from that
        step's results.
    """

    block_size: int = 16
    gpu_mem_util: float = 0.85
    max_tokens_per_step: int = 512
    max_running: int = 256
    enable_prefix_caching: bool = True
    num_kv_blocks: int | None = None
    dtype: str | None = None
    seed: int = 0
    graphs: bool = True
    overlap_steps: bool = True
    device: str = "cuda:0"

    def __post_init__(self):
        if self.block_size < 1:
            raise ValueError(f"block_size must be >= 1, got {self.block_size}")
        if not 0.0 < self.gpu_mem_util <= 1.0:
            raise ValueError(f"gpu_mem_util must be in (0, 1], got {self.gpu_mem_util}")
        if self.max_tokens_per_step < 1:
            raise ValueError(f"max_tokens_per_step must be >= 1, got {self.max_tokens_per_step}")
        if self.max_running < 1:
            raise ValueError(f"max_running must be >= 1, got {self.max_running}")
        if self.num_kv_blocks is not None and self.num_kv_blocks < 1:
            raise ValueError(f"num_kv_blocks must be >= 1, got {self.num_kv_blocks}")
        if self.dtype is not None:
            self.dtype = canonical_dtype(self.dtype)
