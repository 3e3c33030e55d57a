"""shrike_amd: a small inference engine for the Qwen2.5 dense decoder on one
MI355X (gfx950), with hand-written HIP kernels.

``SamplingParams`` is importable without torch being initialised on a GPU;
``LLM`` and ``LLMEngine`` are loaded on first use.
"""

from .engine.request import SamplingParams

__version__ = "0.1.0"

__all__ = ["LLM", "LLMEngine", "SamplingParams", "__version__"]


def __getattr__(name):
    if name in ("LLM", "LLMEngine"):
        from .engine import llm_engine

        return getattr(llm_engine, name)
    raise AttributeError(f"module 'shrike_amd' has no attribute {name!r}")
