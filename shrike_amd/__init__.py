"""shrike_amd: a small inference engine for the Qwen2.5 dense decoder on one
MI355X (gfx950), with hand-written HIP kernels."""

__version__ = "0.1.0"
