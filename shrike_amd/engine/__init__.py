from .request import Request, SamplingParams, Status

__all__ = ["Request", "SamplingParams", "Status"]
