from . import ops
from .lib import KernelError, load

__all__ = ["KernelError", "load", "ops"]
