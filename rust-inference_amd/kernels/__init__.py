from . import ops
from .build import build, load

__all__ = ["ops", "build", "load"]
