from . import ops
from .build import build as build_library, load as load_library

__all__ = ["ops", "build_library", "load_library"]
