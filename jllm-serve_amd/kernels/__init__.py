"""The HIP kernels' Python faces (``ops``) and the in-tree build of their library (``build``)."""
from . import build, ops

__all__ = ["build", "ops"]
