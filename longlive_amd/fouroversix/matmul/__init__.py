from .frontend import fp4_matmul
from . import frontend  # noqa: F401

__all__ = ["fp4_matmul"]
