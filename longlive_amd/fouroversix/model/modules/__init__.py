from .linear import FourOverSixLinear
from . import linear  # noqa: F401

__all__ = ["FourOverSixLinear"]
