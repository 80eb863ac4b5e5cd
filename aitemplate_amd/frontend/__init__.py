"""User-facing names (counterpart of python/aitemplate/frontend/__init__.py)."""
from ..compiler.base import DynamicProfileStrategy, IntImm, IntVar, Tensor  # noqa: F401
from . import nn  # noqa: F401
