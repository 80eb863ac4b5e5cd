"""Graph IR, ops, passes, compile_model and the Model wrapper."""
from . import base, dtype, ops, tensor_accessor, transform  # noqa: F401
from .base import DynamicProfileStrategy  # noqa: F401
from .compiler import compile_model  # noqa: F401
from .model import AITData, AITemplateAllocatorKind, AITemplateMemcpyKind, Model  # noqa: F401
