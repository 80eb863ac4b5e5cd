from .attention import CrossAttention, ScaledDotProductAttention, MultiheadAttention  # noqa: F401
from .dropout import Dropout, DropPath  # noqa: F401
from .linear import Linear  # noqa: F401
from .module import Module  # noqa: F401
from .parameter import Parameter  # noqa: F401
