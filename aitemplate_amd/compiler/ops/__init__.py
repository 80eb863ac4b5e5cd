from .common.view_ops import flatten, reshape, split  # noqa: F401
from .gemm_universal import *  # noqa: F401,F403
