from . import attention, elementwise, gemm  # noqa: F401  (registers the rocm.* hooks)
from .target_def import ROCM  # noqa: F401
