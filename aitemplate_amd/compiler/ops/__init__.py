from .common.elementwise import elementwise  # noqa: F401
from .common.epilogue import FuncEnum  # noqa: F401
from .common.view_ops import concatenate, flatten, reshape, split  # noqa: F401
from .gemm_universal import *  # noqa: F401,F403
from .attention import mem_eff_attention  # noqa: F401
