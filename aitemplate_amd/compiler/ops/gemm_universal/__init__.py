from .bmm import (  # noqa: F401
    bmm,
    bmm_ccr,
    bmm_ccr_add,
    bmm_crr,
    bmm_crr_add,
    bmm_rcr,
    bmm_rcr_permute,
    bmm_rrr,
    bmm_rrr_add,
    bmm_rrr_permute,
)
from .bmm_softmax_bmm import bmm_softmax_bmm  # noqa: F401
from .bmm_softmax_bmm_permute import bmm_softmax_bmm_permute  # noqa: F401
from .gemm_common import gemm  # noqa: F401
from .gemm_rcr import gemm_rcr  # noqa: F401
from .gemm_rrr import gemm_rrr, gemm_rrr_bias, gemm_rrr_bias_permute  # noqa: F401
from .gemm_rcr_bias import (  # noqa: F401
    gemm_rcr_bias,
    gemm_rcr_bias_fast_gelu,
    gemm_rcr_bias_gelu,
    gemm_rcr_bias_hardswish,
    gemm_rcr_bias_relu,
    gemm_rcr_bias_sigmoid,
    gemm_rcr_bias_swish,
    gemm_rcr_bias_tanh,
)
from .gemm_rcr_bias_broadcast import (  # noqa: F401
    gemm_rcr_bias_add,
    gemm_rcr_bias_add_add,
    gemm_rcr_bias_add_add_relu,
    gemm_rcr_bias_add_relu,
    gemm_rcr_bias_broadcast,
    gemm_rcr_bias_mul,
    gemm_rcr_bias_mul_add,
    gemm_rcr_bias_mul_tanh,
    gemm_rcr_bias_sigmoid_mul,
    gemm_rcr_bias_sigmoid_mul_tanh,
)
from .gemm_rcr_permute import gemm_rcr_bias_permute, gemm_rcr_permute  # noqa: F401
