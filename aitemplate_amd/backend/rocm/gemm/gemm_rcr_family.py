"""Registry hooks of gemm_rcr and all of its bias / activation / residual variants.

One set of functions serves the whole family because the op name alone selects the
epilogue of the prebuilt kernels.  Replaces the per-op modules
python/aitemplate/backend/rocm/gemm/gemm_rcr*.py (e.g. gemm_rcr_bias.py:29-164,
gemm_rcr_bias_add.py:28-200, gemm_rcr_bias_fast_gelu.py:29-152), including the
reference's aliasing of gemm_rcr_bias_gelu to the fast (tanh) form."""
from ... import registry
from . import common

GEMM_RCR_OPS = [
    "gemm_rcr", "gemm_rcr_bias", "gemm_rcr_bias_relu", "gemm_rcr_bias_gelu", "gemm_rcr_bias_fast_gelu",
    "gemm_rcr_bias_sigmoid", "gemm_rcr_bias_tanh", "gemm_rcr_bias_swish", "gemm_rcr_bias_hardswish",
    "gemm_rcr_bias_add", "gemm_rcr_bias_add_add", "gemm_rcr_bias_add_relu", "gemm_rcr_bias_add_add_relu",
    "gemm_rcr_bias_mul", "gemm_rcr_bias_mul_add", "gemm_rcr_bias_sigmoid_mul", "gemm_rcr_bias_sigmoid_mul_tanh",
    "gemm_rcr_bias_mul_tanh",
]


def _register(op: str) -> None:
    registry.reg(f"rocm.{op}.config", lambda func_attrs, dtype="float16": common.gemm_config(func_attrs, dtype, "gemm"))
    registry.reg(f"rocm.{op}.filter", common.gemm_filter)
    registry.reg(f"rocm.{op}.gen_profiler", common.gemm_gen_profiler)
    registry.reg(f"rocm.{op}.select_algo", common.gemm_select_algo)
    registry.reg(f"rocm.{op}.gen_function", common.gemm_gen_function)
    registry.reg(f"rocm.{op}.func_decl", common.gemm_func_decl)
    registry.reg(f"rocm.{op}.func_call", common.gemm_func_call)


for _op in GEMM_RCR_OPS:
    _register(_op)
