"""ctypes binding of ``libaitemplate_amd_kernels.so`` (the gfx950 kernel library).

The library is built in-tree by ``make -C aitemplate_amd/csrc`` and loaded from
``aitemplate_amd/lib``.  There is no fallback: if the shared object is missing
every call raises, so a GPU run can never silently take another path.

The functions here are thin: they pass raw device pointers and sizes to the C
ABI declared in ``include/aitemplate_amd_kernels.h``.  ``torch`` is only used by
callers for device memory and streams.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import List, Optional

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
KERNEL_LIB_NAME = "libaitemplate_amd_kernels.so"
KERNEL_LIB_PATH = os.path.join(_LIB_DIR, KERNEL_LIB_NAME)

# Epilogue ids of the C ABI (include/aitemplate_amd_kernels.h); keyed by the
# reference op name so callers read like the reference's frontend.
EPILOGUE_OF_OP = {
    "gemm_rcr": 0,
    "bmm_rcr": 0,
    "gemm_rcr_bias": 1,
    "gemm_rcr_bias_relu": 2,
    "gemm_rcr_bias_gelu": 3,
    "gemm_rcr_bias_fast_gelu": 3,
    "gemm_rcr_bias_add": 4,
    "gemm_rcr_bias_add_add": 5,
    "gemm_rcr_bias_add_relu": 6,
    "gemm_rcr_bias_add_add_relu": 7,
    "gemm_rcr_bias_sigmoid": 8,
    "gemm_rcr_bias_tanh": 9,
    "gemm_rcr_bias_swish": 10,
    "gemm_rcr_bias_hardswish": 11,
    "gemm_rcr_bias_mul": 12,
    "gemm_rcr_bias_mul_add": 13,
    "gemm_rcr_bias_sigmoid_mul": 14,
    "gemm_rcr_bias_sigmoid_mul_tanh": 15,
    "gemm_rcr_bias_mul_tanh": 16,
}
NUM_RESIDUALS_OF_EPILOGUE = {0: 0, 1: 0, 2: 0, 3: 0, 4: 1, 5: 2, 6: 1, 7: 2, 8: 0, 9: 0,
                             10: 0, 11: 0, 12: 1, 13: 2, 14: 1, 15: 1, 16: 1, 17: 1}
EPI_ADD = 17  # residual without bias: the bmm_*_add ops
DTYPE_ID = {"float16": 0, "bfloat16": 1}

# Ops that store through a 5-D output permutation: name -> (epilogue id, layout id of aitamd_gemm_rcr_permute).
# On ROCm the reference lowers layout "20314" like "m3n2" (gemm_rcr_bias_permute.py:66-72 of
# python/aitemplate/compiler/ops/gemm_universal/).
PERMUTE_M2N3, PERMUTE_M3N2 = 1, 2
LAYOUT_ID = {"rcr": 0, "rrr": 1, "ccr": 2, "crr": 3}
# plain-epilogue ops launched through aitamd_bmm / aitamd_bmm_rcr_permute
LAYOUT_OPS = ("bmm_rcr_permute", "bmm_rrr", "bmm_rrr_permute", "bmm_ccr", "bmm_crr", "gemm_rrr",
              "bmm_rrr_add", "bmm_ccr_add", "bmm_crr_add")
PERMUTE_OPS = {
    "gemm_rcr_permute_m2n3": (0, PERMUTE_M2N3),
    "gemm_rcr_bias_permute_m2n3": (1, PERMUTE_M2N3),
    "gemm_rcr_bias_permute_m3n2": (1, PERMUTE_M3N2),
    "gemm_rcr_bias_permute": (1, PERMUTE_M3N2),
    "gemm_rrr_bias_permute": (1, PERMUTE_M3N2),  # B is [K, N]: operand layout rrr
}
PERMUTE_OPERANDS = {"gemm_rrr_bias_permute": "rrr"}  # every other permuting op is rcr

# Every symbol include/aitemplate_amd_kernels.h declares.
EXPORTED_SYMBOLS = [
    "aitamd_version",
    "aitamd_last_error",
    "aitamd_gemm_num_algos",
    "aitamd_gemm_algo_name",
    "aitamd_gemm_find_algo",
    "aitamd_gemm_algo_supported",
    "aitamd_gemm_heuristic_algo",
    "aitamd_gemm_rcr",
    "aitamd_gemm_rcr_permute",
    "aitamd_bmm_rcr_permute",
    "aitamd_bmm",
    "aitamd_bmm_add",
    "aitamd_gemm_permute",
    "aitamd_gemm_algo_supported_layout",
    "aitamd_gemm_heuristic_algo_layout",
    "aitamd_bmm_rcr",
    "aitamd_bmm_softmax_bmm_permute",
    "aitamd_mem_eff_attention",
    "aitamd_attention_set_variant",
    "aitamd_elementwise",
    "aitamd_elementwise_supported",
    "aitamd_copy_rows",
    "aitamd_gemm_workspace_bytes",
    "aitamd_gemm_rcr_ws",
    "aitamd_gemm_rcr_noalloc",
    "aitamd_gemm_noalloc_scratch_bytes",
]

_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None


class KernelLibraryMissing(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """dlopen the kernel library (once) and declare argument types."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(KERNEL_LIB_PATH):
            raise KernelLibraryMissing(
                f"{KERNEL_LIB_PATH} not found: build it with `make -C aitemplate_amd/csrc -j8` "
                "(or __graft_entry__.build()); there is no non-HIP fallback."
            )
        lib = ctypes.CDLL(KERNEL_LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        i64, i32, vp, cp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p
        lib.aitamd_version.restype = cp
        lib.aitamd_version.argtypes = []
        lib.aitamd_last_error.restype = cp
        lib.aitamd_last_error.argtypes = []
        lib.aitamd_gemm_num_algos.restype = i32
        lib.aitamd_gemm_num_algos.argtypes = [i32, i32]
        lib.aitamd_gemm_algo_name.restype = cp
        lib.aitamd_gemm_algo_name.argtypes = [i32, i32, i32]
        lib.aitamd_gemm_find_algo.restype = i32
        lib.aitamd_gemm_find_algo.argtypes = [i32, i32, cp]
        lib.aitamd_gemm_algo_supported.restype = i32
        lib.aitamd_gemm_algo_supported.argtypes = [i32, i32, i32, i64, i64, i64, i64, i64, i32]
        lib.aitamd_gemm_heuristic_algo.restype = i32
        lib.aitamd_gemm_heuristic_algo.argtypes = [i32, i32, i64, i64, i64, i64, i64, i64, i32]
        lib.aitamd_gemm_rcr.restype = i32
        lib.aitamd_gemm_rcr.argtypes = [i32, i32, i32, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp]
        lib.aitamd_gemm_rcr_permute.restype = i32
        lib.aitamd_gemm_rcr_permute.argtypes = [i32, i32, i32, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, i64, i64, i64, vp]
        lib.aitamd_bmm_rcr_permute.restype = i32
        lib.aitamd_bmm_rcr_permute.argtypes = [i32, i32, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, i64, vp]
        lib.aitamd_bmm.restype = i32
        lib.aitamd_bmm.argtypes = [i32, i32, i32, vp, vp, vp] + [i64] * 11 + [vp]
        lib.aitamd_bmm_add.restype = i32
        lib.aitamd_bmm_add.argtypes = [i32, i32, i32, vp, vp, vp, vp] + [i64] * 12 + [vp]
        lib.aitamd_gemm_permute.restype = i32
        lib.aitamd_gemm_permute.argtypes = [i32, i32, i32, i32, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, i64, i64, i64, vp]
        lib.aitamd_gemm_algo_supported_layout.restype = i32
        lib.aitamd_gemm_algo_supported_layout.argtypes = [i32, i32, i32, i32, i64, i64, i64, i64, i64, i32]
        lib.aitamd_gemm_heuristic_algo_layout.restype = i32
        lib.aitamd_gemm_heuristic_algo_layout.argtypes = [i32, i32, i32, i64, i64, i64, i64, i64, i64, i32]
        lib.aitamd_bmm_rcr.restype = i32
        lib.aitamd_bmm_rcr.argtypes = [i32, i32, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, vp]
        lib.aitamd_bmm_softmax_bmm_permute.restype = i32
        lib.aitamd_bmm_softmax_bmm_permute.argtypes = [i32, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64,
                                                       ctypes.c_float, i32, vp]
        lib.aitamd_mem_eff_attention.restype = i32
        lib.aitamd_mem_eff_attention.argtypes = [i32, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ctypes.c_float, i32,
                                                 vp, vp, vp]
        lib.aitamd_gemm_workspace_bytes.restype = i64
        lib.aitamd_gemm_workspace_bytes.argtypes = [i32, i32, i32, i64, i64, i64, i64]
        lib.aitamd_gemm_rcr_ws.restype = i32
        lib.aitamd_gemm_rcr_ws.argtypes = [i32, i32, i32, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp, i64, vp]
        lib.aitamd_gemm_rcr_noalloc.restype = i32
        lib.aitamd_gemm_rcr_noalloc.argtypes = [i32, i32, i32, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp]
        lib.aitamd_gemm_noalloc_scratch_bytes.restype = i64
        lib.aitamd_gemm_noalloc_scratch_bytes.argtypes = []
        lib.aitamd_attention_set_variant.restype = i32
        lib.aitamd_attention_set_variant.argtypes = [i32]
        lib.aitamd_elementwise.restype = i32
        lib.aitamd_elementwise.argtypes = [i32, i32, vp, vp, vp, i64, i64, ctypes.c_float, i32, vp]
        lib.aitamd_elementwise_supported.restype = i32
        lib.aitamd_elementwise_supported.argtypes = [i32]
        lib.aitamd_copy_rows.restype = i32
        lib.aitamd_copy_rows.argtypes = [vp, vp, i64, i64, i64, i64, vp]
        _lib = lib
        return lib


def last_error() -> str:
    return load().aitamd_last_error().decode()


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed: {last_error()}")


def gemm_algo_names(epilogue: int, dtype: int = 0) -> List[str]:
    lib = load()
    n = lib.aitamd_gemm_num_algos(epilogue, dtype)
    return [lib.aitamd_gemm_algo_name(epilogue, dtype, i).decode() for i in range(n)]
