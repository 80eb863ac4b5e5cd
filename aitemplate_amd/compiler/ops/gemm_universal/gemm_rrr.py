"""gemm_rrr: A[M.., K] row-major  x  B[K, N] row-major  ->  C[M.., N]  (torch.mm(A, B)).

Counterpart of python/aitemplate/compiler/ops/gemm_universal/gemm_rrr.py:27-110."""
from ...base import IntImm, Tensor
from . import gemm_common as common


class gemm_rrr(common.gemm):
    def __init__(self):
        super().__init__()
        self._attrs["op"] = "gemm_rrr"

        def cal_align_ab(m, n, k):
            return common.default_align_ab(k, n, self._attrs["inputs"][0].dtype())

        self._attrs["f_ab_alignment"] = cal_align_ab

    def _infer_shapes(self, a: Tensor, b: Tensor):
        return a._attrs["shape"][:-1] + [b._attrs["shape"][1]]

    def _extract_dims(self, for_profiling: bool = False):
        a_rank = 2 if for_profiling else len(self._attrs["input_accessors"][0].original_shapes)
        lead = list(range(a_rank - 1))
        return {
            "M": [common.DimInfo(common.Source.INPUT, tensor_idx=0, dim_idx=lead),
                  common.DimInfo(common.Source.OUTPUT, tensor_idx=0, dim_idx=lead)],
            "N": [common.DimInfo(common.Source.INPUT, tensor_idx=1, dim_idx=1),
                  common.DimInfo(common.Source.OUTPUT, tensor_idx=0, dim_idx=a_rank - 1)],
            "K": [common.DimInfo(common.Source.INPUT, tensor_idx=0, dim_idx=a_rank - 1),
                  common.DimInfo(common.Source.INPUT, tensor_idx=1, dim_idx=0)],
        }

    def _align_ab(self, a: Tensor, b: Tensor):
        a_shape, b_shape = a._attrs["shape"], b._attrs["shape"]
        if a_shape[-1] != b_shape[0]:
            raise RuntimeError(f"A/B shape mismatch! A: {a_shape}, B: {b_shape}")
        if not isinstance(a_shape[-1], IntImm):
            raise RuntimeError(f"K must be static! k: {a_shape[-1]}")
        return a, b
