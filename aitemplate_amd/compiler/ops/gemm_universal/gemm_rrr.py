"""gemm_rrr: A[M.., K] row-major  x  B[K, N] row-major  ->  C[M.., N]  (torch.mm(A, B)), and the bias +
permuted-store form the ROCm backend has for it.

Counterparts: python/aitemplate/compiler/ops/gemm_universal/gemm_rrr.py:27-110, gemm_rrr_bias.py,
gemm_rrr_bias_permute.py:27-75."""
from typing import Tuple

from ...base import IntImm, Tensor
from ...tensor_accessor import TensorAccessor
from ..common.view_ops import reshape
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


class gemm_rrr_bias(gemm_rrr):
    """torch.mm(A, B) + bias.  Only its permuting subclass has ROCm kernels; this class carries the shape rules."""

    def __init__(self):
        super().__init__()
        self._attrs["op"] = "gemm_rrr_bias"

    @staticmethod
    def is_valid_inputs(a: Tensor, b: Tensor, bias: Tensor):
        bias_shapes = bias._attrs["shape"]
        if len(bias_shapes) != 1 or not isinstance(bias_shapes[0], IntImm):
            return False, f"Bias should be a fixed 1D vector! Current bias shape: {bias_shapes}"
        if b._attrs["shape"][1] != bias_shapes[0]:
            return False, f"GEMM/Bias shape doesn't match! B: {b._attrs['shape']}, bias shape: {bias_shapes[0]}"
        return True, ""

    def __call__(self, a: Tensor, b: Tensor, bias: Tensor) -> Tensor:
        a, b = self._align_ab(a, b)
        ok, msg = self.is_valid_inputs(a, b, bias)
        if not ok:
            raise RuntimeError(msg)
        self._attrs["inputs"] = [a, b, bias]
        self._attrs["input_accessors"] = [TensorAccessor(t) for t in self._attrs["inputs"]]
        self._set_depth()
        self._sanity_check(a, b)
        return self._finish_call([a, b, bias], self._infer_shapes(a, b))


class gemm_rrr_bias_permute(gemm_rrr_bias):
    """permute((A @ B + bias).reshape(M / (t1 t2), t1, t2, t3, N / t3), (2, 0, 3, 1, 4)) with shape = (t1, t2, t3):
    layout "20314" in the form the ROCm backend gives it (gemm_rrr_bias_permute.py:58-66)."""

    def __init__(self, shape: Tuple[int], layout="20314"):
        super().__init__()
        if layout != "20314":
            raise NotImplementedError("{} is not implemented!".format(layout))
        if len(shape) != 3:
            raise RuntimeError(f"shape must have 3 entries, got {shape}")
        self._attrs["op"] = "gemm_rrr_bias_permute"
        self._attrs["shape"] = tuple(int(t) for t in shape)
        self._attrs["layout"] = "Permute5D_{}".format(layout)
        self._attrs["permute_shape"] = "_".join(map(str, shape))

    def _extract_dims(self, for_profiling: bool = False):
        from .gemm_rcr_permute import _flat_output_dims

        return _flat_output_dims(super()._extract_dims(for_profiling))

    def __call__(self, a: Tensor, b: Tensor, bias: Tensor) -> Tensor:
        from .gemm_rcr_permute import _permuted_shape, _static_mn

        a, b = self._align_ab(a, b)
        ok, msg = self.is_valid_inputs(a, b, bias)
        if not ok:
            raise RuntimeError(msg)
        self._attrs["inputs"] = [a, b, bias]
        self._attrs["input_accessors"] = [TensorAccessor(t) for t in self._attrs["inputs"]]
        self._set_depth()
        self._sanity_check(a, b)
        m, n = _static_mn(self._attrs["op"], self._infer_shapes(a, b))
        view_shape = _permuted_shape(self._attrs["op"], "m3n2", self._attrs["shape"], m, n)
        output = Tensor([IntImm(m), IntImm(n)], src_ops={self}, dtype=a.dtype())
        self._attrs["outputs"] = [output]
        self._attrs["output_accessors"] = [TensorAccessor(output)]
        self._extract_epilogue_alignment(view_shape)
        return reshape()(output, view_shape)

    def _get_op_attributes(self):
        return {"layout": self._attrs["layout"].split("_")[-1], "shape": self._attrs["shape"]}
