"""bmm_softmax_bmm_permute: softmax(scale * Q K^T) V with the result permuted to [B/G, M, G, O].

Equivalent PyTorch:
    attn  = torch.softmax(torch.bmm(Q, K.transpose(1, 2)) * scale, dim=-1)
    score = torch.bmm(attn, V).reshape(B // num_heads, num_heads, M, O).permute(0, 2, 1, 3)
Counterpart of python/aitemplate/compiler/ops/gemm_universal/bmm_softmax_bmm_permute.py:30-194."""
from typing import Tuple

from ...base import IntImm, Tensor
from ...tensor_accessor import TensorAccessor
from ..common.view_ops import reshape
from . import gemm_common as common
from .bmm import bmm


class bmm_softmax_bmm_permute(bmm):
    def __init__(self, shape: Tuple[int], scale=1.0, causal=False, layout="0213"):
        """shape: (num_heads,); scale: factor applied to Q K^T; causal: mask keys after the query."""
        super().__init__()
        self._attrs["op"] = "bmm_softmax_bmm_permute" + ("_causal" if causal else "")
        self._attrs["scale"] = scale
        self._attrs["shape"] = shape
        self._attrs["layout"] = f"Permute4DBMM_{layout}"

        def cal_align_ab(m, n, k):
            return common.default_align_ab(k, k, self._attrs["inputs"][0].dtype())

        self._attrs["f_ab_alignment"] = cal_align_ab

    def _infer_shapes(self, a: Tensor, b: Tensor, b1: Tensor):
        a_shapes, b_shapes, b1_shapes = a._attrs["shape"], b._attrs["shape"], b1._attrs["shape"]
        if a_shapes[0] != b_shapes[0] and a_shapes[0] != 1 and b_shapes[0] != 1:
            raise RuntimeError(
                "bmm_rcr operand A and B should have same batch_size, or batch_size = 1! "
                f"Current shape A: {a_shapes} shape B: {b_shapes} .")
        batch = b_shapes[0] if a_shapes[0] == IntImm(1) else a_shapes[0]
        assert a_shapes[2] == b_shapes[2], (
            f"bmm_rcr operand A and B should have the same K dim (dim2)! Current shape A: {a_shapes}, "
            f"shape B: {b_shapes}")
        return [batch, a_shapes[1], b1_shapes[2]]

    def _extract_dims(self, for_profiling: bool = False):
        S = common.Source
        return {
            "B": [common.DimInfo(S.INPUT, 0, 0), common.DimInfo(S.INPUT, 1, 0), common.DimInfo(S.OUTPUT, 0, 0)],
            "M": [common.DimInfo(S.INPUT, 0, 1), common.DimInfo(S.OUTPUT, 0, 1)],
            "N": [common.DimInfo(S.INPUT, 1, 1)],
            "K": [common.DimInfo(S.INPUT, 0, 2), common.DimInfo(S.INPUT, 1, 2)],
            "O": [common.DimInfo(S.OUTPUT, 0, 2)],
        }

    def _get_ab_alignment(self, exec_key):
        k = self._invert_exec_key(exec_key)[3]
        return self._attrs["f_ab_alignment"](0, 0, k)

    def _sanity_check(self, a: Tensor, b: Tensor):
        super()._sanity_check(a, b)
        if len(a._attrs["shape"]) != 3 or len(b._attrs["shape"]) != 3:
            raise RuntimeError("bmm_softmax_bmm_permute operands must be 3-D")

    def __call__(self, a: Tensor, b: Tensor, b1: Tensor) -> Tensor:
        """a: [B, M, K], b: [B, N, K], b1: [B, N, O]  ->  [B / heads, M, heads, O]"""
        a, b = self._align_ab(a, b)
        self._attrs["inputs"] = [a, b, b1]
        self._attrs["input_accessors"] = [TensorAccessor(a), TensorAccessor(b), TensorAccessor(b1)]
        self._set_depth()
        self._sanity_check(a, b)
        output_shape = self._infer_shapes(a, b, b1)
        output = Tensor(output_shape, src_ops={self}, dtype=a.dtype())
        self._attrs["outputs"] = [output]
        self._attrs["output_accessors"] = [TensorAccessor(output)]
        if self._attrs["layout"] != "Permute4DBMM_0213":
            raise NotImplementedError("{} is not implemented!".format(self._attrs["layout"]))
        batch, m, o = output_shape
        heads = self._attrs["shape"][0]
        permuted = [batch.value() // heads, m, heads, o]
        self._extract_epilogue_alignment(permuted)
        # the kernel already writes [B/G, M, G, O]; the reshape is a pure view of its buffer
        return reshape()(output, permuted)

    def _get_op_attributes(self):
        return {
            "causal": self._attrs["op"] == "bmm_softmax_bmm_permute_causal",
            "layout": self._attrs["layout"].split("_")[-1],
            "scale": self._attrs["scale"],
            "shape": self._attrs["shape"],
        }
