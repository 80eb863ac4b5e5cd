"""bmm_softmax_bmm: softmax(scale * Q K^T) V, result [B, M, O].

Equivalent PyTorch:
    attn  = torch.softmax(torch.bmm(Q, K.transpose(1, 2)) * scale, dim=-1)
    score = torch.bmm(attn, V)
Counterpart of python/aitemplate/compiler/ops/gemm_universal/bmm_softmax_bmm.py:27-150.  Runs the
fused attention kernel of bmm_softmax_bmm_permute with one head per batch entry, for which the
permuted layout [B / 1, M, 1, O] is the plain one."""
from ...base import Tensor
from ...tensor_accessor import TensorAccessor
from .bmm_softmax_bmm_permute import bmm_softmax_bmm_permute


class bmm_softmax_bmm(bmm_softmax_bmm_permute):
    def __init__(self, scale=1.0):
        super().__init__(shape=(1,), scale=scale, causal=False)
        self._attrs["op"] = "bmm_softmax_bmm"

    def __call__(self, a: Tensor, b: Tensor, b1: Tensor) -> Tensor:
        """a: [B, M, K], b: [B, N, K], b1: [B, N, O]  ->  [B, M, O]"""
        a, b = self._align_ab(a, b)
        self._attrs["inputs"] = [a, b, b1]
        self._attrs["input_accessors"] = [TensorAccessor(a), TensorAccessor(b), TensorAccessor(b1)]
        self._set_depth()
        self._sanity_check(a, b)
        output_shape = self._infer_shapes(a, b, b1)
        self._extract_epilogue_alignment(output_shape)
        output = Tensor(output_shape, src_ops={self}, dtype=a.dtype())
        self._attrs["outputs"] = [output]
        self._attrs["output_accessors"] = [TensorAccessor(output)]
        return output

    def _get_op_attributes(self):
        return {"scale": self._attrs["scale"]}
