"""gemm_rcr_bias and its activation variants: epilogue(A @ B^T + bias).

Counterparts: gemm_rcr_bias.py:27-111, gemm_rcr_bias_relu.py:24-43, gemm_rcr_bias_gelu.py:24-43,
gemm_rcr_bias_fast_gelu.py, gemm_rcr_bias_sigmoid.py, gemm_rcr_bias_tanh.py, gemm_rcr_bias_swish.py,
gemm_rcr_bias_hardswish.py of python/aitemplate/compiler/ops/gemm_universal/."""
from ...base import IntImm, Tensor
from ...tensor_accessor import TensorAccessor
from .gemm_rcr import gemm_rcr


class gemm_rcr_bias(gemm_rcr):
    """y = torch.nn.functional.linear(A, B, bias=Bias)"""

    def __init__(self):
        super().__init__()
        self._attrs["op"] = "gemm_rcr_bias"

    @staticmethod
    def is_valid_inputs(X: Tensor, W: Tensor, bias: Tensor):
        bias_shapes = bias._attrs["shape"]
        if len(bias_shapes) != 1:
            return False, f"Bias should be 1D vector! Current bias shape: {bias_shapes}"
        if not isinstance(bias_shapes[0], IntImm):
            return False, f"Bias should be fixed 1D vector! Current bias shape: {bias_shapes[0]}"
        outshape = gemm_rcr()._infer_shapes(X, W)
        if outshape[-1] != bias_shapes[0]:
            return False, f"GEMM/Bias shape doesn't match! Gemm shape: {outshape}, bias shape: {bias_shapes[0]}"
        return True, ""

    def _infer_shapes(self, a: Tensor, b: Tensor, bias: Tensor):
        ok, msg = self.is_valid_inputs(a, b, bias)
        if not ok:
            raise RuntimeError(msg)
        return super()._infer_shapes(a, b)

    def __call__(self, a: Tensor, b: Tensor, bias: Tensor) -> Tensor:
        a, b = self._align_ab(a, b)
        self._attrs["inputs"] = [a, b, bias]
        self._attrs["input_accessors"] = [TensorAccessor(t) for t in self._attrs["inputs"]]
        self._set_depth()
        self._sanity_check(a, b)
        return self._finish_call([a, b, bias], self._infer_shapes(a, b, bias))


def _activation_variant(op_name: str, doc: str):
    def __init__(self):
        gemm_rcr_bias.__init__(self)
        self._attrs["op"] = op_name

    return type(op_name, (gemm_rcr_bias,), {"__init__": __init__, "__doc__": doc})


gemm_rcr_bias_relu = _activation_variant("gemm_rcr_bias_relu", "y = relu(linear(A, B, bias))")
gemm_rcr_bias_gelu = _activation_variant(
    "gemm_rcr_bias_gelu", "y = gelu(linear(A, B, bias)); the ROCm backend evaluates the tanh (fast) form")
gemm_rcr_bias_fast_gelu = _activation_variant(
    "gemm_rcr_bias_fast_gelu", "y = gelu(linear(A, B, bias), approximate='tanh')")
gemm_rcr_bias_sigmoid = _activation_variant("gemm_rcr_bias_sigmoid", "y = sigmoid(linear(A, B, bias))")
gemm_rcr_bias_tanh = _activation_variant("gemm_rcr_bias_tanh", "y = tanh(linear(A, B, bias))")
gemm_rcr_bias_swish = _activation_variant("gemm_rcr_bias_swish", "y = silu(linear(A, B, bias))")
gemm_rcr_bias_hardswish = _activation_variant("gemm_rcr_bias_hardswish", "y = hardswish(linear(A, B, bias))")
