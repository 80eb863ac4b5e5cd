"""gemm_rcr_bias fused with one or two tensors of the output's shape (residual adds, gates).

Counterparts: gemm_rcr_bias_broadcast.py:27-74 (base), gemm_rcr_bias_add.py:26-47,
gemm_rcr_bias_add_add.py:26-48, gemm_rcr_bias_add_relu.py, gemm_rcr_bias_add_add_relu.py,
gemm_rcr_bias_mul.py, gemm_rcr_bias_mul_add.py, gemm_rcr_bias_sigmoid_mul.py,
gemm_rcr_bias_sigmoid_mul_tanh.py, gemm_rcr_bias_mul_tanh.py of
python/aitemplate/compiler/ops/gemm_universal/."""
from ...base import Tensor
from ...tensor_accessor import TensorAccessor
from .gemm_rcr_bias import gemm_rcr_bias


class gemm_rcr_bias_broadcast(gemm_rcr_bias):
    def __init__(self):
        super().__init__()
        self._attrs["epilogue"] = "LinearCombinationResidualBlock"

    @staticmethod
    def is_valid_inputs(*inputs):
        if len(inputs) < 3:
            return False, f"input for gemm_rcr_bias_broadcast should be at least 3, got {len(inputs)} instead."
        ok, msg = gemm_rcr_bias.is_valid_inputs(inputs[0], inputs[1], inputs[2])
        if not ok:
            return False, msg
        if len(inputs) > 3:
            base_shape = gemm_rcr_bias()._infer_shapes(inputs[0], inputs[1], inputs[2])
            for d in inputs[3:]:
                if d.shape() != base_shape:
                    return False, f"Additional elementwise shape {d.shape()} doesn't match gemm_bias' shape {base_shape}"
        return True, ""

    def __call__(self, a: Tensor, b: Tensor, bias: Tensor, d0: Tensor, d1: Tensor = None) -> Tensor:
        a, b = self._align_ab(a, b)
        self._attrs["inputs"] = [a, b, bias, d0] + ([d1] if d1 is not None else [])
        if len(self._attrs["inputs"]) - 3 != self._attrs["num_sources"]:
            raise RuntimeError(
                f"{self._attrs['op']} takes {self._attrs['num_sources']} tensor(s) besides A, B and bias, "
                f"got {len(self._attrs['inputs']) - 3}")
        ok, msg = self.is_valid_inputs(*self._attrs["inputs"])
        if not ok:
            raise RuntimeError(msg)
        self._attrs["input_accessors"] = [TensorAccessor(t) for t in self._attrs["inputs"]]
        self._set_depth()
        self._sanity_check(a, b)
        return self._finish_call(self._attrs["inputs"], self._infer_shapes(a, b, bias))


def _variant(op_name: str, num_sources: int, doc: str):
    def __init__(self):
        gemm_rcr_bias_broadcast.__init__(self)
        self._attrs["op"] = op_name
        self._attrs["num_sources"] = num_sources

    return type(op_name, (gemm_rcr_bias_broadcast,), {"__init__": __init__, "__doc__": doc})


gemm_rcr_bias_add = _variant("gemm_rcr_bias_add", 1, "y = linear(A, B, bias) + D0")
gemm_rcr_bias_add_add = _variant("gemm_rcr_bias_add_add", 2, "y = linear(A, B, bias) + D0 + D1")
gemm_rcr_bias_add_relu = _variant("gemm_rcr_bias_add_relu", 1, "y = relu(linear(A, B, bias) + D0)")
gemm_rcr_bias_add_add_relu = _variant("gemm_rcr_bias_add_add_relu", 2, "y = relu(linear(A, B, bias) + D0 + D1)")
gemm_rcr_bias_mul = _variant("gemm_rcr_bias_mul", 1, "y = linear(A, B, bias) * D0")
gemm_rcr_bias_mul_add = _variant("gemm_rcr_bias_mul_add", 2, "y = linear(A, B, bias) * D0 + D1")
gemm_rcr_bias_sigmoid_mul = _variant("gemm_rcr_bias_sigmoid_mul", 1, "y = sigmoid(linear(A, B, bias)) * D0")
gemm_rcr_bias_sigmoid_mul_tanh = _variant(
    "gemm_rcr_bias_sigmoid_mul_tanh", 1, "y = tanh(sigmoid(linear(A, B, bias)) * D0)")
gemm_rcr_bias_mul_tanh = _variant("gemm_rcr_bias_mul_tanh", 1, "y = tanh(linear(A, B, bias) * D0)")
