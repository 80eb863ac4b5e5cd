"""nn.Linear: y = x W^T (+ b) with an optional fused epilogue chosen by name.

Counterpart of python/aitemplate/frontend/nn/linear.py:24-101: `specialization` is appended
to "gemm_rcr[_bias]" to pick the fused op ("relu", "gelu", "fast_gelu", "add", "add_add",
"sigmoid", "tanh", "swish", "hardswish", "mul", "mul_add", "add_relu", ...)."""
from ...compiler import ops
from .module import Module
from .parameter import Parameter


class Linear(Module):
    def __init__(self, in_channels: int, out_channels: int, bias: bool = True, specialization: str = None,
                 dtype: str = "float16", **kwargs):
        super().__init__()
        self.weight = Parameter(shape=[out_channels, in_channels], dtype=dtype)
        op_name = "gemm_rcr_bias" if bias else "gemm_rcr"
        if specialization is not None:
            op_name += "_" + specialization
        if bias:
            self.bias = Parameter(shape=[out_channels], dtype=dtype)
        if not hasattr(ops, op_name):
            raise NotImplementedError(f"{op_name} is not an op of this backend")
        self.op = getattr(ops, op_name)(**kwargs)
        self.use_bias = bias
        self.in_channels = in_channels

    def forward(self, *args):
        assert len(args) >= 1
        x = args[0]
        inputs = [x, self.weight.tensor()]
        if self.use_bias:
            inputs.append(self.bias.tensor())
        inputs.extend(args[1:])
        return self.op(*inputs)
