"""gemm_rcr / gemm_rcr_bias whose result is stored through a 5-D output permutation.

Counterparts: python/aitemplate/compiler/ops/gemm_universal/gemm_rcr_permute.py:27-96 and
gemm_rcr_bias_permute.py:28-84.  With shape = (t1, t2, t3) and a [M, N] product:

  layout "m2n3":            view [M/t1, t1, t2, t3, N/(t2*t3)], store dims (2, 0, 3, 1, 4)
                            -> [t2, M/t1, t3, t1, N/(t2*t3)]
  layout "m3n2" / "20314":  view [M/(t1*t2), t1, t2, t3, N/t3], store dims (2, 0, 3, 1, 4)
                            -> [t2, M/(t1*t2), t3, t1, N/t3]

("20314" takes the m3n2 form on ROCm: gemm_rcr_bias_permute.py:66-72; the bias-free op exists on ROCm for
"m2n3" only, the other layouts of gemm_rcr_permute.py are CUDA kernels.)  The packed QKV projection of
nn.MultiheadAttention uses "m2n3" with shape (seq_len, 3, heads) to get [3, batch, heads, seq_len, head_dim]."""
from typing import Tuple

from ...base import IntImm, Tensor
from ...tensor_accessor import TensorAccessor
from ..common.view_ops import reshape
from .gemm_rcr import gemm_rcr
from .gemm_rcr_bias import gemm_rcr_bias


def _static_mn(op_name: str, output_shape):
    m = 1
    for d in output_shape[:-1]:
        if not isinstance(d, IntImm):
            raise RuntimeError(f"{op_name} needs a static M, got {output_shape}")
        m *= d.value()
    n = output_shape[-1]
    if not isinstance(n, IntImm):
        raise RuntimeError(f"{op_name} needs a static N, got {output_shape}")
    return m, n.value()


def _permuted_shape(op_name: str, layout: str, shape, m: int, n: int):
    t1, t2, t3 = (int(t) for t in shape)
    if layout == "m2n3":
        if m % t1 or n % (t2 * t3):
            raise RuntimeError(f"{op_name}: [{m}, {n}] does not split by shape {tuple(shape)}")
        return [t2, m // t1, t3, t1, n // (t2 * t3)]
    if m % (t1 * t2) or n % t3:
        raise RuntimeError(f"{op_name}: [{m}, {n}] does not split by shape {tuple(shape)}")
    return [t2, m // (t1 * t2), t3, t1, n // t3]


class _permute_mixin:
    """Shared tail of __call__: the op's own output stays [M, N] (its memory holds the permuted order) and
    the caller gets the 5-D view, as in the reference."""

    def _set_layout(self, shape: Tuple[int], layout: str, op_of_layout) -> None:
        if layout not in op_of_layout:
            raise NotImplementedError("{} is not implemented!".format(layout))
        if len(shape) != 3:
            raise RuntimeError(f"shape must have 3 entries, got {shape}")
        self._attrs["op"] = op_of_layout[layout]
        self._attrs["shape"] = tuple(int(t) for t in shape)
        self._attrs["layout"] = "Permute5D_{}".format(layout)
        self._attrs["permute_shape"] = "_".join(map(str, shape))

    def _permuted_view(self, inputs, output_shape) -> Tensor:
        layout = self._attrs["layout"].split("_")[-1]
        m, n = _static_mn(self._attrs["op"], output_shape)
        view_shape = _permuted_shape(self._attrs["op"], "m2n3" if layout == "m2n3" else "m3n2",
                                     self._attrs["shape"], m, n)
        flat_shape = [IntImm(m), IntImm(n)]
        output = Tensor(flat_shape, src_ops={self}, dtype=inputs[0].dtype())
        self._attrs["outputs"] = [output]
        self._attrs["output_accessors"] = [TensorAccessor(output)]
        # the stores are vectorised along the innermost permuted dim
        self._extract_epilogue_alignment(view_shape)
        return reshape()(output, view_shape)

    def _get_op_attributes(self):
        return {"layout": self._attrs["layout"].split("_")[-1], "shape": self._attrs["shape"]}


class gemm_rcr_permute(_permute_mixin, gemm_rcr):
    """permute(linear(A, B).reshape(...), (2, 0, 3, 1, 4)); ROCm implements layout "m2n3"."""

    def __init__(self, shape: Tuple[int], layout: str = "m2n3"):
        gemm_rcr.__init__(self)
        self._set_layout(shape, layout, {"m2n3": "gemm_rcr_permute_m2n3"})

    def _extract_dims(self, for_profiling: bool = False):
        return _flat_output_dims(gemm_rcr._extract_dims(self, for_profiling))

    def __call__(self, a: Tensor, b: Tensor) -> Tensor:
        a, b = self._align_ab(a, b)
        self._attrs["inputs"] = [a, b]
        self._attrs["input_accessors"] = [TensorAccessor(a), TensorAccessor(b)]
        self._set_depth()
        self._sanity_check(a, b)
        return self._permuted_view([a, b], self._infer_shapes(a, b))


class gemm_rcr_bias_permute(_permute_mixin, gemm_rcr_bias):
    """permute(linear(A, B, bias).reshape(...), (2, 0, 3, 1, 4)) for layouts "20314", "m2n3", "m3n2"."""

    def __init__(self, shape: Tuple[int], layout: str = "20314"):
        gemm_rcr_bias.__init__(self)
        self._set_layout(shape, layout, {"20314": "gemm_rcr_bias_permute", "m2n3": "gemm_rcr_bias_permute_m2n3",
                                         "m3n2": "gemm_rcr_bias_permute_m3n2"})

    def _extract_dims(self, for_profiling: bool = False):
        return _flat_output_dims(gemm_rcr_bias._extract_dims(self, for_profiling))

    def __call__(self, a: Tensor, b: Tensor, bias: Tensor) -> Tensor:
        a, b = self._align_ab(a, b)
        self._attrs["inputs"] = [a, b, bias]
        self._attrs["input_accessors"] = [TensorAccessor(t) for t in self._attrs["inputs"]]
        self._set_depth()
        self._sanity_check(a, b)
        return self._permuted_view([a, b, bias], self._infer_shapes(a, b, bias))


def _flat_output_dims(dims):
    """The output tensor of a permuting op is 2-D whatever A's rank: M is its dim 0, N its dim 1."""
    from .gemm_common import DimInfo, Source

    fixed = {}
    for name, infos in dims.items():
        kept = [d for d in infos if d.source != Source.OUTPUT]
        if name == "M":
            kept.append(DimInfo(Source.OUTPUT, tensor_idx=0, dim_idx=0))
        elif name == "N":
            kept.append(DimInfo(Source.OUTPUT, tensor_idx=0, dim_idx=1))
        fixed[name] = kept
    return fixed
