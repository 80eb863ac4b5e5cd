"""The element-wise graph op.

Counterpart of python/aitemplate/compiler/ops/common/elementwise.py:165-296, without jagged tensors and
type promotion.  Graphs written as `gemm_rcr_bias(...)` followed by element-wise ops are built unchanged
and `transform.fuse_mm_elementwise` folds those chains into the fused GEMM epilogues.  An element-wise op
that survives the pass runs as one launch of the stand-alone kernel (one op per launch: the reference
fuses such groups into one generated kernel, fused_elementwise.py); `standalone_plan` says which forms
that kernel takes, and `compile_model` raises for the others."""
from typing import List, Optional, Tuple

from ...base import IntImm, IntVar, Operator, Tensor
from .epilogue import FuncEnum


def _broadcast_shapes(shapes: List[List[IntVar]]) -> List[IntVar]:
    """numpy-style broadcast of dense shapes (reference: elementwise.py:68-87)."""
    rank = max(len(s) for s in shapes)
    out: List[IntVar] = []
    for i in range(rank):
        dim = None
        for s in shapes:
            j = i - (rank - len(s))
            if j < 0:
                continue
            d = s[j]
            if dim is None or (isinstance(dim, IntImm) and dim.value() == 1):
                dim = d
            elif isinstance(d, IntImm) and d.value() == 1:
                continue
            elif d != dim:
                raise RuntimeError(f"Tensor shapes of elementwise ops are not compatible! Shapes: {shapes}")
        out.append(dim)
    return out


# functions of the stand-alone kernel (the library's aitamd_elementwise_supported answers the same)
STANDALONE_FUNCS = frozenset({
    FuncEnum.ADD, FuncEnum.SUB, FuncEnum.MUL, FuncEnum.DIV, FuncEnum.TANH, FuncEnum.ABS, FuncEnum.EXP, FuncEnum.SQRT,
    FuncEnum.MAX, FuncEnum.MIN, FuncEnum.SIGMOID, FuncEnum.RELU, FuncEnum.SILU, FuncEnum.GELU, FuncEnum.FASTGELU,
    FuncEnum.COS, FuncEnum.SIN, FuncEnum.SIGN, FuncEnum.LOGE, FuncEnum.LRELU, FuncEnum.POW, FuncEnum.SOFTSIGN,
    FuncEnum.FLOOR, FuncEnum.LOG1P, FuncEnum.RECIPROCAL,
})
_BINARY_FUNCS = frozenset({FuncEnum.ADD, FuncEnum.SUB, FuncEnum.MUL, FuncEnum.DIV, FuncEnum.MAX, FuncEnum.MIN,
                           FuncEnum.LRELU, FuncEnum.POW})


def _strip_leading_ones(shape: List[IntVar]) -> List[IntVar]:
    i = 0
    while i < len(shape) and isinstance(shape[i], IntImm) and shape[i].value() == 1:
        i += 1
    return list(shape[i:])


def standalone_plan(func_attrs) -> Tuple[Tensor, Optional[Tensor], float, int]:
    """How the stand-alone kernel runs this op: (operand of the output's shape, operand that tiles the
    flattened output or None, constant second operand, 1 when the function takes them in the other order).

    The kernel computes out[i] = f(a[i], b[i % numel(b)]): the second operand is a number, or a tensor
    whose dims, leading 1s dropped, are the output's trailing dims (same shape, a bias row, one element).
    Anything else (both operands broadcast, a broadcast over inner dims, three operands, a function the
    kernel does not have) raises NotImplementedError."""
    func, args = func_attrs["func"], func_attrs["args"]
    out_shape = list(func_attrs["outputs"][0]._attrs["shape"])
    what = f"elementwise({func.name})"
    if func not in STANDALONE_FUNCS:
        raise NotImplementedError(f"{what} has no stand-alone kernel in this backend")
    want = 2 if func in _BINARY_FUNCS else 1
    if len(args) != want:
        raise NotImplementedError(f"{what} with {len(args)} operands is not supported")
    if want == 1:
        if args[0].is_a_const_num():
            raise NotImplementedError(f"{what} of a constant number is not supported")
        return args[0], None, 0.0, 0
    full = [i for i, a in enumerate(args) if not a.is_a_const_num() and list(a._attrs["shape"]) == out_shape]
    if not full:
        raise NotImplementedError(f"{what}: neither operand has the output's shape (both broadcast)")
    first = full[0]
    a, b = args[first], args[1 - first]
    if b.is_a_const_num():
        return a, None, float(b._attrs["value"]), first
    tail = _strip_leading_ones(b._attrs["shape"])
    if tail != out_shape[len(out_shape) - len(tail):]:
        raise NotImplementedError(
            f"{what}: an operand of shape {[str(d) for d in b._attrs['shape']]} does not tile the flattened "
            f"output of shape {[str(d) for d in out_shape]} (only a broadcast over leading dims does)")
    return a, b, 0.0, first


class elementwise(Operator):
    def __init__(self, func_enum: FuncEnum) -> None:
        super().__init__()
        self._attrs["op"] = "elementwise"
        self._attrs["func"] = func_enum
        self._attrs["has_profiler"] = False

    def __call__(self, *args) -> Tensor:
        if len(args) == 0:
            raise RuntimeError("Elementwise op {} doesn't have inputs!".format(self._attrs["func"]))
        converted, dtype = [], None
        for arg in args:
            if isinstance(arg, (int, float)):
                converted.append(Tensor(shape=[], value=arg))
            elif isinstance(arg, Tensor):
                if not arg.is_a_const_num():
                    if dtype is None:
                        dtype = arg.dtype()
                    elif arg.dtype() != dtype:
                        raise NotImplementedError(
                            f"Type promotions are not supported; got dtype {arg.dtype()}, but expected {dtype}")
                converted.append(arg)
            else:
                raise RuntimeError(f"Unsupported data type {arg} in elementwise {self}!")
        dtype = dtype or "float16"
        for arg in converted:
            if arg.is_a_const_num():
                arg._attrs["dtype"] = dtype
        self._attrs["args"] = list(converted)
        self._attrs["inputs"] = [a for a in converted if not a.is_a_const_num()]
        self._set_depth()
        shape = _broadcast_shapes([a._attrs["shape"] for a in converted])
        output = Tensor(shape, src_ops={self}, dtype=dtype)
        self._attrs["outputs"] = [output]
        return output

    def _get_op_attributes(self):
        return {"func_enum": self._attrs["func"]}

    def replace_input_tensor(self, old_tensor, new_tensor) -> None:
        super().replace_input_tensor(old_tensor, new_tensor)
        self._attrs["args"] = [new_tensor if t is old_tensor else t for t in self._attrs["args"]]

    def standalone_plan(self) -> Tuple[Tensor, Optional[Tensor], float, int]:
        return standalone_plan(self._attrs)

    def gen_function(self) -> str:
        from ....backend import registry
        from ....backend.target import Target

        return registry.get(f"{Target.current().name()}.elementwise.gen_function")(self._attrs)
