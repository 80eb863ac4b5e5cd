"""The element-wise graph op.

Counterpart of python/aitemplate/compiler/ops/common/elementwise.py:165-296, without jagged tensors and
type promotion.  This backend has no stand-alone element-wise kernels: the op exists so that graphs
written as `gemm_rcr_bias(...)` followed by element-wise ops can be built unchanged, and
`transform.fuse_mm_elementwise` folds those chains into the fused GEMM epilogues.  An element-wise op
that survives the pass makes `compile_model` raise."""
from typing import List

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

    def gen_function(self) -> str:
        raise NotImplementedError(
            f"elementwise({self._attrs['func']}) was not fused into a GEMM epilogue and this backend has no "
            "stand-alone element-wise kernels")
