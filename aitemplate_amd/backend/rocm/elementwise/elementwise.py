"""Registry hooks of the stand-alone element-wise op.

Take the place of python/aitemplate/backend/rocm/elementwise/fused_elementwise.py:27-65 (`fused_elementwise_gen_function`,
`fused_elementwise_gen_function_decl`, `fused_elementwise_gen_function_call`, which generate one kernel per fused
group through backend/common/elementwise_common.py) for the one-op case: an `elementwise` op that no GEMM epilogue
absorbed becomes one launch of `aitamd_elementwise`.  The output has the shape of the larger operand; the other
operand is a constant number or a tensor whose dims, leading 1s dropped, are the output's trailing dims (a bias row,
a same-shape residual, a one-element tensor): it tiles the flattened output with period prod(its dims)."""
import math
from typing import Any, Dict, List

from ....compiler.ops.common.elementwise import standalone_plan
from ... import registry
from ..gemm import common


def _dims(t) -> List:
    return t._attrs["shape"]


def _signature(func_name: str) -> str:
    return (f"void {func_name}(void* out, const void* a, const void* b, int64_t numel, int64_t b_period, "
            "hipStream_t stream)")


def float_literal(value: float) -> str:
    """C++ spelling of a constant operand: a float literal, or the <cmath> macros for the values that have none
    (repr() gives 'inf' and 'nan', and 'inff' is not C++)."""
    value = float(value)
    if math.isnan(value):
        return "NAN"
    if math.isinf(value):
        return "INFINITY" if value > 0 else "-INFINITY"
    return f"{value!r}f"


def gen_function(func_attrs: Dict[str, Any]) -> str:
    func_name = func_attrs["name"]
    a, b, value, swap = standalone_plan(func_attrs)
    dtype = common.DTYPE_ID[a._attrs["dtype"]]
    return f"""{common.HEADER}
{_signature(func_name)} {{
  check_rc(aitamd_elementwise({func_attrs["func"].value} /* {func_attrs["func"].name} */, {dtype}, a, b, out, numel, b_period,
                              {float_literal(value)}, {swap}, stream), "{func_name}");
}}
{common.FOOTER}"""


def func_decl(func_attrs: Dict[str, Any]) -> str:
    return _signature(func_attrs["name"]) + ";"


def _numel(t) -> str:
    return " * ".join(d._attrs["name"] for d in _dims(t)) or "1"


def func_call(func_attrs: Dict[str, Any], indent: str = "  ") -> str:
    a, b, _, _ = standalone_plan(func_attrs)
    out = func_attrs["outputs"][0]
    args = [out._attrs["name"], a._attrs["name"], b._attrs["name"] if b is not None else "nullptr", _numel(out),
            _numel(b) if b is not None else "1", "stream"]
    return f"{indent}{func_attrs['name']}({', '.join(args)});"


registry.reg("rocm.elementwise.gen_function", gen_function)
registry.reg("rocm.elementwise.func_decl", func_decl)
registry.reg("rocm.elementwise.func_call", func_call)
