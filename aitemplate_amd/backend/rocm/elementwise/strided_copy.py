"""Registry hooks of the strided row copy that a split or a concatenate becomes where no GEMM-family op takes the
piece as a view.

Take the place of python/aitemplate/backend/rocm/tensor/split.py and concatenate.py (which instantiate
backend/common/split_common.py:479-560 and concatenate_common.py:661-860): one generated function per op, with the
row length, the pitch and the offset of the strided side as literals and the number of rows (the product of the
dims in front of the split / concatenated dim, which may be dynamic) as its argument."""
from typing import Any, Dict

from ....compiler.ops.common.view_ops import copy_geometry
from ... import registry
from ..gemm import common


def _signature(func_name: str) -> str:
    return f"void {func_name}(void* dst, const void* src, int64_t rows, hipStream_t stream)"


def gen_function(func_attrs: Dict[str, Any]) -> str:
    func_name = func_attrs["name"]
    _, _, row_bytes, pitch, offset = copy_geometry(func_attrs)
    if func_attrs["copy_kind"] == "slice":
        src, dst, src_pitch, dst_pitch = f"static_cast<const char*>(src) + {offset}", "dst", pitch, row_bytes
    else:
        src, dst, src_pitch, dst_pitch = "src", f"static_cast<char*>(dst) + {offset}", row_bytes, pitch
    return f"""{common.HEADER}
{_signature(func_name)} {{
  check_rc(aitamd_copy_rows({src}, {dst}, rows, {row_bytes}, {src_pitch}, {dst_pitch}, stream), "{func_name}");
}}
{common.FOOTER}"""


def func_decl(func_attrs: Dict[str, Any]) -> str:
    return _signature(func_attrs["name"]) + ";"


def func_call(func_attrs: Dict[str, Any], indent: str = "  ") -> str:
    full = copy_geometry(func_attrs)[0]
    rows = " * ".join(d._attrs["name"] for d in full._attrs["shape"][:func_attrs["copy_dim"]]) or "1"
    args = [func_attrs["outputs"][0]._attrs["name"], func_attrs["inputs"][0]._attrs["name"], rows, "stream"]
    return f"{indent}{func_attrs['name']}({', '.join(args)});"


registry.reg("rocm.strided_copy.gen_function", gen_function)
registry.reg("rocm.strided_copy.func_decl", func_decl)
registry.reg("rocm.strided_copy.func_call", func_call)
