"""ROCm (gfx950) code generation shared by the GEMM-family ops.

Replaces python/aitemplate/backend/rocm/gemm/common.py:29-1020 (jinja2 templates that
instantiate Composable Kernel device ops and compile one profiler per instance).  Here
the kernels are prebuilt in libaitemplate_amd_kernels.so, so

  * `config` lists the library's instances for the op's epilogue and dtype,
  * `filter` asks the library whether an instance supports the workload's alignment,
  * `gen_profiler` has nothing to compile: it places the prebuilt profiler executable at
    the path the frontend expects (<workdir>/profiler/<op>/<profiler_filename>),
  * `gen_function` emits a small host function with the reference's launcher signature
        void NAME(void* in, void* weight, void* out, [void* bias, void* d0, void* d1,]
                  int64_t* a_dims..., int64_t* b_dims..., int64_t* c_dims..., hipStream_t)
    (reference: common.py:107-171,491-521) whose body evaluates M/N/K from the dim
    pointers, writes the output dims, picks the profiled instance by the exec condition
    and calls the library's C ABI.
"""
from __future__ import annotations

import os
import shutil
from collections import OrderedDict
from typing import Any, Dict, List

from .... import _kernels
from ....compiler.base import IntImm
from ....compiler.ops.gemm_universal.gemm_common import DimInfo, Source, gemm_inverse_key_func
from ...target import Target

DTYPE_ID = {"float16": 0, "bfloat16": 1}

# reference op name -> (epilogue id, extra pointer arguments after `out`)
EXTRA_PTRS = {0: [], 1: ["bias_ptr"]}


def epilogue_id(op_name: str) -> int:
    if op_name in _kernels.PERMUTE_OPS:
        return _kernels.PERMUTE_OPS[op_name][0]
    if op_name in _kernels.LAYOUT_OPS:
        return _kernels.EPI_ADD if op_name.endswith("_add") else 0
    return _kernels.EPILOGUE_OF_OP[op_name]


def extra_pointer_names(op_name: str) -> List[str]:
    epi = epilogue_id(op_name)
    if epi == 0:
        return []
    n = _kernels.NUM_RESIDUALS_OF_EPILOGUE[epi]
    return ["bias_ptr"] + [f"d{i}_ptr" for i in range(n)]


# ---- config / filter / profiler --------------------------------------------------
def gemm_config(func_attrs: Dict[str, Any], dtype: str = "float16", kind: str = "gemm") -> None:
    """Fill func_attrs["op_instance"] with {instance name: algo index} for this op."""
    if dtype not in DTYPE_ID:
        raise NotImplementedError(f"the gfx950 GEMM backend supports float16 and bfloat16, not {dtype}")
    op = func_attrs["op"]
    epi = epilogue_id(op)
    names = _kernels.gemm_algo_names(epi, DTYPE_ID[dtype])
    if not names:
        raise RuntimeError(f"kernel library has no instances for {op} / {dtype}")
    func_attrs["op_instance"] = OrderedDict((n, i) for i, n in enumerate(names))
    func_attrs["profiler_args"] = [kind, op, str(DTYPE_ID[dtype])]


def gemm_filter(instance_name: str, func_attrs: Dict[str, Any], ab_alignment: int) -> bool:
    """True when the instance can run every profiled workload of the op (load-width vs K alignment)."""
    lib = _kernels.load()
    dtype = DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    epi = epilogue_id(func_attrs["op"])
    algo = func_attrs["op_instance"][instance_name]
    for key in func_attrs["exec_path"]:
        m, n, k = gemm_inverse_key_func(key)[-3:]
        # ab_alignment is in elements; the library wants the byte alignment of the operand rows
        if not lib.aitamd_gemm_algo_supported(epi, dtype, algo, m, n, k, k, k, max(2, min(16, ab_alignment * 2))):
            return False
    return True


def place_profiler(func_attrs: Dict[str, Any], workdir: str, profiler_filename: str):
    """Make <workdir>/profiler/<op>/<profiler_filename> the prebuilt profiler; returns [(sources, exe)]."""
    target = Target.current()
    src_exe = target.profiler_executable()
    op_dir = os.path.join(workdir, "profiler", func_attrs["op"])
    os.makedirs(op_dir, exist_ok=True)
    exe = os.path.join(op_dir, profiler_filename)
    if os.path.lexists(exe):
        os.remove(exe)
    try:
        os.symlink(src_exe, exe)
    except OSError:
        shutil.copy2(src_exe, exe)
    return [([], exe)]


def gemm_gen_profiler(func_attrs, workdir, profiler_filename, dim_info_dict):
    return place_profiler(func_attrs, workdir, profiler_filename)


def gemm_select_algo(func_attrs: Dict[str, Any], exec_key: str) -> str:
    """Instance chosen without timing (CI_FLAG=CIRCLECI or no GPU): the library's shape heuristic."""
    lib = _kernels.load()
    dtype = DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    epi = epilogue_id(func_attrs["op"])
    dims = gemm_inverse_key_func(exec_key)
    m, n, k = dims[-3:]
    batch = dims[0] if len(dims) == 4 else 1
    align = 16
    while align > 2 and (k * 2) % align != 0:
        align //= 2
    algo = lib.aitamd_gemm_heuristic_algo(epi, dtype, batch, m, n, k, k, k, align)
    names = list(func_attrs["op_instance"].keys())
    all_names = _kernels.gemm_algo_names(epi, dtype)
    if algo >= 0 and all_names[algo] in func_attrs["op_instance"]:
        return all_names[algo]
    return Target.current().select_minimal_algo(names)


# ---- source generation ---------------------------------------------------------------
def dim_param_names(prefix: str, rank: int) -> List[str]:
    return [f"{prefix}_dim{i}" for i in range(rank)]


def gen_dim_calculator(dim_info: DimInfo, arg_prefixes: Dict[Source, List[str]]) -> str:
    """C++ expression for one problem dim as a product of dereferenced dim pointers
    (reference: backend/common/gemm_common.py:25-46)."""
    prefix = arg_prefixes[dim_info.source][dim_info.tensor_idx]
    return " * ".join(f"(*{prefix}_dim{i})" for i in dim_info.dim_idx) or "1"


def gen_shape_eval_code(dim_info_dict: Dict[str, List[DimInfo]], in_prefixes: List[str], out_prefixes: List[str],
                        indent: str = "  ") -> str:
    """`int64_t M = ...;` lines from the input dims, then the output dims written back
    (reference: backend/common/gemm_common.py:48-71)."""
    prefixes = {Source.INPUT: in_prefixes, Source.OUTPUT: out_prefixes}
    lines = []
    for name, infos in dim_info_dict.items():
        src = None
        for d in infos:
            if d.source == Source.INPUT and not d.placeholder:
                src = d
                break
        if src is None:  # dims only the output carries (none in this family) keep their current value
            src = next(d for d in infos if not d.placeholder)
        lines.append(f"{indent}const int64_t {name} = {gen_dim_calculator(src, prefixes)};")
    for name, infos in dim_info_dict.items():
        for d in infos:
            if d.source == Source.OUTPUT and len(d.dim_idx) == 1:
                lines.append(f"{indent}*{out_prefixes[d.tensor_idx]}_dim{d.dim_idx[0]} = {name};")
    return "\n".join(lines)


def accessor_offset_and_pitch(accessor, what: str):
    """(element offset, row pitch expression or None) of a 2-D-viewed operand."""
    offset = int(getattr(accessor, "offset", 0) or 0)
    pitch = None
    if getattr(accessor, "actual_shapes", None) is not None:
        pitch = accessor.row_pitch()
    return offset, pitch


HEADER = """// generated by aitemplate_amd (ROCm / gfx950 GEMM backend) - do not edit
#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <cmath>
#include <stdexcept>
#include <string>

#include "aitemplate_amd_kernels.h"

namespace {

int resolve_instance(int epilogue, int dtype, const char* name) {
  const int algo = aitamd_gemm_find_algo(epilogue, dtype, name);
  if (algo < 0) throw std::runtime_error(std::string("kernel instance not found in the library: ") + name);
  return algo;
}

void check_rc(int rc, const char* op) {
  if (rc != 0) throw std::runtime_error(std::string(op) + ": " + aitamd_last_error());
}

}  // namespace

namespace ait {
"""

FOOTER = "\n}  // namespace ait\n"


def header_with_table(epilogue: int, dtype: int) -> str:
    """HEADER plus a reference that makes the linker take the instance table of (epilogue, dtype) out of the
    kernel archive: a model library carries the kernels of the tables its op functions name, nothing else."""
    sym = f"aitamd_gemm_table_{epilogue}_{dtype}"
    ref = (f'extern "C" void {sym}();\n'
           f"namespace {{\n__attribute__((used)) void (*const keep_{sym})() = &{sym};\n}}  // namespace\n")
    return HEADER.replace("\nnamespace ait {\n", "\n" + ref + "\nnamespace ait {\n")


def gemm_signature(func_name: str, op_name: str, a_rank: int, b_rank: int, c_rank: int, pdims: int = 0,
                   with_workspace: bool = False) -> str:
    """Launcher prototype; `pdims` trailing `const int p_dim<i>` carry a permuting op's shape attribute
    (reference: backend/rocm/gemm/common.py:140-160).  Ops whose profiled instance needs scratch memory take the
    model's shared workspace and its size after the tensor pointers (the reference's CUDA launchers do the same,
    backend/cuda/gemm_universal/common.py:317-345)."""
    ptrs = ["void* in_ptr", "void* weight_ptr", "void* out_ptr"] + [f"void* {p}" for p in extra_pointer_names(op_name)]
    if with_workspace:
        ptrs += ["uint8_t* workspace", "int64_t workspace_bytes"]
    dims = [f"int64_t* {n}" for n in dim_param_names("a", a_rank) + dim_param_names("b", b_rank)
            + dim_param_names("c", c_rank)]
    perm = [f"const int p_dim{i}" for i in range(pdims)]
    return f"void {func_name}({', '.join(ptrs + dims + perm + ['hipStream_t stream'])})"


def uses_workspace(func_attrs: Dict[str, Any]) -> bool:
    """The op's profiled instances asked for scratch memory (the profiler's WS field, kept as the op's
    `workspace` attribute)."""
    return int(func_attrs.get("workspace", 0) or 0) > 0


def gemm_gen_function(func_attrs: Dict[str, Any], exec_cond_template: str, dim_info_dict) -> str:
    op = func_attrs["op"]
    func_name = func_attrs["name"]
    dtype = DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    epi = epilogue_id(op)
    a_acc, b_acc = func_attrs["input_accessors"][0], func_attrs["input_accessors"][1]
    c_acc = func_attrs["output_accessors"][0]
    a_rank, b_rank, c_rank = len(a_acc.original_shapes), len(b_acc.original_shapes), len(c_acc.original_shapes)
    off_a, lda = accessor_offset_and_pitch(a_acc, "a")
    off_b, ldb = accessor_offset_and_pitch(b_acc, "b")
    off_c, ldc = accessor_offset_and_pitch(c_acc, "c")
    extras = extra_pointer_names(op)
    elem = "uint16_t"  # both supported dtypes are 2 bytes wide: offsets are applied on 16-bit pointers

    shape_code = gen_shape_eval_code(dim_info_dict, ["a", "b"] + [f"x{i}" for i in range(len(extras))], ["c"])
    bias_arg = "bias_ptr" if "bias_ptr" in extras else "nullptr"
    d0_arg = "d0_ptr" if "d0_ptr" in extras else "nullptr"
    d1_arg = "d1_ptr" if "d1_ptr" in extras else "nullptr"
    # residual tensors may be strided views as well: each has its own offset, both share one row pitch
    ldd = "N"
    res_offsets = {}
    pitches = set()
    for name in extras:
        if name == "bias_ptr":
            continue
        off_d, p = accessor_offset_and_pitch(func_attrs["input_accessors"][2 + extras.index(name)], name)
        res_offsets[name] = off_d
        pitches.add(p)
    if len(pitches) > 1:
        raise NotImplementedError(f"{op}: the two residuals must have the same row pitch, got {sorted(map(str, pitches))}")
    if pitches and next(iter(pitches)) is not None:
        ldd = str(next(iter(pitches)))
    if "bias_ptr" in extras:
        b_off, b_pitch = accessor_offset_and_pitch(func_attrs["input_accessors"][2], "bias")
        if b_off or b_pitch is not None:
            raise NotImplementedError(f"{op}: the bias cannot be a view of a wider tensor")
    if d0_arg != "nullptr":
        d0_arg = "d0"
    if d1_arg != "nullptr":
        d1_arg = "d1"
    residual_ptrs = "".join(
        f"  const {elem}* {n[:-4]} = static_cast<const {elem}*>({n}) + {res_offsets[n]};\n" for n in res_offsets)
    # The instance was profiled on contiguous operands.  A view whose offset or pitch is not a whole number of
    # 16-byte pieces can rule that instance out; the library then picks among the instances that fit.
    misaligned = any(v % 8 for v in (off_a, off_b, lda or 0, ldb or 0))
    algo_expr = "-1" if misaligned else "algo"

    launches = []
    for key, item in func_attrs["exec_path"].items():
        if not item.algo:
            raise RuntimeError(f"{func_name}: workload {key} has no kernel instance; run profiling first")
        if uses_workspace(func_attrs):
            # a dynamic dim can ask for more scratch memory than the profiled sizes did: the library's own choice
            # among the instances that fit takes over then
            call = (f"aitamd_gemm_rcr_ws({epi}, {dtype}, "
                    f"aitamd_gemm_workspace_bytes({epi}, {dtype}, algo, 1, M, N, K) <= workspace_bytes ? {algo_expr} : -1, "
                    f"a, b, {bias_arg}, {d0_arg}, {d1_arg}, c, M, N, K, "
                    f"lda, ldb, ldc, ldd, workspace, workspace_bytes, stream)")
        else:
            call = (f"aitamd_gemm_rcr({epi}, {dtype}, {algo_expr}, a, b, {bias_arg}, {d0_arg}, {d1_arg}, c, M, N, K, "
                    f"lda, ldb, ldc, ldd, stream)")
        program = (
            f'static const int algo = resolve_instance({epi}, {dtype}, "{item.algo}");\n'
            f'    check_rc({call}, "{func_name}");'
        )
        launches.append(exec_cond_template.format(indent="  ", cond=item.exec_cond, program=program))

    return f"""{header_with_table(epi, dtype)}
{gemm_signature(func_name, op, a_rank, b_rank, c_rank, with_workspace=uses_workspace(func_attrs))} {{
{shape_code}
  const {elem}* a = static_cast<const {elem}*>(in_ptr) + {off_a};
  const {elem}* b = static_cast<const {elem}*>(weight_ptr) + {off_b};
  {elem}* c = static_cast<{elem}*>(out_ptr) + {off_c};
{residual_ptrs}  const int64_t lda = {lda if lda is not None else "K"};
  const int64_t ldb = {ldb if ldb is not None else "K"};
  const int64_t ldc = {ldc if ldc is not None else "N"};
  const int64_t ldd = {ldd};
  if (M == 0 || N == 0) return;  // empty output
{"".join(launches)}
  throw std::runtime_error(
      "Unsupported workload for this {op} specialization: M=" + std::to_string(M) + " N=" + std::to_string(N) +
      " K=" + std::to_string(K));
}}
{FOOTER}"""


def gemm_func_decl(func_attrs: Dict[str, Any]) -> str:
    a_rank = len(func_attrs["input_accessors"][0].original_shapes)
    b_rank = len(func_attrs["input_accessors"][1].original_shapes)
    c_rank = len(func_attrs["output_accessors"][0].original_shapes)
    return gemm_signature(func_attrs["name"], func_attrs["op"], a_rank, b_rank, c_rank,
                          with_workspace=uses_workspace(func_attrs)) + ";"


def gemm_func_call(func_attrs: Dict[str, Any], indent: str = "  ") -> str:
    """The call placed in the model's op list: tensor members, then the address of every dim member."""
    inputs, output = func_attrs["inputs"], func_attrs["outputs"][0]
    ptrs = [t._attrs["name"] for t in inputs[:2]] + [output._attrs["name"]] + [t._attrs["name"] for t in inputs[2:]]
    if uses_workspace(func_attrs):
        # every op gets the whole shared workspace: ops of one model run one after the other on its stream
        ptrs += ["workspace_", "workspace_size_"]
    dims = []
    for acc in (func_attrs["input_accessors"][0], func_attrs["input_accessors"][1],
                func_attrs["output_accessors"][0]):
        dims += ["&" + d._attrs["name"] for d in acc.original_shapes]
    return f"{indent}{func_attrs['name']}({', '.join(ptrs + dims + ['stream'])});"
