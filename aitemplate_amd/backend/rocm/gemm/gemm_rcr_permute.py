"""Registry hooks of the permuting GEMMs: gemm_rcr_permute_m2n3, gemm_rcr_bias_permute,
gemm_rcr_bias_permute_m2n3, gemm_rcr_bias_permute_m3n2 and gemm_rrr_bias_permute (B stored [K, N]).

Replaces python/aitemplate/backend/rocm/gemm/gemm_rcr_permute_m2n3.py, gemm_rcr_bias_permute.py,
gemm_rcr_bias_permute_m2n3.py:30-160 and gemm_rcr_bias_permute_m3n2.py with their stride tables in
permute_common.py:20-130.  The launcher keeps the reference's shape: the usual pointers and dim pointers,
then `const int p_dim0, p_dim1, p_dim2` (the op's shape attribute) before the stream."""
from typing import Any, Dict

from .... import _kernels
from ....compiler.ops.gemm_universal.gemm_common import gemm_inverse_key_func
from ... import registry
from ...target import Target
from . import common

PERMUTE_OPS = list(_kernels.PERMUTE_OPS)


def _operands(op: str) -> int:
    return _kernels.LAYOUT_ID[_kernels.PERMUTE_OPERANDS.get(op, "rcr")]


def _ranks(func_attrs):
    return (len(func_attrs["input_accessors"][0].original_shapes),
            len(func_attrs["input_accessors"][1].original_shapes),
            len(func_attrs["output_accessors"][0].original_shapes))


def _signature(func_attrs) -> str:
    a_rank, b_rank, c_rank = _ranks(func_attrs)
    return common.gemm_signature(func_attrs["name"], func_attrs["op"], a_rank, b_rank, c_rank,
                                 pdims=len(func_attrs["shape"]))


def gen_function(func_attrs: Dict[str, Any], exec_cond_template: str, dim_info_dict) -> str:
    op = func_attrs["op"]
    func_name = func_attrs["name"]
    dtype = common.DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    epi, layout = _kernels.PERMUTE_OPS[op]
    a_acc, b_acc = func_attrs["input_accessors"][0], func_attrs["input_accessors"][1]
    c_acc = func_attrs["output_accessors"][0]
    if getattr(c_acc, "actual_shapes", None) is not None or getattr(c_acc, "offset", 0):
        raise NotImplementedError(f"{op} writes a contiguous permuted buffer; its output cannot be a strided view")
    off_a, lda = common.accessor_offset_and_pitch(a_acc, "a")
    off_b, ldb = common.accessor_offset_and_pitch(b_acc, "b")
    extras = common.extra_pointer_names(op)
    shape_code = common.gen_shape_eval_code(dim_info_dict, ["a", "b"] + [f"x{i}" for i in range(len(extras))], ["c"])
    bias_arg = "bias_ptr" if "bias_ptr" in extras else "nullptr"
    launches = []
    for key, item in func_attrs["exec_path"].items():
        if not item.algo:
            raise RuntimeError(f"{func_name}: workload {key} has no kernel instance; run profiling first")
        program = (
            f'static const int algo = resolve_instance({epi}, {dtype}, "{item.algo}");\n'
            f"    check_rc(aitamd_gemm_permute({_operands(op)}, {epi}, {dtype}, algo, a, b, {bias_arg}, out_ptr, M, N, K, "
            f'lda, ldb, {layout}, p_dim0, p_dim1, p_dim2, stream), "{func_name}");'
        )
        launches.append(exec_cond_template.format(indent="  ", cond=item.exec_cond, program=program))
    return f"""{common.header_with_table(epi, dtype)}
{_signature(func_attrs)} {{
{shape_code}
  const uint16_t* a = static_cast<const uint16_t*>(in_ptr) + {off_a};
  const uint16_t* b = static_cast<const uint16_t*>(weight_ptr) + {off_b};
  const int64_t lda = {lda if lda is not None else "K"};
  const int64_t ldb = {ldb if ldb is not None else ("N" if _operands(op) & 1 else "K")};
  if (M == 0 || N == 0) return;  // empty output
{"".join(launches)}
  throw std::runtime_error(
      "Unsupported workload for this {op} specialization: M=" + std::to_string(M) + " N=" + std::to_string(N) +
      " K=" + std::to_string(K));
}}
{common.FOOTER}"""


def func_decl(func_attrs: Dict[str, Any]) -> str:
    return _signature(func_attrs) + ";"


def func_call(func_attrs: Dict[str, Any], indent: str = "  ") -> str:
    call = common.gemm_func_call(func_attrs, indent)
    pdims = ", ".join(str(int(t)) for t in func_attrs["shape"])
    head, tail = call.rsplit("stream);", 1)
    return f"{head}{pdims}, stream);{tail}"


def _config(func_attrs, dtype="float16"):
    common.gemm_config(func_attrs, dtype, "gemm_permute")


def _filter(instance_name, func_attrs, ab_alignment) -> bool:
    operands = _operands(func_attrs["op"])
    if operands == 0:
        return common.gemm_filter(instance_name, func_attrs, ab_alignment)
    lib = _kernels.load()
    dtype = common.DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    epi = _kernels.PERMUTE_OPS[func_attrs["op"]][0]
    algo = func_attrs["op_instance"][instance_name]
    for key in func_attrs["exec_path"]:
        m, n, k = gemm_inverse_key_func(key)[-3:]
        if not lib.aitamd_gemm_algo_supported_layout(epi, dtype, operands, algo, m, n, k, k, n,
                                                     max(2, min(16, ab_alignment * 2))):
            return False
    return True


def _select_algo(func_attrs, exec_key) -> str:
    operands = _operands(func_attrs["op"])
    if operands == 0:
        return common.gemm_select_algo(func_attrs, exec_key)
    lib = _kernels.load()
    dtype = common.DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    epi = _kernels.PERMUTE_OPS[func_attrs["op"]][0]
    m, n, k = gemm_inverse_key_func(exec_key)[-3:]
    algo = lib.aitamd_gemm_heuristic_algo_layout(epi, dtype, operands, 1, m, n, k, k, n, 16)
    all_names = _kernels.gemm_algo_names(epi, dtype)
    if algo >= 0 and all_names[algo] in func_attrs["op_instance"]:
        return all_names[algo]
    return Target.current().select_minimal_algo(list(func_attrs["op_instance"].keys()))


for _op in PERMUTE_OPS:
    registry.reg(f"rocm.{_op}.config", _config)
    registry.reg(f"rocm.{_op}.filter", _filter)
    registry.reg(f"rocm.{_op}.gen_profiler", common.gemm_gen_profiler)
    registry.reg(f"rocm.{_op}.select_algo", _select_algo)
    registry.reg(f"rocm.{_op}.gen_function", gen_function)
    registry.reg(f"rocm.{_op}.func_decl", func_decl)
    registry.reg(f"rocm.{_op}.func_call", func_call)
