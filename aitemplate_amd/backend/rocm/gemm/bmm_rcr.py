"""Registry hooks of bmm_rcr.  Replaces python/aitemplate/backend/rocm/gemm/bmm_rcr.py:27-182 and
bmm_common.py:22-363: same launcher signature (3-D dim pointers), batch strides derived from the
operand ranks (a 2-D or batch-1 operand broadcasts with stride 0)."""
from typing import Any, Dict

from ... import registry
from . import common


def _config(func_attrs, dtype="float16"):
    common.gemm_config(func_attrs, dtype, "bmm")


def _signature(func_name: str, ranks) -> str:
    ptrs = ["void* in_ptr", "void* weight_ptr", "void* out_ptr"]
    dims = [f"int64_t* {n}" for prefix, r in zip("abc", ranks) for n in common.dim_param_names(prefix, r)]
    return f"void {func_name}({', '.join(ptrs + dims + ['hipStream_t stream'])})"


def _ranks(func_attrs):
    return (len(func_attrs["input_accessors"][0].original_shapes),
            len(func_attrs["input_accessors"][1].original_shapes),
            len(func_attrs["output_accessors"][0].original_shapes))


def gen_function(func_attrs: Dict[str, Any], exec_cond_template: str, dim_info_dict) -> str:
    func_name = func_attrs["name"]
    dtype = common.DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    ra, rb, rc = _ranks(func_attrs)
    off_a, lda = common.accessor_offset_and_pitch(func_attrs["input_accessors"][0], "a")
    off_b, ldb = common.accessor_offset_and_pitch(func_attrs["input_accessors"][1], "b")
    off_c, ldc = common.accessor_offset_and_pitch(func_attrs["output_accessors"][0], "c")
    shape_code = common.gen_shape_eval_code(dim_info_dict, ["a", "b"], ["c"])
    # an operand broadcasts when it is 2-D or its batch dim is 1 while B > 1
    a_batch = "(*a_dim0)" if ra == 3 else "1"
    b_batch = "(*b_dim0)" if rb == 3 else "1"
    launches = []
    for key, item in func_attrs["exec_path"].items():
        if not item.algo:
            raise RuntimeError(f"{func_name}: workload {key} has no kernel instance; run profiling first")
        program = (
            f'static const int algo = resolve_instance(0, {dtype}, "{item.algo}");\n'
            f"    check_rc(aitamd_bmm_rcr({dtype}, algo, a, b, c, B, M, N, K, lda, ldb, ldc, stride_a, stride_b, "
            f'stride_c, stream), "{func_name}");'
        )
        launches.append(exec_cond_template.format(indent="  ", cond=item.exec_cond, program=program))
    return f"""{common.HEADER}
{_signature(func_name, (ra, rb, rc))} {{
{shape_code}
  const uint16_t* a = static_cast<const uint16_t*>(in_ptr) + {off_a};
  const uint16_t* b = static_cast<const uint16_t*>(weight_ptr) + {off_b};
  uint16_t* c = static_cast<uint16_t*>(out_ptr) + {off_c};
  const int64_t lda = {lda if lda is not None else "K"};
  const int64_t ldb = {ldb if ldb is not None else "K"};
  const int64_t ldc = {ldc if ldc is not None else "N"};
  const int64_t stride_a = ({a_batch} == 1 && B > 1) ? 0 : M * lda;
  const int64_t stride_b = ({b_batch} == 1 && B > 1) ? 0 : N * ldb;
  const int64_t stride_c = M * ldc;
  if (B == 0 || M == 0 || N == 0) return;
{"".join(launches)}
  throw std::runtime_error(
      "Unsupported workload for this bmm_rcr specialization: B=" + std::to_string(B) + " M=" + std::to_string(M) +
      " N=" + std::to_string(N) + " K=" + std::to_string(K));
}}
{common.FOOTER}"""


def func_decl(func_attrs) -> str:
    return _signature(func_attrs["name"], _ranks(func_attrs)) + ";"


def func_call(func_attrs, indent="  ") -> str:
    a, b = func_attrs["inputs"][:2]
    c = func_attrs["outputs"][0]
    dims = []
    for acc in (func_attrs["input_accessors"][0], func_attrs["input_accessors"][1],
                func_attrs["output_accessors"][0]):
        dims += ["&" + d._attrs["name"] for d in acc.original_shapes]
    args = [a._attrs["name"], b._attrs["name"], c._attrs["name"]] + dims + ["stream"]
    return f"{indent}{func_attrs['name']}({', '.join(args)});"


registry.reg("rocm.bmm_rcr.config", _config)
registry.reg("rocm.bmm_rcr.filter", common.gemm_filter)
registry.reg("rocm.bmm_rcr.gen_profiler", common.gemm_gen_profiler)
registry.reg("rocm.bmm_rcr.select_algo", common.gemm_select_algo)
registry.reg("rocm.bmm_rcr.gen_function", gen_function)
registry.reg("rocm.bmm_rcr.func_decl", func_decl)
registry.reg("rocm.bmm_rcr.func_call", func_call)
