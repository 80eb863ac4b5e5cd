"""Registry hooks of the batched GEMMs (bmm_rcr, bmm_rrr, bmm_ccr, bmm_crr, their *_permute forms) and gemm_rrr.  Replaces python/aitemplate/backend/rocm/gemm/bmm_rcr.py:27-182,
bmm_rcr_permute.py and bmm_common.py:22-363 / bmm_permute_common.py:22-80: same launcher signature (3-D dim
pointers; bmm_rcr_permute adds `const int p_dim0` = d1 before the stream), batch strides derived from the
operand ranks (a 2-D or batch-1 operand broadcasts with stride 0)."""
from typing import Any, Dict

from ... import registry
from . import common


from .... import _kernels
from ....compiler.ops.gemm_universal.gemm_common import gemm_inverse_key_func
from ...target import Target

# op -> operand layout ("r": K-contiguous A / [K, N] B; "c": [K, M] A / K-contiguous B), as in
# python/aitemplate/backend/rocm/gemm/layout.py
LAYOUT_OF_OP = {"bmm_rcr": "rcr", "bmm_rcr_permute": "rcr", "bmm_rrr": "rrr", "bmm_rrr_permute": "rrr",
                "bmm_ccr": "ccr", "bmm_crr": "crr", "gemm_rrr": "rrr",
                "bmm_rrr_add": "rrr", "bmm_ccr_add": "ccr", "bmm_crr_add": "crr"}


def _is_add(func_attrs) -> bool:
    return func_attrs["op"].endswith("_add")


def _epi(func_attrs) -> int:
    return _kernels.EPI_ADD if _is_add(func_attrs) else 0


def _layout(func_attrs):
    lay = LAYOUT_OF_OP[func_attrs["op"]]
    return lay, lay[0] == "c", lay[1] == "r"


def _pitches(func_attrs, m, n, k):
    _, a_col, b_row = _layout(func_attrs)
    return (m if a_col else k), (n if b_row else k)


def _config(func_attrs, dtype="float16"):
    common.gemm_config(func_attrs, dtype, "bmm")


def _config_layout(func_attrs, dtype="float16"):
    common.gemm_config(func_attrs, dtype, "gemm_layout" if func_attrs["op"].startswith("gemm_") else "bmm_layout")


def _filter(instance_name, func_attrs, ab_alignment) -> bool:
    """True when the instance has a kernel for the op's layout and can run every profiled workload."""
    lib = _kernels.load()
    dtype = common.DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    lay = _kernels.LAYOUT_ID[_layout(func_attrs)[0]]
    algo = func_attrs["op_instance"][instance_name]
    dyn_a, dyn_b = _dynamic_pitch(func_attrs)
    for key in func_attrs["exec_path"]:
        m, n, k = gemm_inverse_key_func(key)[-3:]
        lda, ldb = _pitches(func_attrs, m, n, k)
        # a pitch that follows a dynamic dim can take any value at run time: only instances that need no
        # pitch alignment qualify (asked for with an odd pitch)
        lda = lda | 1 if dyn_a else lda
        ldb = ldb | 1 if dyn_b else ldb
        if not lib.aitamd_gemm_algo_supported_layout(_epi(func_attrs), dtype, lay, algo, m, n, k, lda, ldb,
                                                     max(2, min(16, ab_alignment * 2))):
            return False
    return True


def _dynamic_pitch(func_attrs):
    """(A, B): True when the operand's row pitch (its innermost dim) has more than one possible value."""
    def last_dim_is_dynamic(tensor):
        return len(tensor._attrs["shape"][-1]._attrs["values"]) > 1
    return last_dim_is_dynamic(func_attrs["inputs"][0]), last_dim_is_dynamic(func_attrs["inputs"][1])


def _select_algo(func_attrs, exec_key) -> str:
    lib = _kernels.load()
    dtype = common.DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    lay = _kernels.LAYOUT_ID[_layout(func_attrs)[0]]
    dims = gemm_inverse_key_func(exec_key)
    m, n, k = dims[-3:]
    batch = dims[0] if len(dims) == 4 else 1
    lda, ldb = _pitches(func_attrs, m, n, k)
    algo = lib.aitamd_gemm_heuristic_algo_layout(_epi(func_attrs), dtype, lay, batch, m, n, k, lda, ldb, 16)
    all_names = _kernels.gemm_algo_names(_epi(func_attrs), dtype)
    if algo >= 0 and all_names[algo] in func_attrs["op_instance"]:
        return all_names[algo]
    return Target.current().select_minimal_algo(list(func_attrs["op_instance"].keys()))


def _signature(func_name: str, ranks, permute: bool = False, add: bool = False) -> str:
    # the residual of the *_add ops travels as `bias_ptr`, as in the reference (backend/rocm/gemm/common.py:135-137)
    ptrs = ["void* in_ptr", "void* weight_ptr", "void* out_ptr"] + (["void* bias_ptr"] if add else [])
    dims = [f"int64_t* {n}" for prefix, r in zip("abc", ranks) for n in common.dim_param_names(prefix, r)]
    pdims = ["const int p_dim0"] if permute else []
    return f"void {func_name}({', '.join(ptrs + dims + pdims + ['hipStream_t stream'])})"


def _is_permute(func_attrs) -> bool:
    return func_attrs["op"].endswith("_permute")


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
    if "B" not in dim_info_dict:  # gemm_rrr: one batch
        shape_code = "  const int64_t B = 1;\n" + shape_code
    layout, a_col, b_row = _layout(func_attrs)
    # an operand broadcasts when it is 2-D or its batch dim is 1 while B > 1
    a_batch = "(*a_dim0)" if ra == 3 else "1"
    b_batch = "(*b_dim0)" if rb == 3 else "1"
    permute = _is_permute(func_attrs)
    if permute and (off_c or ldc is not None):
        raise NotImplementedError(f"{func_attrs['op']} writes a contiguous permuted buffer; its output cannot be a view")
    plain_rcr = layout == "rcr" and not permute
    add = _is_add(func_attrs)
    epi = _epi(func_attrs)
    ldd = "N"
    if add:
        off_d, pitch_d = common.accessor_offset_and_pitch(func_attrs["input_accessors"][2], "d0")
        if off_d:
            raise NotImplementedError(f"{func_attrs['op']}: the residual cannot be an offset view")
        if pitch_d is not None:
            ldd = str(pitch_d)
    launches = []
    for key, item in func_attrs["exec_path"].items():
        if not item.algo:
            raise RuntimeError(f"{func_name}: workload {key} has no kernel instance; run profiling first")
        if add:
            call = (f"aitamd_bmm_add({_kernels.LAYOUT_ID[layout]}, {dtype}, algo, a, b, bias_ptr, c, B, M, N, K, lda, ldb, "
                    f"ldc, {ldd}, stride_a, stride_b, stride_c, M * {ldd}, stream)")
        elif plain_rcr:
            call = (f"aitamd_bmm_rcr({dtype}, algo, a, b, c, B, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, "
                    "stream)")
        elif layout == "rcr":
            call = (f"aitamd_bmm_rcr_permute({dtype}, algo, a, b, c, B, M, N, K, lda, ldb, stride_a, stride_b, p_dim0, "
                    "stream)")
        else:
            call = (f"aitamd_bmm({_kernels.LAYOUT_ID[layout]}, {dtype}, algo, a, b, c, B, M, N, K, lda, ldb, ldc, "
                    f"stride_a, stride_b, stride_c, {'p_dim0' if permute else '0'}, stream)")
        program = (
            f'static const int algo = resolve_instance({epi}, {dtype}, "{item.algo}");\n'
            f'    check_rc({call}, "{func_name}");'
        )
        launches.append(exec_cond_template.format(indent="  ", cond=item.exec_cond, program=program))
    return f"""{common.header_with_table(epi, dtype)}
{_signature(func_name, (ra, rb, rc), permute, add)} {{
{shape_code}
  const uint16_t* a = static_cast<const uint16_t*>(in_ptr) + {off_a};
  const uint16_t* b = static_cast<const uint16_t*>(weight_ptr) + {off_b};
  uint16_t* c = static_cast<uint16_t*>(out_ptr) + {off_c};
  const int64_t lda = {lda if lda is not None else ("M" if a_col else "K")};
  const int64_t ldb = {ldb if ldb is not None else ("N" if b_row else "K")};
  const int64_t ldc = {ldc if ldc is not None else "N"};
  const int64_t stride_a = ({a_batch} == 1 && B > 1) ? 0 : {"K" if a_col else "M"} * lda;
  const int64_t stride_b = ({b_batch} == 1 && B > 1) ? 0 : {"K" if b_row else "N"} * ldb;
  const int64_t stride_c = M * ldc;
  if (B == 0 || M == 0 || N == 0) return;
{"".join(launches)}
  throw std::runtime_error(
      "Unsupported workload for this {func_attrs["op"]} specialization: B=" + std::to_string(B) + " M=" + std::to_string(M) +
      " N=" + std::to_string(N) + " K=" + std::to_string(K));
}}
{common.FOOTER}"""


def func_decl(func_attrs) -> str:
    return _signature(func_attrs["name"], _ranks(func_attrs), _is_permute(func_attrs), _is_add(func_attrs)) + ";"


def func_call(func_attrs, indent="  ") -> str:
    a, b = func_attrs["inputs"][:2]
    c = func_attrs["outputs"][0]
    dims = []
    for acc in (func_attrs["input_accessors"][0], func_attrs["input_accessors"][1],
                func_attrs["output_accessors"][0]):
        dims += ["&" + d._attrs["name"] for d in acc.original_shapes]
    pdims = [str(int(func_attrs["shape"][0]))] if _is_permute(func_attrs) else []
    extra = [func_attrs["inputs"][2]._attrs["name"]] if _is_add(func_attrs) else []
    args = [a._attrs["name"], b._attrs["name"], c._attrs["name"]] + extra + dims + pdims + ["stream"]
    return f"{indent}{func_attrs['name']}({', '.join(args)});"


def _config_permute(func_attrs, dtype="float16"):
    common.gemm_config(func_attrs, dtype, "bmm_permute")


for _op in LAYOUT_OF_OP:
    if _op == "bmm_rcr":
        _cfg = _config
    elif _op == "bmm_rcr_permute":
        _cfg = _config_permute
    else:
        _cfg = _config_layout
    registry.reg(f"rocm.{_op}.config", _cfg)
    registry.reg(f"rocm.{_op}.filter", _filter)
    registry.reg(f"rocm.{_op}.gen_profiler", common.gemm_gen_profiler)
    registry.reg(f"rocm.{_op}.select_algo", _select_algo)
    registry.reg(f"rocm.{_op}.gen_function", gen_function)
    registry.reg(f"rocm.{_op}.func_decl", func_decl)
    registry.reg(f"rocm.{_op}.func_call", func_call)
