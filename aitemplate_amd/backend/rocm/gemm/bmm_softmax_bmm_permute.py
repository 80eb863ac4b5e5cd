"""Registry hooks of bmm_softmax_bmm_permute, its causal variant and bmm_softmax_bmm.

Replaces python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:32-388.  The launcher
keeps the reference's shape: the 4th pointer is V, the dim pointers cover Q, K and the [B, M, O]
result, and a trailing `const int p_dim0` carries the number of heads."""
from collections import OrderedDict
from typing import Any, Dict

from ... import registry
from ...target import Target
from . import common

# bmm_softmax_bmm (reference hooks: backend/rocm/gemm/bmm_softmax_bmm.py) is the one-head case of the same launcher
_OPS = ("bmm_softmax_bmm_permute", "bmm_softmax_bmm_permute_causal", "bmm_softmax_bmm")
_INSTANCE = "attention_q128"


def _config(func_attrs, dtype="float16"):
    if dtype not in common.DTYPE_ID:
        raise NotImplementedError(f"the gfx950 attention kernel supports float16 and bfloat16, not {dtype}")
    func_attrs["op_instance"] = OrderedDict([(_INSTANCE, 0)])
    func_attrs["profiler_args"] = ["attn", "bmm_softmax_bmm_permute", str(common.DTYPE_ID[dtype])]


def _filter(instance_name, func_attrs, ab_alignment) -> bool:
    return True


def _select_algo(func_attrs, exec_key) -> str:
    return _INSTANCE


def _signature(func_name: str) -> str:
    ptrs = ["void* in_ptr", "void* weight_ptr", "void* out_ptr", "void* bias_ptr"]
    dims = [f"int64_t* {n}" for prefix in "abc" for n in common.dim_param_names(prefix, 3)]
    return f"void {func_name}({', '.join(ptrs + dims + ['const int p_dim0', 'hipStream_t stream'])})"


def gen_function(func_attrs: Dict[str, Any], exec_cond_template: str, dim_info_dict) -> str:
    func_name = func_attrs["name"]
    dtype = common.DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    causal = 1 if func_attrs["op"].endswith("_causal") else 0
    scale = float(func_attrs["scale"])
    for acc in func_attrs["input_accessors"] + func_attrs["output_accessors"]:
        if getattr(acc, "actual_shapes", None) is not None or getattr(acc, "offset", 0):
            raise NotImplementedError("bmm_softmax_bmm_permute operands must be contiguous tensors")
    conds = " || ".join(f"({item.exec_cond})" for item in func_attrs["exec_path"].values()) or "true"
    return f"""{common.HEADER}
{_signature(func_name)} {{
  const int64_t B = *a_dim0;
  const int64_t M = *a_dim1;
  const int64_t K = *a_dim2;
  const int64_t N = *b_dim1;
  const int64_t O = *c_dim2;
  *c_dim0 = B;
  *c_dim1 = M;
  if (!({conds})) {{
    throw std::runtime_error(
        "Unsupported workload for this bmm_softmax_bmm_permute specialization: B=" + std::to_string(B) +
        " M=" + std::to_string(M) + " N=" + std::to_string(N) + " K=" + std::to_string(K) + " O=" + std::to_string(O));
  }}
  // in_ptr = Q [B,M,K], weight_ptr = K [B,N,K], bias_ptr = V [B,N,O]; out is written as [B/heads, M, heads, O]
  check_rc(aitamd_bmm_softmax_bmm_permute({dtype}, in_ptr, weight_ptr, bias_ptr, out_ptr, B, M, N, K, O, p_dim0,
                                          {scale!r}f, {causal}, stream), "{func_name}");
}}
{common.FOOTER}"""


def func_decl(func_attrs) -> str:
    return _signature(func_attrs["name"]) + ";"


def func_call(func_attrs, indent="  ") -> str:
    q, k, v = func_attrs["inputs"]
    out = func_attrs["outputs"][0]
    dims = []
    for acc in (func_attrs["input_accessors"][0], func_attrs["input_accessors"][1],
                func_attrs["output_accessors"][0]):
        dims += ["&" + d._attrs["name"] for d in acc.original_shapes]
    args = [q._attrs["name"], k._attrs["name"], out._attrs["name"], v._attrs["name"]] + dims
    args += [str(int(func_attrs["shape"][0])), "stream"]
    return f"{indent}{func_attrs['name']}({', '.join(args)});"


for _op in _OPS:
    registry.reg(f"rocm.{_op}.config", _config)
    registry.reg(f"rocm.{_op}.filter", _filter)
    registry.reg(f"rocm.{_op}.gen_profiler", lambda a, w, f, d: common.place_profiler(a, w, f))
    registry.reg(f"rocm.{_op}.select_algo", _select_algo)
    registry.reg(f"rocm.{_op}.gen_function", gen_function)
    registry.reg(f"rocm.{_op}.func_decl", func_decl)
    registry.reg(f"rocm.{_op}.func_call", func_call)
