"""Registry hooks of mem_eff_attention.

Takes the place of python/aitemplate/backend/rocm/attention/mem_eff_attention.py:305-365 (`gen_function`,
`func_decl`, `func_call` under the same registry keys).  [batch, heads, seq, head_dim] operands are the
[batch * heads, seq, head_dim] operands of the fused attention kernel, and the op's [batch, seq, heads, head_dim_v]
result is that kernel's permuted store with heads as the group size, so the launcher is one call; the scale is
head_dim ** -0.5 as the reference passes it (mem_eff_attention.py:343).  Key and query lengths stay on the device: the kernel
reads its batch entry's lengths itself (the reference's hook copies nothing either but dereferences the device pointer
on the host, mem_eff_attention.py:181-182)."""
from typing import Any, Dict

from ... import registry
from ..gemm import common


def _signature(func_name: str) -> str:
    return (f"void {func_name}(void* output, const void* q, const void* k, const void* v, const void* lengths_kv, "
            "const void* lengths_q, int64_t* batch_size, int64_t* seq_len, int64_t* seq_len_kv, int num_heads, int head_dim, "
            "int head_dim_v, float softmax_scale, hipStream_t stream)")


def gen_function(func_attrs: Dict[str, Any]) -> str:
    func_name = func_attrs["name"]
    dtype = common.DTYPE_ID[func_attrs["inputs"][0]._attrs["dtype"]]
    causal = 1 if func_attrs["causal"] else 0
    return f"""{common.HEADER}
{_signature(func_name)} {{
  check_rc(aitamd_mem_eff_attention({dtype}, q, k, v, output, *batch_size, num_heads, *seq_len, *seq_len_kv, head_dim,
                                    head_dim_v, softmax_scale, {causal},
                                    static_cast<const int32_t*>(lengths_kv), static_cast<const int32_t*>(lengths_q),
                                    stream), "{func_name}");
}}
{common.FOOTER}"""


def func_decl(func_attrs: Dict[str, Any]) -> str:
    return _signature(func_attrs["name"]) + ";"


def func_call(func_attrs: Dict[str, Any], indent: str = "  ") -> str:
    q, k, v = func_attrs["inputs"][:3]
    extra = [t._attrs["name"] for t in func_attrs["inputs"][3:]]  # lengths_kv, then lengths_q, each if its flag is set
    lengths_kv = extra.pop(0) if func_attrs["variable_seq_length_kv"] else "nullptr"
    lengths_q = extra.pop(0) if func_attrs["variable_seq_length_q"] else "nullptr"
    out = func_attrs["outputs"][0]
    qs, ks, vs = q._attrs["shape"], k._attrs["shape"], v._attrs["shape"]
    heads = qs[1]._attrs["values"][0]
    head_dim = qs[3]._attrs["values"][0]
    head_dim_v = vs[3]._attrs["values"][0]
    scale = head_dim ** (-0.5)
    args = [out._attrs["name"], q._attrs["name"], k._attrs["name"], v._attrs["name"], lengths_kv, lengths_q, "&" + qs[0]._attrs["name"],
            "&" + qs[2]._attrs["name"], "&" + ks[2]._attrs["name"], str(heads), str(head_dim), str(head_dim_v),
            f"{scale!r}f", "stream"]
    return f"{indent}{func_attrs['name']}({', '.join(args)});"


registry.reg("rocm.mem_eff_attention.gen_function", gen_function)
registry.reg("rocm.mem_eff_attention.func_decl", func_decl)
registry.reg("rocm.mem_eff_attention.func_call", func_call)
