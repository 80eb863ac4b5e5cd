"""mem_eff_attention: fused multi-head attention on [batch, heads, seq, head_dim] operands,
softmax(Q K^T / sqrt(head_dim)) V, written as [batch, seq, heads, head_dim_v].

Counterpart of python/aitemplate/compiler/ops/attention/mem_eff_attention.py:49-263 (constructor arguments,
`__call__(q, k, v, lengths_kv=None, lengths_q=None)`, output shape, exec keys, `_get_op_attributes`).  The
reference's ROCm hook (backend/rocm/attention/mem_eff_attention.py) reads the device-side lengths on the host and is
skipped by its own test on ROCm (tests/unittest/ops/test_attention.py:705); the meaning built here is the one that
test states for every backend (test_attention.py:504-523, 593, 661-664): `lengths_kv` [batch, 1] int32 is a key-padding
mask (batch entry b attends to its first lengths_kv[b] keys); rows past `lengths_q` are unspecified there and are
written as zeros here (blocks of query rows that are all padding do no work).  `nn.CrossAttention` uses the fixed-length form (frontend/nn/attention.py:338).
`use_grouped_fmha` selects between two CUDA kernels in the reference and changes nothing here."""
import itertools
from collections import OrderedDict
from typing import Optional

from ....backend import registry
from ....backend.target import Target
from ...base import Operator, Tensor


class mem_eff_attention(Operator):
    def __init__(self, causal, dropout=0, variable_seq_length_kv=False, variable_seq_length_q=False,
                 use_grouped_fmha=False) -> None:
        super().__init__()
        assert dropout == 0
        self._attrs["op"] = "mem_eff_attention"
        self._attrs["has_profiler"] = False
        self._attrs["dropout"] = dropout
        self._attrs["causal"] = causal
        self._attrs["variable_seq_length_kv"] = variable_seq_length_kv
        self._attrs["variable_seq_length_q"] = variable_seq_length_q
        self._attrs["head_size"] = -1
        self._attrs["workspace"] = 0
        self._attrs["use_grouped_fmha"] = use_grouped_fmha

    def _infer_shapes(self, q: Tensor, v: Tensor):
        qs, vs = q._attrs["shape"], v._attrs["shape"]
        # [batch, heads, seq, head_dim] -> [batch, seq, heads, head_dim_v]
        return [qs[0], qs[2], qs[1], vs[-1]]

    def __call__(self, q: Tensor, k: Tensor, v: Tensor, lengths_kv: Optional[Tensor] = None,
                 lengths_q: Optional[Tensor] = None) -> Tensor:
        for t, name in ((q, "q"), (k, "k"), (v, "v")):
            if len(t._attrs["shape"]) != 4:
                raise RuntimeError(f"mem_eff_attention: {name} must be [batch, heads, seq, head_dim]")
        for dim in (1, 3):
            if len(q._attrs["shape"][dim]._attrs["values"]) != 1:
                raise RuntimeError("mem_eff_attention: the number of heads and the head dim must be static")
        if q._attrs["shape"][3] != k._attrs["shape"][3] or k._attrs["shape"][2] != v._attrs["shape"][2]:
            raise RuntimeError("mem_eff_attention: q / k head dims and k / v sequence lengths must agree")
        for t, name in ((k, "k"), (v, "v")):
            if t._attrs["shape"][0] != q._attrs["shape"][0] or t._attrs["shape"][1] != q._attrs["shape"][1]:
                raise RuntimeError(f"mem_eff_attention: batch and heads of {name} differ from q's")
        self._attrs["head_size"] = v._attrs["shape"][3]._attrs["values"][0]
        self._attrs["inputs"] = [q, k, v]
        for flag, lengths, name in ((self._attrs["variable_seq_length_kv"], lengths_kv, "lengths_kv"),
                                    (self._attrs["variable_seq_length_q"], lengths_q, "lengths_q")):
            if flag:
                assert lengths is not None, f"mem_eff_attention: {name} is required"
                if lengths._attrs["dtype"] != "int32":
                    raise RuntimeError(f"mem_eff_attention: {name} must be int32, got {lengths._attrs['dtype']}")
                lshape = lengths._attrs["shape"]
                if lshape[0] != q._attrs["shape"][0] or any(d._attrs["values"] != [1] for d in lshape[1:]):
                    raise RuntimeError(f"mem_eff_attention: {name} must hold one entry per batch ([batch] or [batch, 1])")
                self._attrs["inputs"].append(lengths)
        self._set_depth()
        self._extract_exec_path(q)
        output = Tensor(self._infer_shapes(q, v), src_ops={self}, dtype=q._attrs["dtype"])
        self._attrs["outputs"] = [output]
        return output

    def _get_op_attributes(self):
        # (the reference returns "causal" only, so a copy of a variable-length op loses its flags there)
        return {name: self._attrs[name] for name in ("causal", "variable_seq_length_kv", "variable_seq_length_q",
                                                     "use_grouped_fmha")}

    def _gen_exec_key(self, shape):
        return (f"batch_size == {shape[0]} && num_heads == {shape[1]} && seq_len == {shape[2]} && "
                f"head_sizes == {shape[3]}")

    def _extract_exec_path(self, x: Tensor):
        values = [dim._attrs["values"] for dim in x._attrs["shape"]]
        self._attrs["exec_path"] = OrderedDict((self._gen_exec_key(s), "") for s in itertools.product(*values))

    def gen_function(self) -> str:
        target = Target.current()
        return registry.get(f"{target.name()}.{self._attrs['op']}.gen_function")(self._attrs)
