"""Classify tensors: parameters (graph inputs / constants), outputs, and the storage each
tensor uses once views are resolved.

Counterpart of python/aitemplate/compiler/transform/mark_param_tensor.py:52-72 plus the
alias handling of backend/codegen.py:620-642: a view shares the memory of the tensor it
views; if any member of such an alias group is a graph output, the whole group lives in
that output's buffer (this is how bmm_softmax_bmm_permute writes straight into the reshaped
output)."""
from typing import Dict, List

from ..base import Tensor


def storage_root(t: Tensor) -> Tensor:
    while t._attrs["is_view_of"] is not None:
        t = t._attrs["is_view_of"]
    return t


def storage_offset_bytes(t: Tensor) -> int:
    """Byte offset of `t` inside its storage root (non-zero below a split view)."""
    off = 0
    while t._attrs["is_view_of"] is not None:
        off += int(t._attrs.get("view_offset_bytes", 0) or 0)
        t = t._attrs["is_view_of"]
    return off


def mark_param_tensor(sorted_graph: List[Tensor], output_tensors: List[Tensor] = None) -> None:
    """Sets is_param, and for every tensor that does not own its memory
    `external_tensor` = the tensor whose buffer it uses:
      * views of an input / constant use that parameter's memory,
      * a group containing graph outputs lives in its first output's buffer, unless that output covers
        only a part of the group's memory (it sits below a split): then the group keeps its own buffer
        and the outputs are copied out after the ops ran,
      * otherwise views use the memory-planned buffer of the tensor they view."""
    for t in sorted_graph:
        if not t.src_ops():
            t._attrs["is_param"] = True  # input or constant
    order = {id(t): i for i, t in enumerate(output_tensors or [])}
    groups: Dict[int, List[Tensor]] = {}
    for t in sorted_graph:
        groups.setdefault(id(storage_root(t)), []).append(t)
    for members in groups.values():
        root = storage_root(members[0])
        outs = sorted((m for m in members if m._attrs["is_output"]), key=lambda m: order.get(id(m), 1 << 30))
        partial = any(storage_offset_bytes(m) != 0 or m.size_bytes() != root.size_bytes() for m in members)
        if root._attrs["is_param"] or not outs or partial:
            owner = root
        else:
            owner = outs[0]
        for m in members:
            m._attrs["external_tensor"] = None if m is owner else owner
            m._attrs["has_output_aliases"] = (m is not owner) and owner._attrs["is_output"] and not m._attrs["is_output"]
