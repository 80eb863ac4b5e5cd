"""Assign activation-memory offsets to internal tensors and size the shared workspace.

A minimal form of python/aitemplate/compiler/transform/memory_planning.py:155-194: tensors
are packed first-fit by lifetime (a buffer is released after its last consumer ran), 64-byte
aligned; views, parameters and tensors that live in an output buffer take no space.
Returns (blob bytes, workspace bytes)."""
from typing import List, Tuple

from ..base import Tensor
from .mark_param_tensor import storage_root
from .transform_utils import get_sorted_ops

ALIGN = 64


def memory_planning(sorted_graph: List[Tensor]) -> Tuple[int, int]:
    ops = get_sorted_ops(sorted_graph)
    step_of = {id(op): i for i, op in enumerate(ops)}
    need = []  # (tensor, first step, last step, bytes)
    for t in sorted_graph:
        t._attrs["offset"] = None
        if t._attrs["is_param"] or t._attrs["is_output"] or t._attrs["is_view_of"] is not None:
            continue
        if t._attrs["external_tensor"] is not None:
            continue
        first = min((step_of[id(op)] for op in t.src_ops()), default=0)
        last = first
        # consumers of the tensor and of every view of it
        for other in sorted_graph:
            if other is t or storage_root(other) is t:
                for op in other.dst_ops():
                    if id(op) in step_of:
                        last = max(last, step_of[id(op)])
        need.append((t, first, last, t.size_bytes(alignment=ALIGN)))
    placed = []  # (offset, size, first, last)
    blob = 0
    for t, first, last, size in need:
        offset = 0
        for o, s, f, l in sorted(placed):
            overlaps_time = not (last < f or first > l)
            if overlaps_time and offset < o + s and o < offset + size:
                offset = o + s
        t._attrs["offset"] = offset
        placed.append((offset, size, first, last))
        blob = max(blob, offset + size)
    workspace = max((op._attrs.get("workspace", 0) or 0 for op in ops), default=0)
    return blob, workspace
