"""Graph helpers shared by the passes."""
from typing import List

from ..base import Operator, Tensor


def get_sorted_ops(sorted_graph: List[Tensor]) -> List[Operator]:
    """Operators of a topologically sorted tensor list, each once, in execution order."""
    seen, ops = set(), []
    for t in sorted_graph:
        for op in t.src_ops():
            if id(op) not in seen:
                seen.add(id(op))
                ops.append(op)
    return ops


def is_view_op(op: Operator) -> bool:
    return bool(op._attrs.get("is_view_op", False))
