"""Topological order of all tensors reachable from the outputs
(counterpart of python/aitemplate/compiler/transform/toposort.py)."""
from typing import List, Union

from ..base import Tensor


def toposort(outputs: Union[Tensor, List[Tensor]]) -> List[Tensor]:
    if isinstance(outputs, Tensor):
        outputs = [outputs]
    order: List[Tensor] = []
    state = {}

    def visit(t: Tensor):
        stack = [(t, False)]
        while stack:
            node, expanded = stack.pop()
            if expanded:
                if state.get(id(node)) != 2:
                    state[id(node)] = 2
                    order.append(node)
                continue
            if state.get(id(node)) == 2:
                continue
            if state.get(id(node)) == 1:
                continue
            state[id(node)] = 1
            stack.append((node, True))
            for op in node.src_ops():
                for inp in reversed(op._attrs["inputs"] or []):
                    if state.get(id(inp)) is None:
                        stack.append((inp, False))

    for out in outputs:
        visit(out)
    return order
