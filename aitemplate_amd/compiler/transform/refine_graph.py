"""Let ops with the same signature share one generated function.

Counterpart of python/aitemplate/compiler/transform/refine_graph.py:31-100: two ops are
interchangeable when op type, attributes that reach the generated code, input / output
dtypes and shapes, and profiled instances agree; the later op then takes the earlier op's
function name and keeps its own `original_name`."""
from typing import List

from ..base import IntImm, Tensor
from .transform_utils import get_sorted_ops


def _shape_sig(t: Tensor):
    return tuple((tuple(d._attrs["values"])) for d in t._attrs["shape"])


def _signature(op):
    a = op._attrs
    parts = [a["op"], a.get("scale"), tuple(a["shape"]) if isinstance(a.get("shape"), (tuple, list)) else a.get("shape"),
             a.get("layout")]
    for t in a.get("inputs") or []:
        parts.append((t.dtype(), _shape_sig(t)))
    for t in a.get("outputs") or []:
        parts.append((t.dtype(), _shape_sig(t)))
    for acc in (a.get("input_accessors") or []) + (a.get("output_accessors") or []):
        parts.append((getattr(acc, "offset", 0), tuple(_s(d) for d in (acc.actual_shapes or []))))
    for key, item in (a.get("exec_path") or {}).items():
        parts.append((key, item.exec_cond, item.algo))
    return repr(parts)


def _s(d):
    return tuple(d._attrs["values"])


def refine_graph(sorted_graph: List[Tensor]) -> None:
    seen = {}
    for op in get_sorted_ops(sorted_graph):
        if not op._attrs.get("has_profiler"):
            continue
        sig = _signature(op)
        if sig in seen:
            op._attrs["name"] = seen[sig]
        else:
            seen[sig] = op._attrs["name"]
