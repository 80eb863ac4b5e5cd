"""Give every op, tensor and dim a unique C++-safe name.

Follows the reference's scheme (python/aitemplate/compiler/transform/name_graph.py:51-125):
ops `<op>_<n>`, op outputs `<func>_<k>`, unnamed graph inputs `tensor_<n>`, unnamed dims
`<tensor>_dim_<i>`; user names are sanitised with re.sub(r"\\W|^(?=\\d)", "_", name)."""
import re
from typing import List

from ..base import IntImm, Tensor
from .transform_utils import get_sorted_ops

_counters = {"func": 0, "tensor": 0}


def reset_name_counters() -> None:
    _counters["func"] = 0
    _counters["tensor"] = 0


def valid_c_name(name: str) -> str:
    return re.sub(r"\W|^(?=\d)", "_", name)


def name_graph(sorted_graph: List[Tensor]) -> None:
    used = set()

    def unique(name: str) -> str:
        base, n, i = name, name, 0
        while n in used:
            i += 1
            n = f"{base}_{i}"
        used.add(n)
        return n

    # user-given tensor names first: they are part of the model's interface
    for t in sorted_graph:
        if t._attrs["name"] is not None:
            if t._attrs["original_name"] is None:
                t._attrs["original_name"] = t._attrs["name"]
            t._attrs["name"] = valid_c_name(t._attrs["name"])
            if t._attrs["name"] in used and (t._attrs["is_input"] or t._attrs["is_output"]):
                raise RuntimeError(f"duplicate tensor name {t._attrs['name']}")
            used.add(t._attrs["name"])
    for op in get_sorted_ops(sorted_graph):
        if op._attrs["name"] is None:
            op._attrs["name"] = unique(f"{op._attrs['op']}_{_counters['func']}")
            _counters["func"] += 1
        else:
            op._attrs["name"] = valid_c_name(op._attrs["name"])
        if "original_name" not in op._attrs or op._attrs.get("original_name") is None:
            op._attrs["original_name"] = op._attrs["name"]
        for k, out in enumerate(op._attrs.get("outputs") or []):
            if out._attrs["name"] is None:
                out._attrs["name"] = unique(f"{op._attrs['name']}_{k}")
    for t in sorted_graph:
        if t._attrs["name"] is None:
            t._attrs["name"] = unique(f"tensor_{_counters['tensor']}")
            _counters["tensor"] += 1
    # dims: an IntVar object shared by several tensors is named once
    dim_names = set()
    for t in sorted_graph:
        for i, d in enumerate(t._attrs["shape"]):
            if d._attrs["name"] is None:
                d._attrs["name"] = f"{t._attrs['name']}_dim_{i}"
            else:
                d._attrs["name"] = valid_c_name(d._attrs["name"])
            dim_names.add(d._attrs["name"])
    # dims that only an accessor still holds: the shape of a tensor that a split / concatenate fusion took out of
    # the graph (the op reads or writes a view of a wider tensor, and its launcher is handed the view's dims)
    for op in get_sorted_ops(sorted_graph):
        for kind in ("input_accessors", "output_accessors"):
            for k, acc in enumerate(op._attrs.get(kind) or []):
                for i, d in enumerate(acc.original_shapes):
                    if d._attrs["name"] is None:
                        d._attrs["name"] = unique(f"{op._attrs['name']}_{kind[:-10]}{k}_dim_{i}")
                    dim_names.add(d._attrs["name"])
    clash = dim_names & {t._attrs["name"] for t in sorted_graph}
    if clash:
        raise RuntimeError(f"dim names collide with tensor names: {sorted(clash)}")
