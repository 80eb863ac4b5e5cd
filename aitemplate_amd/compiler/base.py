"""Graph IR nodes the GEMM-family ops touch: IntVar / IntImm dims, Tensor, Operator.

A thin counterpart of python/aitemplate/compiler/base.py: the constructor
signatures, the `_attrs` dictionaries and the helper methods the ops and the
reference's tests rely on (Tensor :728-830, IntVar :84-305, IntImm :319-371,
Operator :1104-1149, ExecItem / DynamicProfileStrategy :1081-1101) are kept;
symbolic arithmetic, jagged dims and constant-data plumbing that the GEMM path
never reaches are not.
"""
from __future__ import annotations

import copy
import math
from dataclasses import dataclass
from enum import Enum
from pprint import pformat
from typing import Any, Dict, Iterable, List, Optional, Union

from .dtype import get_dtype_size, normalize_dtype


class StableSet:
    """Insertion-ordered set (graphs must be walked deterministically)."""

    def __init__(self, items: Optional[Iterable] = None):
        self._d: Dict[Any, None] = {}
        if items is not None:
            for it in items:
                self._d[it] = None

    def add(self, item):
        self._d[item] = None

    def discard(self, item):
        self._d.pop(item, None)

    def remove(self, item):
        del self._d[item]

    def update(self, items):
        for it in items:
            self._d[it] = None

    def __contains__(self, item):
        return item in self._d

    def __iter__(self):
        return iter(list(self._d.keys()))

    def __len__(self):
        return len(self._d)

    def __bool__(self):
        return bool(self._d)

    def __eq__(self, other):
        if isinstance(other, (StableSet, set, frozenset)):
            return set(self._d.keys()) == set(other)
        return NotImplemented

    def __repr__(self):
        return "StableSet(" + repr(list(self._d.keys())) + ")"

    def __deepcopy__(self, memo):
        return StableSet(copy.deepcopy(list(self._d.keys()), memo))


class Node:
    """Anything in the graph: carries a dictionary of attributes."""

    def __init__(self) -> None:
        self._attrs: Dict[str, Any] = {"name": None, "depth": 0, "nop": False}

    def __str__(self) -> str:
        return pformat(self._attrs, indent=2)

    def __repr__(self) -> str:
        return f"{type(self).__name__}({self._attrs.get('name')})"

    def pseudo_code(self, with_shape: bool = False) -> str:
        raise NotImplementedError()


class IntVar(Node):
    """A dynamic dimension with an inclusive [lower, upper] range."""

    def __init__(self, values: List[int], name: Optional[str] = None, symbolic_value: Any = None) -> None:
        super().__init__()
        self._attrs["name"] = name
        if values is None or len(values) < 2:
            raise RuntimeError(f"IntVar 'values' field must have at least 2 values! values: {values}, name: {name}")
        if min(values) < 0:
            raise RuntimeError(f"IntVar has < 0 value! values: {values}, name: {name}")
        uniq = sorted(set(values))
        if len(uniq) == 1:
            # degenerate range: behaves as a fixed value but keeps two entries
            self._attrs["values"] = uniq * 2
            self._attrs["symbolic_value"] = uniq[0]
        else:
            self._attrs["values"] = uniq
            if symbolic_value is None:
                # named dims are the same symbol wherever the name re-appears; unnamed ones are unique
                symbolic_value = name if name is not None else f"_dim_{id(self)}"
            self._attrs["symbolic_value"] = symbolic_value

    def __eq__(self, another: Any) -> bool:
        return isinstance(another, IntVar) and self._attrs["symbolic_value"] == another._attrs["symbolic_value"]

    def __hash__(self) -> int:
        return hash((self._attrs["name"], tuple(self._attrs["values"]), self._attrs["symbolic_value"]))

    def lower_bound(self) -> int:
        return self._attrs["values"][0]

    def upper_bound(self) -> int:
        return self._attrs["values"][-1]

    def symbolic_value(self):
        return self._attrs["symbolic_value"]

    def pseudo_code(self, with_shape: bool = False) -> str:
        return self._attrs["name"] if self._attrs["name"] is not None else f"IntVar({self._attrs['values']})"

    # conservative interval arithmetic, enough for shape products
    def _combine(self, other, fn):
        ov = other._attrs["values"] if isinstance(other, IntVar) else [int(other)]
        sv = self._attrs["values"]
        cands = [fn(a, b) for a in (sv[0], sv[-1]) for b in (ov[0], ov[-1])]
        lo, hi = min(cands), max(cands)
        return IntImm(lo) if lo == hi else IntVar([lo, hi])

    def __add__(self, other):
        return self._combine(other, lambda a, b: a + b)

    def __mul__(self, other):
        return self._combine(other, lambda a, b: a * b)

    __radd__ = __add__
    __rmul__ = __mul__


class IntImm(IntVar):
    """A static dimension."""

    def __init__(self, value: int, name: Optional[str] = None) -> None:
        if not isinstance(value, int) or isinstance(value, bool):
            raise RuntimeError(f"IntImm only takes an int value! Name: {name}, current value: {value}")
        Node.__init__(self)
        self._attrs["name"] = name
        self._attrs["values"] = [value]
        self._attrs["symbolic_value"] = value

    def __eq__(self, another: Any) -> bool:
        if isinstance(another, int) and not isinstance(another, bool):
            return self.value() == another
        return isinstance(another, IntImm) and self._attrs["values"] == another._attrs["values"]

    def __hash__(self) -> int:
        return hash(("imm", self._attrs["values"][0]))

    def value(self) -> int:
        return self._attrs["values"][0]

    def pseudo_code(self, with_shape: bool = False) -> str:
        return str(self.value())


def wrap_dim(idx: int, rank: int) -> int:
    if idx < 0:
        idx += rank
    if idx < 0 or idx >= rank:
        raise IndexError(f"dim {idx} out of range for rank {rank}")
    return idx


def get_aligned_size(shape: List[IntVar], dtype: str, alignment: int = 64) -> int:
    """Bytes a tensor of (maximum) `shape` occupies, rounded up to `alignment`."""
    size = get_dtype_size(dtype)
    for d in shape:
        size *= d.upper_bound() if isinstance(d, IntVar) else int(d)
    if alignment > 1 and size % alignment != 0:
        size = (size // alignment + 1) * alignment
    return size


class Tensor(Node):
    """A piece of data: input / output of Operators."""

    def __init__(
        self,
        shape: List[Union[int, IntVar]],
        name: Optional[str] = None,
        src_ops: Optional[Iterable[Node]] = None,
        dst_ops: Optional[Iterable[Node]] = None,
        dtype: str = "float16",
        is_input: bool = False,
        is_output: bool = False,
        value: Any = None,
        is_view_of: Any = None,
        is_internal_constant: bool = False,
        skip_constant_folding: bool = False,
        check_nan_and_inf: bool = False,
        check_outputs: bool = False,
        original_name: Optional[str] = None,
    ) -> None:
        super().__init__()
        self._attrs["shape"] = self._convert_shape(shape)
        self._attrs["name"] = name
        self._attrs["src_ops"] = StableSet(src_ops)
        self._attrs["dst_ops"] = StableSet(dst_ops)
        self._attrs["dtype"] = normalize_dtype(dtype)
        self._attrs["is_output"] = is_output
        self._attrs["is_input"] = is_input
        self._attrs["is_param"] = False
        self._attrs["is_internal_constant"] = is_internal_constant
        self._attrs["skip_constant_folding"] = skip_constant_folding
        self._attrs["has_output_aliases"] = False
        self._attrs["external_tensor"] = None
        self._attrs["is_view_of"] = is_view_of
        if is_view_of is not None:
            self._attrs["dtype"] = is_view_of._attrs["dtype"]
        self._attrs["value"] = value
        depths = [op._attrs["depth"] for op in self._attrs["src_ops"]]
        self._attrs["depth"] = max(depths) + 1 if depths else 0
        self._attrs["offset"] = None
        self._attrs["data"] = None
        self._attrs["constant_folding_output_idx"] = None
        self._attrs["check_nan_and_inf"] = check_nan_and_inf
        self._attrs["check_outputs"] = check_outputs
        self._attrs["original_name"] = original_name

    def __str__(self) -> str:
        out = {}
        for key, val in self._attrs.items():
            if key in ("src_ops", "dst_ops") and val is not None:
                out[key] = [x._attrs["name"] for x in val]
            else:
                out[key] = val
        return pformat(out, indent=2)

    @staticmethod
    def _convert_shape(shape) -> List[IntVar]:
        out = []
        for v in shape:
            if isinstance(v, bool):
                raise RuntimeError(f"Unsupported dim type: {type(v)}, dim: {v}")
            if isinstance(v, int):
                out.append(IntImm(v))
            elif isinstance(v, IntVar):
                out.append(v)
            else:
                raise RuntimeError(f"Unsupported dim type: {type(v)}, dim: {v}")
        return out

    def shape(self) -> List[IntVar]:
        return self._attrs["shape"]

    def _rank(self) -> int:
        return len(self._attrs["shape"])

    def _size(self, dim: int) -> IntVar:
        return self._attrs["shape"][wrap_dim(dim, self._rank())]

    def dtype(self) -> str:
        return self._attrs["dtype"]

    def src_ops(self):
        return self._attrs["src_ops"]

    def dst_ops(self):
        return self._attrs["dst_ops"]

    # arithmetic builds element-wise ops (reference: compiler/base.py:958-990)
    def _elementwise(self, func_name: str, lhs, rhs) -> "Tensor":
        from .ops.common.elementwise import elementwise
        from .ops.common.epilogue import FuncEnum

        return elementwise(FuncEnum[func_name])(lhs, rhs)

    def __add__(self, other) -> "Tensor":
        return self._elementwise("ADD", self, other)

    def __radd__(self, other) -> "Tensor":
        return self._elementwise("ADD", other, self)

    def __sub__(self, other) -> "Tensor":
        return self._elementwise("SUB", self, other)

    def __rsub__(self, other) -> "Tensor":
        return self._elementwise("SUB", other, self)

    def __mul__(self, other) -> "Tensor":
        return self._elementwise("MUL", self, other)

    def __rmul__(self, other) -> "Tensor":
        return self._elementwise("MUL", other, self)

    def __truediv__(self, other) -> "Tensor":
        return self._elementwise("DIV", self, other)

    def __rtruediv__(self, other) -> "Tensor":
        return self._elementwise("DIV", other, self)

    def is_a_const_num(self) -> bool:
        return len(self._attrs["shape"]) == 0 and self._attrs["value"] is not None

    def is_jagged(self) -> bool:
        return False

    def size_bytes(self, alignment: int = 1) -> int:
        return get_aligned_size(self._attrs["shape"], self.dtype(), alignment)

    def pseudo_code(self, with_shape: bool = True) -> str:
        args = [f"name={self._attrs['name']}"]
        if with_shape:
            args.append("shape=[" + ", ".join(d.pseudo_code() for d in self._attrs["shape"]) + "]")
        return f"Tensor({', '.join(args)})"

    def _bind_data(self, data: "ConstantTensorData") -> None:
        """Attach constant bytes (weights given to compile_model(constants=...))."""
        if self.src_ops():
            raise ValueError(f"Cannot bind tensor {self._attrs['name']}; it is produced by an op")
        if data.dtype != self._attrs["dtype"]:
            raise ValueError(f"data's dtype did not match: expected {self._attrs['dtype']}, got {data.dtype}")
        if len(data) != self.size_bytes(alignment=1):
            raise ValueError(
                f"ConstantTensor's maximum size is not equal to len(data)! Got {len(data)}, expected "
                f"{self.size_bytes(alignment=1)} bytes."
            )
        self._attrs["data"] = data

    def __deepcopy__(self, memo):
        result = Tensor(self.shape())
        memo[id(self)] = result
        result._attrs = copy.deepcopy(self._attrs, memo)
        return result


class ConstantTensorData:
    """Host bytes of a bound constant."""

    def __init__(self, raw: bytes, dtype: str):
        self.raw = bytes(raw)
        self.dtype = normalize_dtype(dtype)

    def __len__(self) -> int:
        return len(self.raw)

    def to_bytes(self) -> bytes:
        return self.raw

    @staticmethod
    def from_torch(t) -> "ConstantTensorData":
        import torch

        name = {torch.float16: "float16", torch.bfloat16: "bfloat16", torch.float32: "float32",
                torch.int32: "int32", torch.int64: "int64", torch.bool: "bool"}[t.dtype]
        c = t.detach().contiguous().cpu()
        if c.dtype == torch.bfloat16:
            raw = c.view(torch.int16).numpy().tobytes()
        else:
            raw = c.numpy().tobytes()
        return ConstantTensorData(raw, name)


class DynamicProfileStrategy(Enum):
    """Which end of a dynamic range the profiler times (compiler/base.py:1081-1094 of the reference)."""

    MIN = 1
    MAX = 2
    HINTS = 3


@dataclass
class ExecItem:
    """One profiled workload of an op: the key that was timed, the run-time condition that
    selects it, and the kernel instance (algo) that won."""

    profiling_key: str
    exec_cond: str
    algo: str


class Operator(Node):
    """Base of all ops: inputs, profiler flag, depth bookkeeping, deep copy via ctor attributes."""

    def __init__(self) -> None:
        super().__init__()
        self._attrs["inputs"] = None
        self._attrs["has_profiler"] = False

    def __call__(self, *args: List[Tensor]) -> List[Tensor]:
        raise NotImplementedError

    def __deepcopy__(self, memo):
        result = type(self)(**self._get_op_attributes())
        memo[id(self)] = result
        result._attrs = copy.deepcopy(self._attrs, memo)
        return result

    def _set_depth(self) -> None:
        max_d = 0
        if self._attrs["inputs"] is not None:
            for inp in self._attrs["inputs"]:
                max_d = max(max_d, inp._attrs["depth"])
                inp._attrs["dst_ops"].add(self)
        self._attrs["depth"] = max_d

    def __str__(self) -> str:
        out = {}
        for key, val in self._attrs.items():
            if key in ("inputs", "args", "outputs", "original_inputs") and val is not None:
                out[key] = [x._attrs["name"] if isinstance(x, Node) else x for x in val]
            else:
                out[key] = val
        return pformat(out, indent=2)

    def gen_profiler(self, workdir: str = None, dynamic_profiling_strategy=None) -> None:
        return

    def profile(self, workdir="./", devices=None, dynamic_profiling_strategy=DynamicProfileStrategy.MAX) -> None:
        return

    def gen_function(self) -> str:
        raise NotImplementedError("gen_function is not defined for {}".format(self))

    def replace_input_tensor(self, old_tensor, new_tensor) -> None:
        self._attrs["inputs"] = [new_tensor if t is old_tensor else t for t in self._attrs["inputs"]]

    def _get_op_attributes(self) -> Dict[str, Any]:
        """Keyword arguments that re-create this op through its constructor."""
        return {}

    def _inputs_for_pseudo_code(self):
        return self._attrs["inputs"]

    def _outputs_for_pseudo_code(self):
        return self._attrs.get("outputs", [])

    def pseudo_code(self, with_shape: bool = True) -> str:
        ins = ", ".join(t.pseudo_code(with_shape) for t in self._inputs_for_pseudo_code() or [])
        outs = ", ".join(t.pseudo_code(with_shape) for t in self._outputs_for_pseudo_code() or [])
        return f"({outs}) = {self._attrs['op']}({ins})"


def prod_bounds(dims: List[IntVar]):
    """(min, max) of the product of a list of dims."""
    return (math.prod(d.lower_bound() for d in dims), math.prod(d.upper_bound() for d in dims))
