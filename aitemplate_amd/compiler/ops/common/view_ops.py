"""View ops: reshape (and flatten via reshape) — outputs alias their input's memory.

Counterpart of the reshape in python/aitemplate/compiler/ops/common/view_ops.py, reduced
to static target shapes with at most one -1 (what the GEMM-family graphs use)."""
from typing import List, Union

from ...base import IntImm, IntVar, Operator, Tensor


class _view(Operator):
    """Marker base: the op moves no data."""

    def gen_function(self) -> str:
        return ""


class reshape(_view):
    def __init__(self):
        super().__init__()
        self._attrs["op"] = "reshape"
        self._attrs["is_view_op"] = True

    @staticmethod
    def _resolve(in_shape: List[IntVar], new_shape: List[Union[int, IntVar]]) -> List[IntVar]:
        out = [IntImm(d) if isinstance(d, int) else d for d in new_shape]
        unknown = [i for i, d in enumerate(out) if isinstance(d, IntImm) and d.value() == -1]
        if len(unknown) > 1:
            raise RuntimeError("reshape accepts at most one -1")
        if unknown:
            if not all(isinstance(d, IntImm) for d in in_shape) or not all(
                    isinstance(d, IntImm) for i, d in enumerate(out) if i != unknown[0]):
                raise RuntimeError("reshape with -1 needs static shapes")
            total = 1
            for d in in_shape:
                total *= d.value()
            known = 1
            for i, d in enumerate(out):
                if i != unknown[0]:
                    known *= d.value()
            if known == 0 or total % known != 0:
                raise RuntimeError(f"cannot reshape {in_shape} to {new_shape}")
            out[unknown[0]] = IntImm(total // known)
        # static element counts must agree
        if all(isinstance(d, IntImm) for d in in_shape) and all(isinstance(d, IntImm) for d in out):
            a = 1
            for d in in_shape:
                a *= d.value()
            b = 1
            for d in out:
                b *= d.value()
            if a != b:
                raise RuntimeError(f"cannot reshape {[d.value() for d in in_shape]} to {[d.value() for d in out]}")
        return out

    def __call__(self, x: Tensor, shape: List[Union[int, IntVar]]) -> Tensor:
        self._attrs["inputs"] = [x]
        self._attrs["shape"] = shape
        self._set_depth()
        out_shape = self._resolve(x._attrs["shape"], shape)
        output = Tensor(out_shape, src_ops={self}, is_view_of=x, dtype=x.dtype())
        self._attrs["outputs"] = [output]
        return output

    def _get_op_attributes(self):
        return {}


class flatten(reshape):
    def __init__(self, start_dim: int = 0, end_dim: int = -1):
        super().__init__()
        self._attrs["op"] = "flatten"
        self._attrs["start"] = start_dim
        self._attrs["end"] = end_dim

    def __call__(self, x: Tensor) -> Tensor:
        rank = x._rank()
        s = self._attrs["start"] % rank
        e = self._attrs["end"] % rank
        shape = x.shape()
        merged = shape[s]
        for d in shape[s + 1:e + 1]:
            merged = merged * d
        return super().__call__(x, shape[:s] + [merged] + shape[e + 1:])

    def _get_op_attributes(self):
        return {"start_dim": self._attrs["start"], "end_dim": self._attrs["end"]}
