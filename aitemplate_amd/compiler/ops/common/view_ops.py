"""View ops: reshape (and flatten via reshape) and split along the outermost dim — outputs alias their
input's memory.

Counterpart of the reshape in python/aitemplate/compiler/ops/common/view_ops.py, reduced
to static target shapes with at most one -1 (what the GEMM-family graphs use), and of
python/aitemplate/compiler/ops/tensor/split.py:31-170 for the case that needs no copy."""
from typing import List, Sequence, Union

from ...base import IntImm, IntVar, Operator, Tensor
from ...dtype import get_dtype_size


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


class split(_view):
    """torch.split(x, split_size_or_sections, dim) -> tuple of tensors.

    Only splits that leave every piece contiguous are supported (dim 0, or a dim preceded by dims of
    size 1) with static shapes: each piece is then a view at a byte offset into x and no kernel runs.
    This is the split nn.MultiheadAttention applies to the packed [3, batch, heads, seq, head_dim]
    projection.  The reference materialises every split with a copy kernel unless a later pass removes
    it (split.py:172-214)."""

    def __init__(self):
        super().__init__()
        self._attrs["op"] = "split"
        self._attrs["is_view_op"] = True
        self._attrs["has_profiler"] = False

    def __call__(self, x: Tensor, split_size_or_sections: Union[int, Sequence[int]], dim: int = 0):
        shape = x._attrs["shape"]
        rank = len(shape)
        if rank <= 0:
            raise RuntimeError("expected a non-scalar tensor")
        if not -rank <= dim < rank:
            raise RuntimeError(f"split dim ({dim}) expected to be less than rank ({rank})")
        dim %= rank
        if not all(isinstance(d, IntImm) for d in shape):
            raise NotImplementedError("split needs static shapes on this backend")
        if any(d.value() != 1 for d in shape[:dim]):
            raise NotImplementedError("split along an inner dim would need a copy kernel; only dim 0 "
                                      "(or a dim behind dims of size 1) is supported")
        size = shape[dim].value()
        if isinstance(split_size_or_sections, (list, tuple)):
            sizes = [int(v.value()) if isinstance(v, IntImm) else int(v) for v in split_size_or_sections]
            if len(sizes) < 1:
                raise RuntimeError(f"the number of splits expected >=0 but got {len(sizes)}")
            if sum(sizes) != size:
                raise RuntimeError(f"sum of split_sizes ({sizes}) does not match split_dim_size ({size})")
        else:
            step = split_size_or_sections.value() if isinstance(split_size_or_sections, IntImm) \
                else split_size_or_sections
            if not isinstance(step, int):
                raise RuntimeError("split_size expected to be of int")
            if size == 0:
                sizes = [0]
            else:
                if step <= 0:
                    raise RuntimeError("split_size expected to be > 0")
                sizes = [step] * (size // step) + ([size % step] if size % step else [])
        self._attrs["inputs"] = [x]
        self._attrs["split_dim"] = dim
        self._attrs["split_sizes"] = sizes
        self._set_depth()
        inner = get_dtype_size(x.dtype())
        for d in shape[dim + 1:]:
            inner *= d.value()
        outputs, start = [], 0
        for n in sizes:
            out_shape = list(shape[:dim]) + [IntImm(n)] + list(shape[dim + 1:])
            t = Tensor(out_shape, src_ops={self}, is_view_of=x, dtype=x.dtype())
            t._attrs["view_offset_bytes"] = start * inner
            outputs.append(t)
            start += n
        self._attrs["outputs"] = outputs
        return tuple(outputs)

    def _get_op_attributes(self):
        return {}
