"""View ops: reshape (and flatten via reshape), split and concatenate — ops that move no data on this
backend wherever a GEMM-family op can take the piece as a view, and `strided_copy`, the row copy that the
strided-view pass puts in their place where none can.

Counterpart of the reshape in python/aitemplate/compiler/ops/common/view_ops.py, reduced
to static target shapes with at most one -1 (what the GEMM-family graphs use), of
python/aitemplate/compiler/ops/tensor/split.py:31-170 and of
python/aitemplate/compiler/ops/tensor/concatenate.py:31-170 for the cases that need no copy:
an outer-dim split is a byte offset into its input; a last-dim split or concatenate only
exists until the strided-view pass has turned it into offsets and row pitches of the GEMM
ops on either side (the reference's transform_strided_ops.py does the same, and falls back
to a copy kernel, as the strided-view pass here falls back to `strided_copy`)."""
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

    Two kinds of split run no kernel here.  A split that leaves every piece contiguous (dim 0, or a
    dim preceded by dims of size 1, static shapes) makes each piece a view at a byte offset into x:
    the split nn.MultiheadAttention applies to the packed [3, batch, heads, seq, head_dim]
    projection.  A split along the last dim makes pieces that are strided views (`strided_view_of`
    = (x, dim, first element)); every consumer has to be an op that can read an operand through an
    offset and a row pitch, and the strided-view pass of compile_model rewires them to x.  Every other
    piece (a split along a middle dim, a piece that is a graph output or feeds an op that reads contiguous
    tensors only) becomes a `strided_copy` in that pass.  The reference materialises every split with a
    copy kernel unless a later pass removes it (split.py:172-214)."""

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
        if not all(isinstance(d, IntImm) for d in shape[dim:]):
            raise NotImplementedError("split needs static shapes from the split dim on")
        contiguous = all(isinstance(d, IntImm) and d.value() == 1 for d in shape[:dim])
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
            if contiguous:
                t._attrs["view_offset_bytes"] = start * inner
            else:
                t._attrs["strided_view_of"] = (x, dim, start)
            outputs.append(t)
            start += n
        self._attrs["outputs"] = outputs
        return tuple(outputs)

    def _get_op_attributes(self):
        return {}


class concatenate(_view):
    """torch.cat(tensors, dim).

    The op is a placeholder: the strided-view pass of compile_model makes every GEMM-family producer of a
    last-dim concatenate write its columns of the output directly (offset + row pitch of its C accessor),
    gives every other input (a graph input, a constant, a tensor with other consumers, any input of a
    concatenate along another dim) a `strided_copy` into its rows of the output, as the reference's copy
    kernel does (backend/rocm/tensor/concatenate.py), and drops the op."""

    def __init__(self):
        super().__init__()
        self._attrs["op"] = "concatenate"
        self._attrs["is_view_op"] = True
        self._attrs["has_profiler"] = False

    def __call__(self, inputs: Sequence[Tensor], dim: int = -1) -> Tensor:
        inputs = list(inputs)
        if len(inputs) < 1:
            raise RuntimeError("concatenate expects at least one tensor")
        rank = inputs[0]._rank()
        if not -rank <= dim < rank:
            raise RuntimeError(f"concatenate dim ({dim}) expected to be less than rank ({rank})")
        dim %= rank
        first = inputs[0]._attrs["shape"]
        if not all(isinstance(d, IntImm) for d in first[dim + 1:]):
            raise NotImplementedError("concatenate needs static shapes behind the concatenated dim")
        total = 0
        for t in inputs:
            shape = t._attrs["shape"]
            if len(shape) != rank:
                raise RuntimeError("concatenate expects tensors of the same rank")
            if t.dtype() != inputs[0].dtype():
                raise RuntimeError("concatenate expects tensors of the same dtype")
            for i, (d0, d1) in enumerate(zip(first, shape)):
                if i != dim and d0 != d1:
                    raise RuntimeError(f"concatenate: dim {i} differs between inputs ({d0} vs {d1})")
            if not isinstance(shape[dim], IntImm):
                raise NotImplementedError("concatenate needs a static size along the concatenated dim")
            total += shape[dim].value()
        self._attrs["inputs"] = inputs
        self._attrs["concat_dim"] = dim
        self._set_depth()
        out_shape = list(first[:dim]) + [IntImm(total)] + list(first[dim + 1:])
        output = Tensor(out_shape, src_ops={self}, dtype=inputs[0].dtype())
        self._attrs["outputs"] = [output]
        return output

    def _get_op_attributes(self):
        return {}


def copy_geometry(func_attrs):
    """(full tensor, piece tensor, row bytes, pitch bytes of the full tensor, byte offset into it) of a
    strided_copy op."""
    src, dst = func_attrs["inputs"][0], func_attrs["outputs"][0]
    full, piece = (src, dst) if func_attrs["copy_kind"] == "slice" else (dst, src)
    dim = func_attrs["copy_dim"]
    inner = get_dtype_size(full.dtype())
    for d in full._attrs["shape"][dim + 1:]:
        inner *= d.value()
    length = piece._attrs["shape"][dim].value()
    return full, piece, length * inner, full._attrs["shape"][dim].value() * inner, func_attrs["copy_start"] * inner


class strided_copy(Operator):
    """One piece of a split copied out of its input ("slice"), or one input of a concatenate copied into
    its place in the output ("place"): rows of `length * inner` elements, `full * inner` elements apart on
    the strided side, where inner is the product of the dims behind `dim`.  Created by the strided-view
    pass only; one launch of the library's row copy.  Stands for the reference's split and concatenate
    kernels (python/aitemplate/backend/common/split_common.py, concatenate_common.py)."""

    def __init__(self, kind: str, dim: int, start: int):
        super().__init__()
        assert kind in ("slice", "place")
        self._attrs["op"] = "strided_copy"
        self._attrs["copy_kind"] = kind
        self._attrs["copy_dim"] = dim
        self._attrs["copy_start"] = start
        self._attrs["has_profiler"] = False

    def bind(self, src: Tensor, dst: Tensor) -> None:
        """Wire the op between two existing tensors (the pass replaces a view by it)."""
        full, piece = (src, dst) if self._attrs["copy_kind"] == "slice" else (dst, src)
        dim = self._attrs["copy_dim"]
        if not all(isinstance(d, IntImm) for d in full._attrs["shape"][dim:]):
            raise NotImplementedError("a split or concatenate that needs a copy needs static shapes from its dim on")
        if len(piece._attrs["shape"]) != len(full._attrs["shape"]):
            raise RuntimeError("strided_copy: rank mismatch")
        self._attrs["inputs"] = [src]
        self._attrs["outputs"] = [dst]
        self._set_depth()
        dst._attrs["src_ops"].add(self)

    def geometry(self):
        return copy_geometry(self._attrs)

    def _get_op_attributes(self):
        return {"kind": self._attrs["copy_kind"], "dim": self._attrs["copy_dim"], "start": self._attrs["copy_start"]}

    def gen_function(self) -> str:
        from ....backend import registry
        from ....backend.target import Target

        return registry.get(f"{Target.current().name()}.strided_copy.gen_function")(self._attrs)
