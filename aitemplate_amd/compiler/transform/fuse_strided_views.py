"""Turn last-dim split / concatenate ops into offsets and row pitches of the GEMM ops around them.

Counterpart of python/aitemplate/compiler/transform/transform_strided_ops.py:33-64 with its two
rewrites that matter for the GEMM family:

* split + strided op (transform_strided_ops.py `_fuse_split_and_strided_op`): an op that reads a
  piece of a last-dim split reads the split's input instead, through
  `input_accessors[i].update_base_tensor(x, dim, first element)`; when every piece has been
  rewired the split leaves the graph.
* strided op + concatenate (transform_strided_ops.py `_fuse_strided_op_and_cat`): an op whose
  output feeds a last-dim concatenate writes its columns of the concatenated tensor directly,
  through `output_accessors[0].update_base_tensor(cat_output, dim, first element)`; the
  concatenate leaves the graph and its output has one producer per input.

The reference keeps a split or concatenate it cannot fuse and runs a copy kernel for it.  Here a piece
whose consumer (or producer) cannot take a view, and every piece of a split or concatenate along a dim
other than the last, gets a `strided_copy` op: one launch of the library's row copy per piece.
"""
from typing import List

from ..base import Operator, Tensor
from ..ops.common.view_ops import strided_copy
from .toposort import toposort
from .transform_utils import get_sorted_ops

# ops whose generated launch code applies the accessor's offset and row pitch
_GEMM_RCR_PREFIX = "gemm_rcr"
_BMM_PREFIX = "bmm_"


def _is_permute(name: str) -> bool:
    return "permute" in name


def _is_plain_gemm(name: str) -> bool:
    return name.startswith(_GEMM_RCR_PREFIX) and not _is_permute(name)


def _is_bmm(name: str) -> bool:
    return (name.startswith(_BMM_PREFIX) or name.startswith("gemm_rrr")) and "softmax" not in name


def can_read_strided(op: Operator, input_idx: int) -> bool:
    """The op's launch code honours offset + pitch on input `input_idx`."""
    name = op._attrs["op"]
    if "input_accessors" not in op._attrs:
        return False
    if input_idx in (0, 1):  # A, B
        return name.startswith(_GEMM_RCR_PREFIX) or _is_bmm(name)
    if _is_plain_gemm(name):
        # inputs are a, b, bias, d0, d1: the residuals may be views, the bias not
        return input_idx >= 3
    return False


def can_write_strided(op: Operator) -> bool:
    name = op._attrs["op"]
    if "output_accessors" not in op._attrs or _is_permute(name):
        return False
    return _is_plain_gemm(name) or _is_bmm(name)


def _piece_needs_copy(piece: Tensor, outputs: List[Tensor]) -> bool:
    """Whatever the other pieces turn out to be, this one cannot be read in place."""
    x, dim, _ = piece._attrs["strided_view_of"]
    if dim != len(x._attrs["shape"]) - 1:
        return True  # (accessors describe an offset and a pitch of the last dim only)
    if piece._attrs["is_output"] or any(piece is o for o in outputs):
        return True
    for op in piece.dst_ops():
        for i, t in enumerate(op._attrs["inputs"]):
            if t is piece and not can_read_strided(op, i):
                return True
    return False


def _residual_pitch(op: Operator, idx: int, copied: dict):
    """Row pitch the op's residual input `idx` will have once the pass has run: the width of the tensor a piece
    is read out of when it stays a view, the tensor's own width otherwise."""
    acc = op._attrs["input_accessors"][idx]
    if acc.actual_shapes is not None:
        return acc.row_pitch()
    t = op._attrs["inputs"][idx]
    view = t._attrs.get("strided_view_of")
    if view is not None and id(t) in copied and not copied[id(t)]:
        return view[0]._attrs["shape"][-1].value()
    return t._attrs["shape"][-1].value()


def _decide_copies(pieces: List[Tensor], outputs: List[Tensor]) -> dict:
    """id(piece) -> True when the piece becomes a tensor of its own.  The generated launch passes one row pitch for
    both residuals (`ldd`), so a residual may only be a view when every residual of that op ends up with the same
    pitch; a piece that fails this is copied, which can change the pitch its partner was checked against, hence
    the loop (a piece only ever moves from view to copy)."""
    copied = {id(t): _piece_needs_copy(t, outputs) for t in pieces}
    changed = True
    while changed:
        changed = False
        for piece in pieces:
            if copied[id(piece)]:
                continue
            for op in piece.dst_ops():
                inputs = op._attrs["inputs"]
                res = [i for i in range(3, len(inputs))] if _is_plain_gemm(op._attrs["op"]) else []
                if len(res) < 2 or not any(inputs[i] is piece for i in res):
                    continue
                if len({_residual_pitch(op, i, copied) for i in res}) > 1:
                    copied[id(piece)] = True
                    changed = True
                    break
    return copied


def _rewire_split_piece(piece: Tensor, needs_copy: bool) -> None:
    x, dim, start = piece._attrs["strided_view_of"]
    if needs_copy:
        # the piece becomes a tensor of its own, filled by a row copy out of x
        piece._attrs["strided_view_of"] = None
        piece._attrs["is_view_of"] = None
        for producer in list(piece.src_ops()):
            piece._attrs["src_ops"].discard(producer)
        strided_copy("slice", dim, start).bind(x, piece)
        return
    for op in list(piece.dst_ops()):
        hit = [i for i, t in enumerate(op._attrs["inputs"]) if t is piece]
        for i in hit:
            op._attrs["input_accessors"][i].update_base_tensor(x, dim, start)
        op._attrs["inputs"] = [x if t is piece else t for t in op._attrs["inputs"]]
        piece._attrs["dst_ops"].discard(op)
        x._attrs["dst_ops"].add(op)


def _fuse_splits(graph: List[Tensor], outputs: List[Tensor]) -> bool:
    splits = []
    for op in get_sorted_ops(graph):
        if op._attrs["op"] != "split":
            continue
        pieces = [t for t in op._attrs["outputs"] if t._attrs.get("strided_view_of") is not None]
        if pieces:
            splits.append((op, pieces))
    copied = _decide_copies([t for _, pieces in splits for t in pieces], outputs)
    for op, pieces in splits:
        for piece in pieces:
            _rewire_split_piece(piece, copied[id(piece)])
        # nothing reads the pieces any more: the split is unreachable from the outputs
        op._attrs["inputs"][0]._attrs["dst_ops"].discard(op)
    return bool(splits)


def _fuse_concats(graph: List[Tensor], outputs: List[Tensor]) -> bool:
    changed = False
    for cat in get_sorted_ops(graph):
        if cat._attrs["op"] != "concatenate":
            continue
        out = cat._attrs["outputs"][0]
        dim = cat._attrs["concat_dim"]
        times = {}
        for t in cat._attrs["inputs"]:
            times[id(t)] = times.get(id(t), 0) + 1
        start = 0
        out._attrs["src_ops"].discard(cat)
        last_dim = dim == len(out._attrs["shape"]) - 1
        for t in cat._attrs["inputs"]:
            producers = list(t.src_ops())
            width = t._attrs["shape"][dim].value()
            fusable = (last_dim and times[id(t)] == 1 and len(producers) == 1 and can_write_strided(producers[0])
                       and not (t._attrs["is_output"] or any(t is o for o in outputs))
                       and len(list(t.dst_ops())) == 1 and t._attrs["is_view_of"] is None)
            t._attrs["dst_ops"].discard(cat)
            if fusable:
                producer = producers[0]
                producer._attrs["output_accessors"][0].update_base_tensor(out, dim, start)
                producer._attrs["outputs"] = [out]
                out._attrs["src_ops"].add(producer)
            else:
                # a graph input, a constant, a tensor somebody else reads or writes through a view, an input that
                # appears twice, any input of a concatenate along another dim: copied into its rows of the output
                strided_copy("place", dim, start).bind(t, out)
            start += width
        changed = True
    return changed


def fuse_strided_views(sorted_graph: List[Tensor], outputs: List[Tensor]) -> List[Tensor]:
    """Apply both rewrites and return the re-sorted graph (unchanged object when nothing matched)."""
    changed = _fuse_splits(sorted_graph, outputs)
    changed = _fuse_concats(sorted_graph, outputs) or changed
    return toposort(outputs) if changed else sorted_graph
