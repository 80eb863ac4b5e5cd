"""Batched GEMM: the bmm base class, the four operand layouts with a row-major result (rcr, rrr, ccr, crr)
and the *_permute forms of rcr and rrr.

Counterparts: python/aitemplate/compiler/ops/gemm_universal/bmm.py:69-119 (base, batch broadcast rules),
bmm_xxx.py:22-150,204-278 (layout bookkeeping), bmm_rcr_permute.py, bmm_rrr_permute.py.  The layouts with a
column-major result (bmm_xxc) exist on CUDA only in the reference."""
from ...base import IntImm, Tensor
from ...dtype import is_same_dtype
from ...tensor_accessor import TensorAccessor
from . import gemm_common as common


class bmm(common.gemm):
    """Base class for bmm: operands are 3-D, or 2-D and broadcast over the other's batch."""

    def _get_batch_size(self, a: Tensor, b: Tensor):
        self._sanity_check(a, b)
        a_shapes, b_shapes = a._attrs["shape"], b._attrs["shape"]
        if len(a_shapes) == 2:
            return b_shapes[0]
        if len(b_shapes) == 2:
            return a_shapes[0]
        if a_shapes[0] != b_shapes[0] and a_shapes[0] != 1 and b_shapes[0] != 1:
            raise RuntimeError(
                "bmm operand A and B should have same batch_size, or batch_size = 1! "
                f"Current shape A: {a_shapes} shape B: {b_shapes} .")
        return a_shapes[0] if a_shapes[0] != 1 else b_shapes[0]

    def _sanity_check(self, a: Tensor, b: Tensor):
        a_shapes, b_shapes = a._attrs["shape"], b._attrs["shape"]
        if len(a_shapes) not in (2, 3):
            raise RuntimeError(f"bmm operand A should have 2 or 3 dimensions! Current shape: {a_shapes}.")
        if len(b_shapes) not in (2, 3):
            raise RuntimeError(f"bmm operand B should have 2 or 3 dimensions! Current shape: {b_shapes}.")
        if len(a_shapes) == 2 and len(b_shapes) == 2:
            raise RuntimeError("bmm operand A and B both have 2 dimensions! Use gemm instead.")
        if not is_same_dtype(a.dtype(), b.dtype()):
            raise RuntimeError(
                f"gemm operand A and B should have the same data type! Current A: {a.dtype()}, B: {b.dtype()}.")


class bmm_rcr(bmm):
    """C[b] = A[b] @ B[b]^T with A [B, M, K], B [B, N, K] -> C [B, M, N]
    (torch.bmm(A, B.transpose(2, 1)))."""

    def __init__(self):
        super().__init__()
        self._attrs["op"] = "bmm_rcr"

        def cal_align_ab(m, n, k):
            return common.default_align_ab(k, k, self._attrs["inputs"][0].dtype())

        self._attrs["f_ab_alignment"] = cal_align_ab

    def _infer_shapes(self, a: Tensor, b: Tensor):
        a_shape, b_shape = a.shape(), b.shape()
        if a_shape[-1] != b_shape[-1]:
            raise RuntimeError(f"bmm_rcr operand A and B should have the same K dim! A: {a_shape}, B: {b_shape}")
        return [self._get_batch_size(a, b), a_shape[-2], b_shape[-2]]

    def _extract_dims(self, for_profiling: bool = False):
        a_shapes = common.extract_shape_from_accessor(self._attrs, common.Source.INPUT, 0)
        b_shapes = common.extract_shape_from_accessor(self._attrs, common.Source.INPUT, 1)
        out_shapes = common.extract_shape_from_accessor(self._attrs, common.Source.OUTPUT, 0)
        b_dim = common.create_input_batch_diminfo([a_shapes, b_shapes], [0, 0], out_shapes[0])
        b_dim.append(common.DimInfo(common.Source.OUTPUT, tensor_idx=0, dim_idx=0))
        ra, rb = len(a_shapes), len(b_shapes)
        return {
            "B": b_dim,
            "M": [common.DimInfo(common.Source.INPUT, tensor_idx=0, dim_idx=ra - 2),
                  common.DimInfo(common.Source.OUTPUT, tensor_idx=0, dim_idx=1)],
            "N": [common.DimInfo(common.Source.INPUT, tensor_idx=1, dim_idx=rb - 2),
                  common.DimInfo(common.Source.OUTPUT, tensor_idx=0, dim_idx=2)],
            "K": [common.DimInfo(common.Source.INPUT, tensor_idx=0, dim_idx=ra - 1),
                  common.DimInfo(common.Source.INPUT, tensor_idx=1, dim_idx=rb - 1)],
        }


class bmm_rcr_permute(bmm_rcr):
    """bmm_rcr whose [B, M, N] result is stored as reshape(B // d1, d1, M, N).permute(0, 2, 1, 3), i.e.
    [B // d1, M, d1, N], with shape = (d1,) (layout "0213" only).
    Counterpart of python/aitemplate/compiler/ops/gemm_universal/bmm_rcr_permute.py:28-116."""

    def __init__(self, shape, layout="0213"):
        super().__init__()
        self._attrs["op"] = "bmm_rcr_permute"
        self._attrs["shape"] = tuple(int(v) for v in shape)
        self._attrs["layout"] = "Permute4DBMM_{}".format(layout)
        self._attrs["permute_shape"] = "_".join(map(str, shape))

    def __call__(self, a: Tensor, b: Tensor) -> Tensor:
        from ..common.view_ops import reshape

        if self._attrs["layout"] != "Permute4DBMM_0213":
            raise NotImplementedError("{} is not implemented!".format(self._attrs["layout"]))
        a, b = self._align_ab(a, b)
        self._attrs["inputs"] = [a, b]
        self._attrs["input_accessors"] = [TensorAccessor(a), TensorAccessor(b)]
        self._set_depth()
        self._sanity_check(a, b)
        output_shape = self._infer_shapes(a, b)
        output = Tensor(output_shape, src_ops={self}, dtype=a.dtype())
        self._attrs["outputs"] = [output]
        self._attrs["output_accessors"] = [TensorAccessor(output)]
        batch, m, n = output_shape
        d1 = self._attrs["shape"][0]
        if not isinstance(batch, IntImm) or batch.value() % d1 != 0:
            raise RuntimeError(f"bmm_rcr_permute needs a static batch that is a multiple of {d1}, got {batch}")
        permuted = [batch.value() // d1, m, d1, n]
        self._extract_epilogue_alignment(permuted)
        return reshape()(output, permuted)

    def _get_op_attributes(self):
        return {"layout": self._attrs["layout"].split("_")[-1], "shape": self._attrs["shape"]}


def _layout_class(name: str, a_col: bool, b_row: bool, doc: str):
    """A [B, M, K] (or [B, K, M] when a_col) times B [B, N, K] (or [B, K, N] when b_row) -> [B, M, N]."""

    class _bmm_layout(bmm):
        __doc__ = doc

        def __init__(self):
            super().__init__()
            self._attrs["op"] = name

            def cal_align_ab(m, n, k):
                # the contiguous dim of each operand bounds the load width (bmm_xxx.py:36-43)
                return common.default_align_ab(m if a_col else k, n if b_row else k,
                                               self._attrs["inputs"][0].dtype())

            self._attrs["f_ab_alignment"] = cal_align_ab

        def _mk(self, a: Tensor, b: Tensor):
            a_shape, b_shape = a.shape(), b.shape()
            m, ka = (a_shape[-1], a_shape[-2]) if a_col else (a_shape[-2], a_shape[-1])
            n, kb = (b_shape[-1], b_shape[-2]) if b_row else (b_shape[-2], b_shape[-1])
            return m, n, ka, kb

        def _infer_shapes(self, a: Tensor, b: Tensor):
            m, n, ka, kb = self._mk(a, b)
            if ka != kb:
                raise RuntimeError(f"{name} operand A and B should have the same K dim! A: {a.shape()}, B: {b.shape()}")
            return [self._get_batch_size(a, b), m, n]

        def _extract_dims(self, for_profiling: bool = False):
            S = common.Source
            a_shapes = common.extract_shape_from_accessor(self._attrs, S.INPUT, 0)
            b_shapes = common.extract_shape_from_accessor(self._attrs, S.INPUT, 1)
            out_shapes = common.extract_shape_from_accessor(self._attrs, S.OUTPUT, 0)
            b_dim = common.create_input_batch_diminfo([a_shapes, b_shapes], [0, 0], out_shapes[0])
            b_dim.append(common.DimInfo(S.OUTPUT, tensor_idx=0, dim_idx=0))
            ra, rb = len(a_shapes), len(b_shapes)
            a_m, a_k = (ra - 1, ra - 2) if a_col else (ra - 2, ra - 1)
            b_n, b_k = (rb - 1, rb - 2) if b_row else (rb - 2, rb - 1)
            return {
                "B": b_dim,
                "M": [common.DimInfo(S.INPUT, tensor_idx=0, dim_idx=a_m), common.DimInfo(S.OUTPUT, tensor_idx=0, dim_idx=1)],
                "N": [common.DimInfo(S.INPUT, tensor_idx=1, dim_idx=b_n), common.DimInfo(S.OUTPUT, tensor_idx=0, dim_idx=2)],
                "K": [common.DimInfo(S.INPUT, tensor_idx=0, dim_idx=a_k), common.DimInfo(S.INPUT, tensor_idx=1, dim_idx=b_k)],
            }

        def _align_ab(self, a: Tensor, b: Tensor):
            # K may be dynamic, as in the reference (tests/unittest/ops/test_bmm.py:102-103); an operand that
            # is K-contiguous then needs every K of the range to keep its rows 16-byte aligned
            return a, b

    _bmm_layout.__name__ = _bmm_layout.__qualname__ = name
    return _bmm_layout


bmm_rrr = _layout_class("bmm_rrr", False, True, "C[b] = A[b] @ B[b] with A [B, M, K], B [B, K, N] (torch.bmm(A, B)).")
bmm_ccr = _layout_class("bmm_ccr", True, False,
                        "C[b] = A[b]^T @ B[b]^T with A [B, K, M], B [B, N, K].")
bmm_crr = _layout_class("bmm_crr", True, True, "C[b] = A[b]^T @ B[b] with A [B, K, M], B [B, K, N].")


class bmm_rrr_permute(bmm_rrr):
    """bmm_rrr whose [B, M, N] result is stored as [B // d1, M, d1, N] with shape = (d1,) (layout "0213").
    Counterpart of python/aitemplate/compiler/ops/gemm_universal/bmm_rrr_permute.py."""

    def __init__(self, shape, layout="0213"):
        super().__init__()
        self._attrs["op"] = "bmm_rrr_permute"
        self._attrs["shape"] = tuple(int(v) for v in shape)
        self._attrs["layout"] = "Permute4DBMM_{}".format(layout)
        self._attrs["permute_shape"] = "_".join(map(str, shape))

    __call__ = bmm_rcr_permute.__call__
    _get_op_attributes = bmm_rcr_permute._get_op_attributes


def _add_class(base, name: str):
    """base(A, B) + D with D of the result's shape [B, M, N]
    (python/aitemplate/compiler/ops/gemm_universal/bmm_xxx_add.py:21-64)."""

    class _bmm_add(base):
        __doc__ = f"C[b] = {base.__name__}(A, B)[b] + D[b]"

        def __init__(self):
            super().__init__()
            self._attrs["op"] = name
            self._attrs["num_sources"] = 1

        @classmethod
        def is_valid_inputs(cls, a: Tensor, b: Tensor, d: Tensor):
            out = base()._infer_shapes(a, b)
            if list(d.shape()) != list(out):
                return False, f"Additional elementwise shape {d.shape()} doesn't match bmm's shape {out}"
            return True, ""

        def __call__(self, a: Tensor, b: Tensor, d: Tensor) -> Tensor:
            a, b = self._align_ab(a, b)
            ok, msg = self.is_valid_inputs(a, b, d)
            if not ok:
                raise RuntimeError(msg)
            self._attrs["inputs"] = [a, b, d]
            self._attrs["input_accessors"] = [TensorAccessor(t) for t in self._attrs["inputs"]]
            self._set_depth()
            self._sanity_check(a, b)
            return self._finish_call([a, b, d], self._infer_shapes(a, b))

    _bmm_add.__name__ = _bmm_add.__qualname__ = name
    return _bmm_add


bmm_rrr_add = _add_class(bmm_rrr, "bmm_rrr_add")
bmm_ccr_add = _add_class(bmm_ccr, "bmm_ccr_add")
bmm_crr_add = _add_class(bmm_crr, "bmm_crr_add")
