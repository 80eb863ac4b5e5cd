"""How an op reads or writes a tensor: element offset and row pitch of a (possibly strided) view.

Counterpart of python/aitemplate/compiler/tensor_accessor.py:32-90.  For the GEMM
family every accessor starts as the identity; `update_base_tensor` turns it into a
view of a wider tensor (what the reference's split / concat fusion passes do), and
the launch-code generators honour `offset` and `stride(dim)`.
"""
from __future__ import annotations

import copy
from typing import List, Optional


class TensorAccessor:
    def __init__(self, original_tensor) -> None:
        self.offset = 0
        self.original_shapes = original_tensor._attrs["shape"]
        self.tensor_dtype = original_tensor.dtype()
        self.is_contiguous = True
        self.is_from_strided_tensor = False
        self.stride_dim: Optional[int] = None
        self.actual_shapes: Optional[List] = None
        self.original_total_elements_from_stride_dim = None
        self.actual_total_elements_from_stride_dim = None

    def __deepcopy__(self, memo):
        res = copy.copy(self)
        res.original_shapes = copy.deepcopy(self.original_shapes, memo)
        res.actual_shapes = copy.deepcopy(self.actual_shapes, memo)
        return res

    def __str__(self) -> str:
        return str(vars(self))

    def update_base_tensor(self, new_tensor, stride_dim: int, stride_dim_offset: int) -> None:
        """Make this accessor a view into `new_tensor`, which is wider along `stride_dim`;
        the view starts `stride_dim_offset` elements into that dim."""
        assert self.actual_shapes is None, "an accessor can be re-based once"
        self.actual_shapes = new_tensor._attrs["shape"]
        self.stride_dim = stride_dim
        self.is_from_strided_tensor = True
        inner = 1
        for d in self.actual_shapes[stride_dim + 1:]:
            inner *= d.value()
        self.offset = stride_dim_offset * inner
        self.original_total_elements_from_stride_dim = self.original_shapes[stride_dim].value() * inner
        self.actual_total_elements_from_stride_dim = self.actual_shapes[stride_dim].value() * inner
        self.is_contiguous = (
            self.original_total_elements_from_stride_dim == self.actual_total_elements_from_stride_dim
        )

    def stride(self, dim: int) -> int:
        """Elements between consecutive indices of `dim` (static trailing dims only)."""
        shapes = self.actual_shapes if self.actual_shapes is not None else self.original_shapes
        s = 1
        for d in shapes[dim + 1:]:
            s *= d.value()
        return s

    def row_pitch(self) -> int:
        """Elements between consecutive rows when the tensor is seen as 2-D [rows, last_dim]."""
        shapes = self.actual_shapes if self.actual_shapes is not None else self.original_shapes
        return shapes[-1].value()
