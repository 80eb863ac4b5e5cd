"""Helpers for tests written in the style of the reference's unit tests
(counterpart of python/aitemplate/testing/test_utils.py:37-224)."""
from typing import List

import torch

_TORCH_DTYPE = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32,
                "float": torch.float32, "int32": torch.int32, "int64": torch.int64, "bool": torch.bool}


def string_to_torch_dtype(dtype: str):
    return _TORCH_DTYPE[dtype]


def get_random_torch_tensor(shape: List[int], dtype: str = "float16", device: str = "cuda", seed=None):
    g = None
    if seed is not None:
        g = torch.Generator(device="cpu").manual_seed(seed)
        return torch.randn(*shape, generator=g).to(_TORCH_DTYPE[dtype]).to(device)
    return torch.randn(*shape, device=device).to(_TORCH_DTYPE[dtype])


def get_torch_empty_tensor(shape: List[int], dtype: str = "float16", device: str = "cuda"):
    return torch.empty(*shape, device=device, dtype=_TORCH_DTYPE[dtype])


def get_torch_zeros_tensor(shape: List[int], dtype: str = "float16", device: str = "cuda"):
    return torch.zeros(*shape, device=device, dtype=_TORCH_DTYPE[dtype])


def has_op(sorted_ops, op_str: str) -> bool:
    return any(op._attrs["op"] == op_str for op in sorted_ops)


def count_ops(sorted_ops, op_str: str) -> int:
    return sum(1 for op in sorted_ops if op._attrs["op"] == op_str)


def get_src_op_name(tensor) -> str:
    ops = list(tensor.src_ops())
    assert len(ops) == 1
    return ops[0]._attrs["op"]
