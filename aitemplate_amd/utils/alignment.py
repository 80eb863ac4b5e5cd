"""Vector-width helpers (counterpart of python/aitemplate/utils/alignment.py:26-74).

An "alignment" is the number of consecutive elements that one memory access may
cover; the widest access is 128 bits."""
from typing import List

_ELEM_BYTES = {"float16": 2, "bfloat16": 2, "float32": 4, "float": 4, "int32": 4, "int64": 8, "bool": 1}


def get_alignments(dtype: str) -> List[int]:
    """Candidate alignments for `dtype`, widest first (8,4,2,1 for 2-byte types)."""
    nbytes = _ELEM_BYTES[dtype]
    widest = 16 // nbytes
    out = []
    while widest >= 1:
        out.append(widest)
        widest //= 2
    return out


def find_max_alignment(number: int, dtype: str) -> int:
    """Largest candidate alignment that divides `number` (1 if none does)."""
    if number == 0:
        return get_alignments(dtype)[0]
    for a in get_alignments(dtype):
        if number % a == 0:
            return a
    return 1


def valid_alignment(align: int, dtype: str) -> bool:
    """fp16/bf16 accept any alignment on this backend (scalar-load instances exist); fp32 needs >= 1."""
    return align >= 1


def is_aligned(number: int, dtype: str) -> bool:
    return number % get_alignments(dtype)[0] == 0
