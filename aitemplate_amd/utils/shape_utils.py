"""Shape helpers (counterpart of python/aitemplate/utils/shape_utils.py:42-51)."""
from typing import List, Optional


def gen_int_var_min_max(values: List[int], name: Optional[str] = None):
    """IntVar spanning [min(values), max(values)]; an IntImm when they coincide."""
    from ..compiler.base import IntImm, IntVar

    lo, hi = min(values), max(values)
    if lo == hi:
        return IntImm(lo, name=name)
    return IntVar([lo, hi], name=name)


def gen_int_var(values: List[int], name: Optional[str] = None):
    from ..compiler.base import IntImm, IntVar

    vals = sorted(set(values))
    if len(vals) == 1:
        return IntImm(vals[0], name=name)
    return IntVar(vals, name=name)


def all_static_dimensions(shape, skip=0) -> bool:
    from ..compiler.base import IntImm

    return all(isinstance(d, IntImm) for d in list(shape)[skip:])
