"""String-keyed registry that binds op hooks to a backend:
"<target>.<op>.<hook>" -> function  (counterpart of python/aitemplate/backend/registry.py:27-101)."""
from typing import Callable, Dict, List

_REGISTRY: Dict[str, Callable] = {}


def reg(func_name: str, func: Callable = None) -> Callable:
    """Register `func` under `func_name`; usable as a decorator.  Registering a name twice is an error."""
    if func_name in _REGISTRY:
        raise RuntimeError(f"{func_name} has been registered.")

    def _do_reg(f):
        _REGISTRY[func_name] = f
        return f

    if func is None:
        return _do_reg
    return _do_reg(func)


def get(func_name: str) -> Callable:
    if func_name not in _REGISTRY:
        raise RuntimeError(f"{func_name} has not been registered.")
    return _REGISTRY[func_name]


def exists(func_name: str) -> bool:
    return func_name in _REGISTRY


def list_names() -> List[str]:
    return sorted(_REGISTRY)
