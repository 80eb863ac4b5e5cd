"""Dropout / DropPath: identity at inference.

Counterpart of python/aitemplate/frontend/nn/dropout.py:22-50."""
from .module import Module


class Dropout(Module):
    def __init__(self, p=0, dtype="float16"):
        super().__init__()

    def forward(self, *args):
        assert len(args) == 1
        return args[0]


class DropPath(Dropout):
    def __init__(self, dtype="float16"):
        super().__init__()
