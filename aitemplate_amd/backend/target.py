"""Compilation target: a context manager that ops query through Target.current().

Counterpart of python/aitemplate/backend/target.py:54-113,245-297 reduced to what
the ROCm GEMM path reads: the target name used in registry keys, the compiler
command lines, the device-selection variable and the "dummy profiling" switch.
"""
from __future__ import annotations

import os
from typing import List, Optional

from ..utils import environ

CURRENT_TARGET: Optional["Target"] = None


class Target:
    def __init__(self, static_files_path: str):
        self._target_type = -1
        self._template_path = ""
        self._compile_cmd = ""
        self.static_files_path = static_files_path
        self._kwargs = {}

    def __enter__(self):
        global CURRENT_TARGET
        if CURRENT_TARGET is not None and CURRENT_TARGET is not self:
            raise RuntimeError("Target has been set.")
        self._prev = CURRENT_TARGET
        CURRENT_TARGET = self
        return self

    def __exit__(self, ptype, value, trace):
        global CURRENT_TARGET
        CURRENT_TARGET = None

    @staticmethod
    def current() -> "Target":
        if CURRENT_TARGET is None:
            raise RuntimeError("Target has not been set.")
        return CURRENT_TARGET

    def name(self) -> str:
        raise NotImplementedError

    def cc(self) -> str:
        raise NotImplementedError

    def src_extension(self) -> str:
        return ".cpp"

    def dev_select_flag(self) -> str:
        raise NotImplementedError

    def compile_cmd(self, executable: bool = False) -> str:
        raise NotImplementedError

    def use_dummy_profiling_results(self) -> bool:
        """No GPU timing: pick instances with the library's shape heuristic (CI_FLAG=CIRCLECI)."""
        return environ.ci_dummy_profiling()

    def force_profile(self) -> bool:
        return environ.force_profile()

    def select_minimal_algo(self, algo_names: List[str]) -> str:
        raise NotImplementedError

    def get_profile_cache_version(self, op_class: str) -> int:
        return 1
