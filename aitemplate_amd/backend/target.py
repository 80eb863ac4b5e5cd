"""Compilation target: a context manager that ops query through Target.current().

Counterpart of python/aitemplate/backend/target.py:54-113,245-297 reduced to what
the ROCm GEMM path reads: the target name used in registry keys, the compiler
command lines, the device-selection variable and the "dummy profiling" switch.
"""
from __future__ import annotations

import logging
import os
import pathlib
import tempfile
from typing import Any, Dict, List, Optional, Tuple

from ..utils import environ
from .profiler_cache import ProfileCacheDB

_LOGGER = logging.getLogger(__name__)

CURRENT_TARGET: Optional["Target"] = None


class Target:
    def __init__(self, static_files_path: str):
        self._target_type = -1
        self._template_path = ""
        self._compile_cmd = ""
        self.static_files_path = static_files_path
        self._kwargs = {}
        self._cache_path: Optional[str] = None
        self._profile_cache: Optional[ProfileCacheDB] = None

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
        if self._profile_cache is not None:
            self._profile_cache.close()
            self._profile_cache = None

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

    # ---- profiling-result cache (reference: backend/target.py:299-420) ----------------------
    def device_name(self) -> str:
        """Part of the cache key: results of one device type do not transfer to another."""
        return self.name()

    def _prepare_profile_cache_path(self) -> Optional[str]:
        """<CACHE_DIR or ~/.aitemplate>/<target>.db; FLUSH_PROFILE_CACHE=1 starts it afresh.
        None when instances are picked without timing."""
        if self.use_dummy_profiling_results():
            return None
        prefix = os.environ.get("CACHE_DIR") or os.path.join(pathlib.Path.home(), ".aitemplate")
        try:
            os.makedirs(prefix, exist_ok=True)
        except OSError as error:
            _LOGGER.info("Cannot mkdir at %s due to issue %s", prefix, error)
            prefix = os.path.join(tempfile.mkdtemp(prefix="aitemplate_"), ".aitemplate")
            os.makedirs(prefix, exist_ok=True)
        path = os.path.join(prefix, f"{self.name()}.db")
        if os.environ.get("FLUSH_PROFILE_CACHE", "0") != "0" and os.path.exists(path):
            os.remove(path)
        return path

    def _cache(self) -> Optional[ProfileCacheDB]:
        if self._profile_cache is None:
            self._cache_path = self._prepare_profile_cache_path()
            if self._cache_path is None:
                return None
            _LOGGER.info("Loading profile cache from: %s", self._cache_path)
            self._profile_cache = ProfileCacheDB(self.name(), path=self._cache_path)
        return self._profile_cache

    def get_profile_cache_path(self) -> Optional[str]:
        self._cache()
        return self._cache_path

    def get_profile_cache_version(self, op_class: str) -> int:
        if op_class != "gemm":
            raise NotImplementedError
        from .profiler_cache import GEMM_CACHE_VERSION

        return GEMM_CACHE_VERSION

    def query_profile_cache(self, op_class: str, args: Dict[str, Any]) -> Optional[Tuple[str, int, int]]:
        if op_class != "gemm":
            raise NotImplementedError
        cache = self._cache()
        return None if cache is None else cache.query_gemm(args)

    def insert_profile_cache(self, op_class: str, args: Dict[str, Any]) -> None:
        if op_class != "gemm":
            raise NotImplementedError
        cache = self._cache()
        if cache is not None:
            cache.insert_gemm(args)
