"""Local cache of profiling results, so a workload that was timed once is not timed again.

Counterpart of python/aitemplate/backend/profiler_cache.py:479-921 (ProfileCacheDB, sqlite3, one
table per op class and cache version) restricted to the GEMM family, the only op class of this
backend.  A record is keyed by what decides the winner: op type, element type, device name, the
profiled workload (the exec key, stored with its sha1 like the reference's GemmQueryEntry,
compiler/ops/gemm_universal/cache_entry.py:22-38) and a fingerprint of the kernel library's
instance list - rebuilding the library with other instances must not resurrect old winners.
"""
from __future__ import annotations

import logging
import os
import sqlite3
from hashlib import sha1
from typing import Any, Dict, Optional, Tuple

_LOGGER = logging.getLogger(__name__)

# bump when the table layout changes
GEMM_CACHE_VERSION = 1

_GEMM_COLUMNS = ("op_type", "dtype", "device", "instances_sha1", "exec_entry_sha1")


def exec_entry_sha1(exec_entry: str) -> str:
    return sha1(exec_entry.encode("utf-8")).hexdigest()


class ProfileCacheDB:
    def __init__(self, target: str, path: Optional[str] = None):
        self._target = target
        self._path = path or ":memory:"
        self._con = sqlite3.connect(self._path, timeout=30.0)
        self._table = f"{target}_gemm_{GEMM_CACHE_VERSION}"
        self._con.execute(
            f"CREATE TABLE IF NOT EXISTS {self._table} ("
            "id INTEGER PRIMARY KEY AUTOINCREMENT, exec_entry VARCHAR(8192) NOT NULL, "
            "exec_entry_sha1 VARCHAR(64) NOT NULL, op_type VARCHAR(512) NOT NULL, dtype VARCHAR(32) NOT NULL, "
            "device VARCHAR(128) NOT NULL, instances_sha1 VARCHAR(64) NOT NULL, algo VARCHAR(512) NOT NULL, "
            "workspace INTEGER NOT NULL, split_k INTEGER NOT NULL, duration REAL NOT NULL, "
            "template_ver INTEGER NOT NULL DEFAULT 0, created_at TIMESTAMP DEFAULT CURRENT_TIMESTAMP NOT NULL)")
        self._con.commit()

    @property
    def gemm_cache_version(self) -> int:
        return GEMM_CACHE_VERSION

    @staticmethod
    def _key(args: Dict[str, Any]) -> Tuple:
        missing = [c for c in _GEMM_COLUMNS if c not in args]
        if missing:
            raise KeyError(f"profile cache query lacks {missing}")
        return tuple(str(args[c]) for c in _GEMM_COLUMNS)

    def query_gemm(self, args: Dict[str, Any]) -> Optional[Tuple[str, int, int]]:
        """(algo, workspace, split_k) of the cached winner, or None."""
        where = " AND ".join(f"{c}=?" for c in _GEMM_COLUMNS)
        row = self._con.execute(
            f"SELECT algo, workspace, split_k FROM {self._table} WHERE {where} ORDER BY id DESC LIMIT 1",
            self._key(args)).fetchone()
        return None if row is None else (row[0], int(row[1]), int(row[2]))

    def insert_gemm(self, args: Dict[str, Any]) -> None:
        """Store a winner unless the workload already has one (first writer wins, as in the reference)."""
        if self.query_gemm(args) is not None:
            _LOGGER.debug("profile cache: entry exists for %s, not overwritten", args.get("exec_entry"))
            return
        self._con.execute(
            f"INSERT INTO {self._table} (exec_entry, exec_entry_sha1, op_type, dtype, device, instances_sha1, algo, "
            "workspace, split_k, duration) VALUES (?,?,?,?,?,?,?,?,?,?)",
            (str(args["exec_entry"]), str(args["exec_entry_sha1"]), str(args["op_type"]), str(args["dtype"]),
             str(args["device"]), str(args["instances_sha1"]), str(args["algo"]), int(args.get("workspace", 0)),
             int(args.get("split_k", 1)), float(args.get("duration", 0.0))))
        self._con.commit()

    def num_entries(self) -> int:
        return int(self._con.execute(f"SELECT COUNT(*) FROM {self._table}").fetchone()[0])

    def close(self) -> None:
        if self._con is not None:
            self._con.close()
            self._con = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass
