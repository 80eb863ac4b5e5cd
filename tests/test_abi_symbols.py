"""CPU-only: the kernel library loads and exports every symbol the header declares."""
import os
import re

from aitemplate_amd import _kernels

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    return sorted(set(re.findall(r"AITAMD_API[^;]*?\b(aitamd_\w+)\s*\(", text, re.S)))


def test_kernel_library_exports_every_declared_symbol():
    lib = _kernels.load()
    declared = _declared_symbols("aitemplate_amd_kernels.h")
    assert declared, "no declarations found"
    for sym in declared:
        assert hasattr(lib, sym), f"{sym} declared in the header but not exported"
    assert sorted(_kernels.EXPORTED_SYMBOLS) == declared


def test_instance_tables_are_populated_without_a_gpu():
    lib = _kernels.load()
    assert lib.aitamd_version().decode().endswith("gfx950")
    for epi in range(17):
        for dt in (0, 1):
            names = _kernels.gemm_algo_names(epi, dt)
            assert len(names) >= 4
            assert len(set(names)) == len(names)
            for i, n in enumerate(names):
                assert lib.aitamd_gemm_find_algo(epi, dt, n.encode()) == i
    # alignment gating: K = 4 only fits the narrow-load instances
    ok = [lib.aitamd_gemm_algo_supported(1, 0, i, 4096, 4, 4, 4, 4, 16) for i in range(lib.aitamd_gemm_num_algos(1, 0))]
    names = _kernels.gemm_algo_names(1, 0)
    assert any(ok) and all(("_v8" not in n) for n, o in zip(names, ok) if o)
    assert lib.aitamd_gemm_heuristic_algo(3, 0, 1, 24576, 3072, 768, 768, 768, 16) >= 0
    assert lib.aitamd_gemm_heuristic_algo(1, 0, 1, 7, 3, 5, 5, 5, 2) >= 0  # odd K -> scalar-load instance


def test_error_reporting_without_launch():
    lib = _kernels.load()
    rc = lib.aitamd_gemm_rcr(99, 0, -1, None, None, None, None, None, None, 1, 1, 1, 1, 1, 1, 1, None)
    assert rc != 0 and "epilogue" in _kernels.last_error()
    rc = lib.aitamd_gemm_rcr(1, 0, -1, None, None, None, None, None, None, 4, 4, 4, 4, 4, 4, 4, None)
    assert rc != 0 and "bias" in _kernels.last_error()
    # empty problems are no-ops and need no device
    assert lib.aitamd_gemm_rcr(0, 0, -1, None, None, None, None, None, None, 0, 4, 4, 4, 4, 4, 4, None) == 0
