"""aitamd_gemm_rcr_noalloc - the entry point that allocates nothing: its scratch memory is an array inside the
library's device image - against aitamd_gemm_rcr_ws with a caller's buffer, through the C ABI.  Both run the same
kernels and sum the partial tiles in slab order, so the results must be bit-identical."""
import ctypes

import pytest
import torch

from aitemplate_amd import _kernels
from oracle import oracle

pytestmark = pytest.mark.gpu
EPI_BIAS = 1


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _splitk_algo(lib, tile):
    n = lib.aitamd_gemm_num_algos(EPI_BIAS, 0)
    for i in range(n):
        name = lib.aitamd_gemm_algo_name(EPI_BIAS, 0, i).decode()
        if name.endswith("_splitk") and tile in name:
            return i, name
    raise AssertionError(f"no split-K instance with tile {tile}")


def _operands(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).half()
    w = (torch.randn(N, K, generator=g) * K ** -0.5).half()
    b = ((torch.rand(N, generator=g) - 0.5) * 0.2).half()
    return x, w, b


def test_noalloc_entry_matches_the_workspace_entry_on_two_calls_in_a_row():
    lib = _kernels.load()
    algo, name = _splitk_algo(lib, "64x64x64")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    capacity = lib.aitamd_gemm_noalloc_scratch_bytes()
    # the second problem is smaller than the first: it finds the first one's partial tiles in the scratch memory
    for M, N, K in ((256, 1024, 1024), (100, 200, 4096)):
        need = lib.aitamd_gemm_workspace_bytes(EPI_BIAS, 0, algo, 1, M, N, K)
        assert 0 < need <= capacity, (need, capacity)
        x, w, b = _operands(M, N, K, seed=M + K)
        want = oracle.torch_gemm("gemm_rcr_bias", x, w, b).half().float()
        xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
        print(f"case noalloc {name} M={M} N={N} K={K} scratch needed {need} of {capacity}", flush=True)
        got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        rc = lib.aitamd_gemm_rcr_noalloc(EPI_BIAS, 0, algo, _ptr(xd), _ptr(wd), _ptr(bd), None, None, _ptr(got),
                                         M, N, K, K, K, N, N, stream)
        _kernels.check(rc, "aitamd_gemm_rcr_noalloc")
        ref = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        scratch = torch.zeros(need, dtype=torch.uint8, device="cuda")
        rc = lib.aitamd_gemm_rcr_ws(EPI_BIAS, 0, algo, _ptr(xd), _ptr(wd), _ptr(bd), None, None, _ptr(ref),
                                    M, N, K, K, K, N, N, _ptr(scratch), need, stream)
        _kernels.check(rc, "aitamd_gemm_rcr_ws")
        torch.cuda.synchronize()
        assert torch.equal(got, ref), "no-alloc entry differs from the workspace entry"
        torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)
    # the library's own choice of instance (algo = -1) works too
    M, N, K = 64, 256, 8192
    x, w, b = _operands(M, N, K, seed=3)
    got = torch.empty(M, N, dtype=torch.float16, device="cuda")
    rc = lib.aitamd_gemm_rcr_noalloc(EPI_BIAS, 0, -1, _ptr(x.cuda()), _ptr(w.cuda()), _ptr(b.cuda()), None, None,
                                     _ptr(got), M, N, K, K, K, N, N, stream)
    _kernels.check(rc, "aitamd_gemm_rcr_noalloc")
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), oracle.torch_gemm("gemm_rcr_bias", x, w, b).half().float(),
                               atol=1e-2, rtol=1e-2)


def test_noalloc_entry_refuses_what_does_not_fit():
    lib = _kernels.load()
    algo, name = _splitk_algo(lib, "128x128x32")
    capacity = lib.aitamd_gemm_noalloc_scratch_bytes()
    shape = None
    for M, N in ((256, 1024), (512, 512), (128, 2048)):  # 16 tiles of 128 x 128, 16 workgroups each
        if lib.aitamd_gemm_workspace_bytes(EPI_BIAS, 0, algo, 1, M, N, 8192) > capacity:
            shape = (M, N, 8192)
            break
    assert shape is not None, "no test shape exceeds the built-in scratch memory"
    M, N, K = shape
    x, w, b = _operands(M, N, K, seed=9)
    out = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    rc = lib.aitamd_gemm_rcr_noalloc(EPI_BIAS, 0, algo, _ptr(x.cuda()), _ptr(w.cuda()), _ptr(b.cuda()), None, None,
                                     _ptr(out), M, N, K, K, K, N, N, None)
    assert rc != 0
    assert "scratch memory" in _kernels.last_error()
    torch.cuda.synchronize()
    assert not bool(out.any()), "a refused call must not launch anything"


def test_noalloc_entry_under_stream_capture_and_graph_replay():
    """Two split-K launches captured into one graph (kernel nodes only; the kernels leave their counters zero, so
    nothing clears memory between them) and replayed three times with eager work and synchronisations in between:
    every replay equals the workspace entry's result.  The array's address is looked up beforehand by
    aitamd_gemm_noalloc_scratch_bytes(); the first call of the no-alloc entry itself happens under capture."""
    lib = _kernels.load()
    algo, name = _splitk_algo(lib, "64x64x64")
    assert lib.aitamd_gemm_noalloc_scratch_bytes() >= (16 << 20)  # (also resolves the array's address)
    shapes = ((200, 512, 2048), (64, 256, 4096))
    ops, refs, outs = [], [], []
    for M, N, K in shapes:
        x, w, b = (t.cuda() for t in _operands(M, N, K, seed=M + N))
        need = lib.aitamd_gemm_workspace_bytes(EPI_BIAS, 0, algo, 1, M, N, K)
        assert need > 0
        scratch = torch.zeros(need, dtype=torch.uint8, device="cuda")
        ref = torch.empty(M, N, dtype=torch.float16, device="cuda")
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.aitamd_gemm_rcr_ws(EPI_BIAS, 0, algo, _ptr(x), _ptr(w), _ptr(b), None, None, _ptr(ref), M, N, K, K, K, N, N,
                                    _ptr(scratch), need, stream)
        _kernels.check(rc, "aitamd_gemm_rcr_ws")
        ops.append((x, w, b, M, N, K))
        refs.append(ref)
        outs.append(torch.zeros(M, N, dtype=torch.float16, device="cuda"))
    torch.cuda.synchronize()
    print(f"case noalloc graph capture {name} shapes {shapes}", flush=True)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()  # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            handle = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            for (x, w, b, M, N, K), out in zip(ops, outs):
                rc = lib.aitamd_gemm_rcr_noalloc(EPI_BIAS, 0, algo, _ptr(x), _ptr(w), _ptr(b), None, None, _ptr(out),
                                                 M, N, K, K, K, N, N, handle)
                _kernels.check(rc, "aitamd_gemm_rcr_noalloc under capture")
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert not any(bool(o.any()) for o in outs), "capture must not run anything"
    for replay in range(3):
        for o in outs:
            o.fill_(float("nan"))  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for o, ref in zip(outs, refs):
            assert torch.equal(o, ref), f"replay {replay} differs from the workspace entry"
