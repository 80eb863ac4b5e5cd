"""Split-K instances of the RCR GEMM family through the C ABI: several workgroups share a tile along K, leave fp32
partial tiles in caller-provided scratch memory and the last one to arrive sums them and runs the epilogue.
Checked against the oracle (the fp32 PyTorch expressions of the reference's unit tests,
tests/unittest/ops/test_gemm_bias.py:69 and siblings) at atol = rtol = 1e-2."""
import pytest
import torch

from aitemplate_amd import _kernels, eager
from oracle import oracle

pytestmark = pytest.mark.gpu


def _splitk_algos(op, dtype=0):
    names = _kernels.gemm_algo_names(_kernels.EPILOGUE_OF_OP[op], dtype)
    return [(i, n) for i, n in enumerate(names) if n.endswith("_splitk")]


def _inputs(M, N, K, nres, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * K ** -0.5).to(dtype)
    b = ((torch.rand(N, generator=g) - 0.5) * 0.2).to(dtype)
    d = [torch.randn(M, N, generator=g).to(dtype) for _ in range(nres)]
    return x, w, b, d


@pytest.mark.parametrize("op,nres", [("gemm_rcr", 0), ("gemm_rcr_bias", 0), ("gemm_rcr_bias_gelu", 0),
                                     ("gemm_rcr_bias_add", 1), ("gemm_rcr_bias_add_add", 2)])
@pytest.mark.parametrize("M,N,K", [
    (256, 1024, 1024),   # the plumbing configuration: 64 tiles of 64 x 64, four workgroups each
    (100, 200, 4096),    # ragged tiles, sixteen workgroups per tile
    (64, 64, 264),       # K tail in the last workgroup's share
    (300, 72, 136),      # three K-slabs: one workgroup per tile only (no partial tiles written)
    (512, 768, 3072),    # small-batch BERT down-projection
])
def test_splitk_matches_oracle(op, nres, M, N, K):
    algos = _splitk_algos(op)
    assert algos, "no split-K instance compiled"
    x, w, b, d = _inputs(M, N, K, nres, torch.float16, seed=M + N + K)
    want = oracle.torch_gemm(op, x, w, b if op != "gemm_rcr" else None, *d).half().float()
    xs, ws, bs, ds = x.cuda(), w.cuda(), b.cuda(), [t.cuda() for t in d]
    for algo, name in algos:
        need = eager.gemm_workspace_bytes(op, algo, M, N, K)
        scratch = eager.new_workspace(need)
        print(f"case {op} {name} M={M} N={N} K={K} workspace={need}", flush=True)
        for rep in range(3):  # the counters must be left at zero: later launches reuse the buffer as it is
            out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
            eager.gemm(op, xs, ws, bs if op != "gemm_rcr" else None, *ds, out=out, algo=algo, workspace=scratch)
            torch.cuda.synchronize()
            torch.testing.assert_close(out.cpu().float(), want, atol=1e-2, rtol=1e-2)
        counter_bytes = min(need, 4096)
        assert int(scratch[:counter_bytes].to(torch.int32).sum()) == 0


@pytest.mark.parametrize("M,N,K", [(1, 6912, 8314), (100, 200, 4102), (64, 64, 270), (48, 136, 12)])
def test_splitk_with_dword_aligned_k(M, N, K):
    """K % 8 in {2, 4, 6}: only the instance that takes rows aligned to dwords qualifies; the workgroup with the
    last share of K multiplies the 2, 4 or 6 elements behind the rows' last whole 16-byte piece."""
    op = "gemm_rcr_bias"
    algos = [(i, n) for i, n in _splitk_algos(op) if n.endswith("_k2_splitk")]
    assert algos, "no split-K instance for dword-aligned K compiled"
    lib = _kernels.load()
    x, w, b, _ = _inputs(M, N, K, 0, torch.float16, seed=M + N + K)
    want = oracle.torch_gemm(op, x, w, b).half().float()
    xs, ws, bs = x.cuda(), w.cuda(), b.cuda()
    for algo, name in algos:
        assert lib.aitamd_gemm_algo_supported(_kernels.EPILOGUE_OF_OP[op], 0, algo, M, N, K, K, K, 4)
        need = eager.gemm_workspace_bytes(op, algo, M, N, K)
        scratch = eager.new_workspace(need)
        print(f"case {op} {name} M={M} N={N} K={K} workspace={need}", flush=True)
        for rep in range(2):
            out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
            eager.gemm(op, xs, ws, bs, out=out, algo=algo, workspace=scratch)
            torch.cuda.synchronize()
            torch.testing.assert_close(out.cpu().float(), want, atol=1e-2, rtol=1e-2)
        assert int(scratch[:min(need, 4096)].to(torch.int32).sum()) == 0


def test_splitk_is_deterministic_and_bf16():
    op, (M, N, K) = "gemm_rcr_bias", (192, 320, 2048)
    x, w, b, _ = _inputs(M, N, K, 0, torch.bfloat16, seed=5)
    want = oracle.torch_gemm(op, x, w, b).bfloat16().float()
    for algo, name in _splitk_algos(op, dtype=1):
        scratch = eager.new_workspace(eager.gemm_workspace_bytes(op, algo, M, N, K, dtype=torch.bfloat16))
        outs = [eager.gemm(op, x.cuda(), w.cuda(), b.cuda(), algo=algo, workspace=scratch) for _ in range(4)]
        torch.cuda.synchronize()
        torch.testing.assert_close(outs[0].cpu().float(), want, atol=2e-2, rtol=2e-2)
        # the partial tiles are summed in slab order whoever arrives last: bit-identical from run to run
        for o in outs[1:]:
            assert torch.equal(o, outs[0]), name


def test_splitk_without_workspace_runs_unsplit():
    op, (M, N, K) = "gemm_rcr_bias", (256, 1024, 1024)
    x, w, b, _ = _inputs(M, N, K, 0, torch.float16, seed=1)
    want = oracle.torch_gemm(op, x, w, b).half().float()
    algo, name = _splitk_algos(op)[0]
    need = eager.gemm_workspace_bytes(op, algo, M, N, K)
    assert need > 0
    # no buffer, or one that is too small: one workgroup per tile, and the small buffer is not touched
    out = eager.gemm(op, x.cuda(), w.cuda(), b.cuda(), algo=algo)
    torch.testing.assert_close(out.cpu().float(), want, atol=1e-2, rtol=1e-2)
    small = torch.full((need - 16,), 7, dtype=torch.uint8, device="cuda")
    out = eager.gemm(op, x.cuda(), w.cuda(), b.cuda(), algo=algo, workspace=small)
    torch.testing.assert_close(out.cpu().float(), want, atol=1e-2, rtol=1e-2)
    assert bool((small == 7).all())
    # instances without scratch memory report 0 and ignore a buffer
    assert eager.gemm_workspace_bytes(op, 0, M, N, K) == 0
    out = eager.gemm(op, x.cuda(), w.cuda(), b.cuda(), algo=0, workspace=eager.new_workspace(64))
    torch.testing.assert_close(out.cpu().float(), want, atol=1e-2, rtol=1e-2)


def test_splitk_results_do_not_change_under_cache_pressure():
    """The workgroups of a tile run on different XCDs, whose L2s are not coherent with each other: the partial tiles
    are exchanged with write-through stores and a counter.  About 2000 launches over six shapes; before every launch
    the partial-tile slots of the scratch memory (not its counters) are filled with NaN and a 64 MiB copy goes
    through the L2s, so a workgroup that read a stale or not yet written slot would show.  Every result is compared
    bit for bit with the shape's first one (itself checked against the oracle); the test stops at the first batch
    of launches that holds a mismatch."""
    op = "gemm_rcr_bias"
    shapes = [(256, 1024, 1024), (100, 200, 4096), (512, 768, 3072), (64, 256, 8192), (1, 6912, 8320), (192, 320, 2048)]
    src = torch.empty(64 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    launches_per_shape, batch = 340, 20
    for M, N, K in shapes:
        x, w, b, _ = _inputs(M, N, K, 0, torch.float16, seed=M + N + K + 1)
        want = oracle.torch_gemm(op, x, w, b).half().float()
        xs, ws, bs = x.cuda(), w.cuda(), b.cuda()
        best = None
        for algo, name in _splitk_algos(op):
            need = eager.gemm_workspace_bytes(op, algo, M, N, K)
            if need > 4096 and not name.endswith("_k2_splitk") and (best is None or need > best[2]):
                best = (algo, name, need)
        assert best is not None, f"no split-K instance splits M={M} N={N} K={K}"
        algo, name, need = best
        scratch = eager.new_workspace(need)
        print(f"case split-K soak {name} M={M} N={N} K={K} workspace={need}", flush=True)
        first = eager.gemm(op, xs, ws, bs, algo=algo, workspace=scratch)
        torch.cuda.synchronize()
        torch.testing.assert_close(first.cpu().float(), want, atol=1e-2, rtol=1e-2)
        out = torch.empty_like(first)
        bad = torch.zeros((), dtype=torch.int64, device="cuda")
        slots = scratch[4096:].view(torch.float32)  # the fp32 partial tiles behind the counters
        for i in range(launches_per_shape):
            slots.fill_(float("nan"))
            dst.copy_(src)
            eager.gemm(op, xs, ws, bs, out=out, algo=algo, workspace=scratch)
            bad += (out != first).sum() + torch.isnan(out).sum()
            if (i + 1) % batch == 0:
                assert int(bad) == 0, f"{name} M={M} N={N} K={K}: mismatch within launches {i + 1 - batch}..{i}"
        assert int(bad) == 0
        assert int(scratch[:4096].to(torch.int32).sum()) == 0


def test_splitk_on_two_streams_with_separate_scratch_buffers():
    """Launches that overlap in time need scratch buffers of their own (the header says so): two streams, each with
    its own buffer and output, 100 launches each on different shapes, every result equal to a serial run's."""
    op = "gemm_rcr_bias"
    cases = []
    for M, N, K in ((256, 1024, 1024), (64, 256, 8192)):
        x, w, b, _ = _inputs(M, N, K, 0, torch.float16, seed=M + K)
        algo, name = [(i, n) for i, n in _splitk_algos(op) if "64x64x64" in n and not n.endswith("_k2_splitk")][0]
        need = eager.gemm_workspace_bytes(op, algo, M, N, K)
        assert need > 4096
        xs, ws, bs = x.cuda(), w.cuda(), b.cuda()
        serial = eager.gemm(op, xs, ws, bs, algo=algo, workspace=eager.new_workspace(need))
        torch.cuda.synchronize()
        torch.testing.assert_close(serial.cpu().float(), oracle.torch_gemm(op, x, w, b).half().float(), atol=1e-2, rtol=1e-2)
        cases.append((xs, ws, bs, algo, eager.new_workspace(need), serial, torch.cuda.Stream(),  # default priority
                      torch.zeros((), dtype=torch.int64, device="cuda")))
    torch.cuda.synchronize()
    print("case split-K two streams", flush=True)
    for i in range(100):
        for xs, ws, bs, algo, scratch, serial, stream, bad in cases:
            with torch.cuda.stream(stream):
                out = eager.gemm(op, xs, ws, bs, algo=algo, workspace=scratch)
                bad += (out != serial).sum()
    torch.cuda.synchronize()
    for case in cases:
        assert int(case[-1]) == 0
