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
