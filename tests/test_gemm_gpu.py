"""GPU parity of the RCR GEMM family through the C ABI against the CPU oracle.

Tolerance: atol = rtol = 1e-2 on fp16 outputs with fp32 accumulation (the
tightest the reference uses for this family, tests/unittest/ops/test_gemm.py:31-35);
bf16 uses 3e-2 relative (8-bit mantissa)."""
import pytest
import torch

from aitemplate_amd import _kernels, eager
from oracle import oracle

pytestmark = pytest.mark.gpu

ATOL = RTOL = 1e-2


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _run_and_check(op, M, N, K, dtype=torch.float16, algo=-1, seed=0, tol=None):
    x = _rand((M, K), dtype, seed)
    w = _rand((N, K), dtype, seed + 1, scale=max(K, 1) ** -0.5)
    b = _rand((N,), dtype, seed + 2)
    d0 = _rand((M, N), dtype, seed + 3)
    d1 = _rand((M, N), dtype, seed + 4)
    want = oracle.torch_gemm(op, x, w, b, d0, d1).to(dtype).float()
    nres = _kernels.NUM_RESIDUALS_OF_EPILOGUE[_kernels.EPILOGUE_OF_OP[op]]
    dev = "cuda:0"
    got = eager.gemm(op, x.to(dev), w.to(dev), None if op == "gemm_rcr" else b.to(dev),
                     d0.to(dev) if nres >= 1 else None, d1.to(dev) if nres >= 2 else None, algo=algo)
    torch.cuda.synchronize()
    tol = tol or (ATOL if dtype == torch.float16 else 3e-2)
    torch.testing.assert_close(got.cpu().float(), want, atol=tol, rtol=tol)


ALL_OPS = sorted(set(_kernels.EPILOGUE_OF_OP) - {"bmm_rcr"})


@pytest.mark.parametrize("op", ALL_OPS)
def test_every_epilogue_small(op):
    print(f"case op={op} M=200 N=136 K=192", flush=True)
    _run_and_check(op, 200, 136, 192)


def _algo_cases():
    names = _kernels.gemm_algo_names(1, 0)
    return list(enumerate(names))


@pytest.mark.parametrize("algo,name", _algo_cases())
@pytest.mark.parametrize("shape", [(256, 256, 64), (300, 264, 200), (64, 520, 1024), (1, 8, 8), (515, 40, 72)])
def test_every_instance_with_tails(algo, name, shape):
    M, N, K = shape
    print(f"case instance={name} M={M} N={N} K={K}", flush=True)
    lib = _kernels.load()
    if not lib.aitamd_gemm_algo_supported(1, 0, algo, M, N, K, K, K, 16):
        pytest.skip("instance does not support this alignment")
    _run_and_check("gemm_rcr_bias", M, N, K, algo=algo, seed=algo)
    # instance tables differ per epilogue (the persistent kernels exist for residual-free epilogues only)
    algo5 = lib.aitamd_gemm_find_algo(5, 0, name.encode())
    if algo5 >= 0:
        _run_and_check("gemm_rcr_bias_add_add", M, N, K, algo=algo5, seed=algo + 50)


# shapes of the reference's ROCm tests for this family
def _k2_cases():
    return [(i, n) for i, n in enumerate(_kernels.gemm_algo_names(1, 0)) if n.endswith("_k2")]


@pytest.mark.parametrize("algo,name", _k2_cases())
@pytest.mark.parametrize("shape", [(300, 264, 202), (64, 522, 1028), (515, 41, 70), (130, 200, 6), (257, 130, 8314)])
def test_dword_aligned_k_instances(algo, name, shape):
    """K % 8 in {2, 4, 6}: rows of A and B start 4, 8 or 12 bytes off a 16-byte boundary.  The direct-to-LDS
    instances for such K load whole 16-byte pieces at dword-aligned addresses and take the 2, 4 or 6 elements
    behind them with dword loads; an Inf at the start of one row must stay in that row's results (the elements
    that follow a row's end in memory are the next row's first ones)."""
    M, N, K = shape
    print(f"case instance={name} M={M} N={N} K={K}", flush=True)
    lib = _kernels.load()
    assert lib.aitamd_gemm_algo_supported(1, 0, algo, M, N, K, K, K, 4)
    assert not lib.aitamd_gemm_algo_supported(1, 0, algo, M, N, K + 1, K + 1, K + 1, 4)   # odd K: 2-byte rows
    x = _rand((M, K), torch.float16, algo)
    w = _rand((N, K), torch.float16, algo + 1, scale=K ** -0.5)
    b = _rand((N,), torch.float16, algo + 2)
    hot = min(5, M - 1)
    x[hot, :min(6, K)] = float("inf")
    want = oracle.torch_gemm("gemm_rcr_bias", x, w, b).half().float()
    got = eager.gemm("gemm_rcr_bias", x.cuda(), w.cuda(), b.cuda(), algo=algo).cpu().float()
    keep = [r for r in range(M) if r != hot]
    torch.testing.assert_close(got[keep], want[keep], atol=ATOL, rtol=RTOL)
    assert not torch.isfinite(got[hot]).any()


@pytest.mark.parametrize("N,K", [(8314, 3072), (6912, 8314)])
@pytest.mark.parametrize("M", [1, 2048])
def test_reference_gemm_benchmark_shapes(M, N, K):
    """The reference's own GEMM benchmark (tests/unittest/benchmark/test_gemm_benchmark.py:31-37): gemm_rcr with
    N = 8314 (rows of the output start off 16-byte boundaries) and K = 8314 (so do the rows of both operands), on
    the instance the library picks.  |x.w| sums 8314 products: the tolerance is relative to sqrt(K) rounding."""
    print(f"case reference benchmark gemm_rcr M={M} N={N} K={K}", flush=True)
    lib = _kernels.load()
    algo = lib.aitamd_gemm_heuristic_algo(0, 0, 1, M, N, K, K, K, 4 if K % 8 else 16)
    name = _kernels.gemm_algo_names(0, 0)[algo]
    print(f"  instance {name}", flush=True)
    if K % 8:
        assert name.endswith("_k2"), name
    _run_and_check("gemm_rcr", M, N, K, seed=7)


@pytest.mark.parametrize("op,M,N,K", [
    ("gemm_rcr", 1024, 512, 256),            # test_gemm.py:83-84
    ("gemm_rcr_bias", 4096, 4, 4),           # test_gemm_bias.py:96-99
    ("gemm_rcr_bias", 1000, 81, 1024),
    ("gemm_rcr_bias", 67200, 3, 256),
    ("gemm_rcr_bias_relu", 128, 64, 1024),   # test_gemm_bias_relu.py:75-76
    ("gemm_rcr_bias_fast_gelu", 128, 64, 1024),
    ("gemm_rcr_bias_add", 8, 8, 8),          # test_gemm_bias_broadcast.py
    ("gemm_rcr_bias_add_add", 8, 8, 8),
    ("gemm_rcr_bias", 7, 3, 5),              # odd everything -> scalar loads and stores
    ("gemm_rcr_bias", 33, 6, 10),            # K % 2 == 0 only
])
def test_reference_test_shapes(op, M, N, K):
    print(f"case op={op} M={M} N={N} K={K}", flush=True)
    _run_and_check(op, M, N, K)


@pytest.mark.parametrize("op", ["gemm_rcr_bias", "gemm_rcr_bias_gelu", "gemm_rcr_bias_add_add"])
def test_bf16(op):
    print(f"case bf16 op={op}", flush=True)
    _run_and_check(op, 300, 264, 512, dtype=torch.bfloat16)


def test_leading_dims_are_flattened_and_views_with_pitch():
    dev = "cuda:0"
    x = _rand((4, 50, 64), torch.float16, 1).to(dev)
    w = _rand((72, 64), torch.float16, 2, 0.125).to(dev)
    b = _rand((72,), torch.float16, 3).to(dev)
    y = eager.gemm("gemm_rcr_bias", x, w, b)
    assert y.shape == (4, 50, 72)
    want = oracle.torch_gemm("gemm_rcr_bias", x.reshape(-1, 64), w, b).reshape(4, 50, 72)
    torch.testing.assert_close(y.cpu().float(), want, atol=ATOL, rtol=RTOL)
    # a strided view of A (row pitch 128 > K = 64) and a strided output
    xb = _rand((100, 128), torch.float16, 4).to(dev)
    xv = xb[:, :64]
    outb = torch.zeros(100, 144, dtype=torch.float16, device=dev)
    outv = outb[:, 72:]
    eager.gemm("gemm_rcr_bias", xv, w, b, out=outv)
    want = oracle.torch_gemm("gemm_rcr_bias", xv, w, b)
    torch.testing.assert_close(outv.cpu().float(), want, atol=ATOL, rtol=RTOL)
    assert float(outb[:, :72].abs().max()) == 0.0  # nothing written outside the view


def test_zero_sized_problems_are_noops():
    dev = "cuda:0"
    w = torch.zeros(4, 4, dtype=torch.float16, device=dev)
    b = torch.ones(4, dtype=torch.float16, device=dev)
    y = eager.gemm("gemm_rcr_bias", torch.zeros(0, 4, dtype=torch.float16, device=dev), w, b)
    assert y.shape == (0, 4)
    # K == 0: empty sum -> bias broadcast (what F.linear gives)
    y = eager.gemm("gemm_rcr_bias", torch.zeros(2, 0, dtype=torch.float16, device=dev),
                   torch.zeros(4, 0, dtype=torch.float16, device=dev), b)
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), torch.ones(2, 4, dtype=torch.float16))


def test_cpu_tensor_is_rejected_not_computed():
    x = torch.zeros(4, 8, dtype=torch.float16)
    with pytest.raises(ValueError):
        eager.gemm("gemm_rcr", x, x)


# ---- the benchmark configurations at full size -----------------------------
@pytest.mark.parametrize("cfg", ["c1", "c2a", "c2b", "c3"])
def test_config_full_size(cfg):
    print(f"case config={cfg} full size", flush=True)
    inp = oracle.config_inputs(cfg)
    want = oracle.config_expected(cfg, inp).half().float()
    dev = "cuda:0"
    got = eager.gemm(oracle.CONFIG_OP[cfg], inp["x"].to(dev), inp["w"].to(dev), inp["bias"].to(dev),
                     inp["d0"].to(dev) if "d0" in inp else None, inp["d1"].to(dev) if "d1" in inp else None)
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=ATOL, rtol=RTOL)


def test_c2a_every_large_instance_full_size():
    inp = oracle.config_inputs("c2a", m_override=2048 + 77)
    want = oracle.config_expected("c2a", inp).half().float()
    dev = "cuda:0"
    x, w, b = inp["x"].to(dev), inp["w"].to(dev), inp["bias"].to(dev)
    for algo, name in enumerate(_kernels.gemm_algo_names(3, 0)):
        if "_v8" not in name:
            continue
        print(f"case c2a instance={name}", flush=True)
        got = eager.gemm("gemm_rcr_bias_gelu", x, w, b, algo=algo)
        torch.cuda.synchronize()
        torch.testing.assert_close(got.cpu().float(), want, atol=ATOL, rtol=RTOL)


# ---- bmm_rcr -----------------------------------------------------------------
@pytest.mark.parametrize("B,M,N,K", [(3, 100, 72, 64), (1024, 128, 512, 256), (5, 33, 17, 24), (2, 16, 16, 6)])
def test_bmm_rcr(B, M, N, K):
    print(f"case bmm_rcr B={B} M={M} N={N} K={K}", flush=True)
    q = _rand((B, M, K), torch.float16, 1)
    k = _rand((B, N, K), torch.float16, 2, K ** -0.5)
    want = oracle.torch_bmm_rcr(q, k).half().float()
    got = eager.bmm_rcr(q.cuda(), k.cuda())
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=ATOL, rtol=RTOL)


def test_bmm_rcr_broadcast_operands():
    q = _rand((6, 40, 32), torch.float16, 1)
    k = _rand((1, 24, 32), torch.float16, 2, 0.2)
    want = oracle.torch_bmm_rcr(q, k).half().float()
    got = eager.bmm_rcr(q.cuda(), k.cuda())
    got2 = eager.bmm_rcr(q.cuda(), k[0].cuda())
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=ATOL, rtol=RTOL)
    assert torch.equal(got, got2)


def test_config_c4_full_size():
    inp = oracle.config_inputs("c4")
    want = oracle.config_expected("c4", inp).half().float()
    got = eager.bmm_rcr(inp["q"].cuda(), inp["k"].cuda())
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=ATOL, rtol=RTOL)
