"""GPU parity of the permuting GEMMs (gemm_rcr_permute_m2n3, gemm_rcr_bias_permute[_m2n3|_m3n2]) through
the C ABI.  Two checks per case: against the CPU oracle at the family's tolerance (atol = rtol = 1e-2 for
fp16, 3e-2 for bf16), and bit for bit against the same instance's plain store permuted on the host: the
permutation moves elements, it must not change them.  Shapes follow the reference's
tests/unittest/ops/test_gemm_bias_permute.py:34-42,100-108 and test_gemm_permute.py, plus tails and
unaligned inner dims."""
import pytest
import torch

from aitemplate_amd import _kernels, eager
from oracle import oracle

pytestmark = pytest.mark.gpu


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _case(op, M, N, K, shape, dtype=torch.float16, algo=-1, seed=0):
    print(f"case {op} M={M} N={N} K={K} shape={shape} {dtype} algo={algo}", flush=True)
    base, layout = oracle.PERMUTE_OPS[op]
    x, w = _rand((M, K), dtype, seed), _rand((N, K), dtype, seed + 1, max(K, 1) ** -0.5)
    b = None if base == "gemm_rcr" else _rand((N,), dtype, seed + 2)
    dev = "cuda:0"
    xd, wd, bd = x.to(dev), w.to(dev), None if b is None else b.to(dev)
    got = eager.gemm_permute(op, xd, wd, bd, shape, algo=algo)
    plain = eager.gemm(base, xd, wd, bd, algo=algo)
    torch.cuda.synchronize()
    want = oracle.torch_gemm_permute(op, x, w, b, shape)
    assert tuple(got.shape) == tuple(want.shape)
    tol = 1e-2 if dtype == torch.float16 else 3e-2
    torch.testing.assert_close(got.cpu().float(), want.to(dtype).float(), atol=tol, rtol=tol)
    assert torch.equal(got.cpu(), oracle.permute_5d(plain.cpu(), layout, shape))


def test_reference_shapes():
    _case("gemm_rcr_bias_permute_m2n3", 4 * 256, 4 * 16 * 128, 256, (256, 4, 16))
    _case("gemm_rcr_permute_m2n3", 4 * 256, 4 * 16 * 128, 256, (256, 4, 16))
    _case("gemm_rcr_bias_permute_m3n2", 4 * 16 * 32, 8 * 128, 256, (16, 32, 8))
    _case("gemm_rcr_bias_permute", 4 * 16 * 32, 8 * 128, 256, (16, 32, 8))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,S,D,H", [(2, 384, 768, 12), (3, 197, 768, 12), (1, 64, 1280, 20), (5, 77, 96, 4)])
def test_packed_qkv_projection(B, S, D, H, dtype):
    """shape = (seq, 3, heads): what nn.MultiheadAttention asks for; S = 197 and 77 leave tile tails and
    head_dim = 24 (D = 96, H = 4) keeps the 8-wide stores aligned while N2 is no power of two."""
    _case("gemm_rcr_bias_permute_m2n3", B * S, 3 * D, D, (S, 3, H), dtype)
    _case("gemm_rcr_permute_m2n3", B * S, 3 * D, D, (S, 3, H), dtype)


@pytest.mark.parametrize("op,M,N,K,shape", [
    ("gemm_rcr_bias_permute_m2n3", 6 * 35, 2 * 3 * 5, 40, (35, 2, 3)),     # N2 = 5: element-wise stores
    ("gemm_rcr_bias_permute_m2n3", 8 * 33, 3 * 2 * 12, 72, (33, 3, 2)),    # N2 = 12: 4-wide only
    ("gemm_rcr_bias_permute_m3n2", 3 * 7 * 5, 4 * 9, 24, (7, 5, 4)),       # N1 = 9
    ("gemm_rcr_bias_permute_m3n2", 1 * 1 * 300, 1 * 264, 200, (1, 300, 1)),
    ("gemm_rcr_permute_m2n3", 515, 40, 72, (515, 1, 1)),                  # identity permutation
    ("gemm_rcr_permute_m2n3", 515, 40, 72, (1, 5, 1)),
    ("gemm_rcr_bias_permute", 2 * 3 * 4, 5 * 8, 9, (3, 4, 5)),            # odd K
])
def test_tails_and_unaligned_inner_dims(op, M, N, K, shape):
    _case(op, M, N, K, shape)


def _algos():
    return list(enumerate(_kernels.gemm_algo_names(1, 0)))


@pytest.mark.parametrize("algo,name", _algos())
def test_every_instance_stores_permuted(algo, name):
    lib = _kernels.load()
    for op, M, N, K, shape in (("gemm_rcr_bias_permute_m2n3", 2 * 150, 3 * 2 * 88, 200, (150, 3, 2)),
                               ("gemm_rcr_bias_permute_m3n2", 3 * 10 * 11, 6 * 40, 64, (10, 11, 6)),
                               ("gemm_rcr_bias_permute_m2n3", 4 * 256, 3 * 4 * 64, 256, (256, 3, 4))):
        if not lib.aitamd_gemm_algo_supported(1, 0, algo, M, N, K, K, K, 16):
            continue
        _case(op, M, N, K, shape, algo=algo, seed=algo)


def test_argument_errors():
    x = torch.zeros(12, 8, dtype=torch.float16, device="cuda:0")
    w = torch.zeros(24, 8, dtype=torch.float16, device="cuda:0")
    b = torch.zeros(24, dtype=torch.float16, device="cuda:0")
    with pytest.raises(ValueError, match="does not split"):
        eager.gemm_permute("gemm_rcr_bias_permute_m2n3", x, w, b, (5, 3, 2))
    lib = _kernels.load()
    out = torch.empty(12 * 24, dtype=torch.float16, device="cuda:0")
    args = (x.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(), 12, 24, 8, 8, 8)
    assert lib.aitamd_gemm_rcr_permute(1, 0, -1, *args, 1, 5, 3, 2, None) != 0        # 5 does not divide M
    assert b"m2n3" in lib.aitamd_last_error()
    assert lib.aitamd_gemm_rcr_permute(1, 0, -1, *args, 7, 4, 3, 2, None) != 0        # unknown layout
    assert lib.aitamd_gemm_rcr_permute(4, 0, -1, *args, 1, 4, 3, 2, None) != 0        # residual epilogue
    assert lib.aitamd_gemm_rcr_permute(1, 0, -1, x.data_ptr(), w.data_ptr(), None, out.data_ptr(),
                                       12, 24, 8, 8, 8, 1, 4, 3, 2, None) != 0           # bias missing
    assert lib.aitamd_gemm_rcr_permute(1, 0, -1, *args, 1, 4, 3, 2, None) == 0
    torch.cuda.synchronize()


# ---- bmm_rcr_permute ------------------------------------------------------------------------
@pytest.mark.parametrize("B,M,N,K,d1", [
    (10240, 88, 64, 88, 10), (24, 80, 64, 88, 12), (100, 88, 64, 88, 10),     # tests/unittest/ops/test_bmm_permute.py:109-117
    (768, 384, 384, 64, 12),                                                   # attention scores of BERT-base, per head
    (6, 33, 20, 24, 3), (4, 1, 8, 8, 4), (5, 130, 72, 40, 1),
])
def test_bmm_rcr_permute(B, M, N, K, d1):
    print(f"case bmm_rcr_permute B={B} M={M} N={N} K={K} d1={d1}", flush=True)
    q, k = _rand((B, M, K), torch.float16, 1), _rand((B, N, K), torch.float16, 2, K ** -0.5)
    qd, kd = q.cuda(), k.cuda()
    got = eager.bmm_rcr_permute(qd, kd, (d1,))
    plain = eager.bmm_rcr(qd, kd)
    torch.cuda.synchronize()
    assert tuple(got.shape) == (B // d1, M, d1, N)
    # the permutation moves elements of the plain result, bit for bit (same heuristic instance: same shape)
    assert torch.equal(got.cpu(), plain.cpu().reshape(B // d1, d1, M, N).permute(0, 2, 1, 3))
    if B * M * N <= 1 << 24:
        want = oracle.torch_bmm_rcr_permute(q, k, d1).half().float()
        torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)


def test_bmm_rcr_permute_every_instance_and_errors():
    B, M, N, K, d1 = 12, 200, 136, 72, 4
    q, k = _rand((B, M, K), torch.float16, 3).cuda(), _rand((B, N, K), torch.float16, 4, K ** -0.5).cuda()
    lib = _kernels.load()
    for algo, name in enumerate(_kernels.gemm_algo_names(0, 0)):
        if not lib.aitamd_gemm_algo_supported(0, 0, algo, M, N, K, K, K, 16):
            continue
        print(f"case bmm_rcr_permute instance={name}", flush=True)
        got = eager.bmm_rcr_permute(q, k, (d1,), algo=algo)
        plain = eager.bmm_rcr(q, k, algo=algo)
        torch.cuda.synchronize()
        assert torch.equal(got, plain.reshape(B // d1, d1, M, N).permute(0, 2, 1, 3))
    with pytest.raises(ValueError, match="multiple"):
        eager.bmm_rcr_permute(q, k, (5,))
    out = torch.empty(B * M * N, dtype=torch.float16, device="cuda")
    assert lib.aitamd_bmm_rcr_permute(0, -1, q.data_ptr(), k.data_ptr(), out.data_ptr(), B, M, N, K, K, K, M * K,
                                      N * K, 5, None) != 0
    assert b"multiple" in lib.aitamd_last_error()
