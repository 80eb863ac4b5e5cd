"""GPU parity of the batched GEMMs whose operands are not both K-contiguous (bmm_rrr, bmm_ccr, bmm_crr, gemm_rrr,
bmm_rrr_permute) through the C ABI, against the CPU oracle at atol = rtol = 1e-2 (the reference's tolerance,
tests/unittest/ops/test_bmm.py:57,96,129,160).  The transposed operand goes through LDS as it lies in memory and
is gathered with transposing LDS reads, so every instance that has these kernels is checked on shapes with
tails in M, N and K."""
import pytest
import torch

from aitemplate_amd import _kernels, eager
from oracle import oracle

pytestmark = pytest.mark.gpu
LAYOUTS = ["rrr", "ccr", "crr"]


def _rand(shape, seed, scale=1.0, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _operands(layout, B, M, N, K, dtype=torch.float16, seed=0):
    a = _rand((B, K, M) if layout[0] == "c" else (B, M, K), seed, dtype=dtype)
    b = _rand((B, N, K) if layout[1] == "c" else (B, K, N), seed + 1, K ** -0.5, dtype)
    return a, b


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("B,M,N,K", [
    (1024, 128, 512, 256),     # test_bmm.py:61,100 (static rcr / crr shapes)
    (87, 23, 512, 256),        # test_bmm.py:133 (rrr)
    (77, 256, 64, 128),        # test_bmm.py:163 (ccr)
    (5, 256, 512, 56), (3, 200, 136, 72), (2, 515, 40, 1024), (768, 384, 64, 384),
    # pitches and K that are not multiples of 8: the element-wide instance
    (3, 23, 37, 45), (2, 65, 130, 7), (4, 100, 36, 64), (1, 1, 1, 1),
])
def test_reference_and_ragged_shapes(layout, B, M, N, K):
    print(f"case bmm_{layout} B={B} M={M} N={N} K={K}", flush=True)
    a, b = _operands(layout, B, M, N, K)
    got = eager.bmm(layout, a.cuda(), b.cuda())
    torch.cuda.synchronize()
    want = oracle.torch_bmm(layout, a, b).half().float()
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_every_instance_with_tails_bf16_and_broadcast(layout):
    lib = _kernels.load()
    lay = _kernels.LAYOUT_ID[layout]
    ran = 0
    for dtype, dt_id in ((torch.float16, 0), (torch.bfloat16, 1)):
        for (B, M, N, K) in [(2, 256, 256, 64), (3, 200, 136, 72), (1, 64, 520, 1024), (2, 515, 40, 72), (2, 104, 88, 33)]:
            a, b = _operands(layout, B, M, N, K, dtype, seed=B + M)
            ad, bd = a.cuda(), b.cuda()
            want = oracle.torch_bmm(layout, a, b).to(dtype).float()
            for algo, name in enumerate(_kernels.gemm_algo_names(0, dt_id)):
                if not lib.aitamd_gemm_algo_supported_layout(0, dt_id, lay, algo, M, N, K, a.shape[2], b.shape[2], 16):
                    continue
                print(f"case bmm_{layout} {dtype} B={B} M={M} N={N} K={K} instance={name}", flush=True)
                got = eager.bmm(layout, ad, bd, algo=algo)
                torch.cuda.synchronize()
                tol = 1e-2 if dtype == torch.float16 else 3e-2
                torch.testing.assert_close(got.cpu().float(), want, atol=tol, rtol=tol)
                ran += 1
    assert ran >= 20
    # a 2-D operand broadcasts over the batch of the other (bmm.py:72-90 of the reference ops)
    a, b = _operands(layout, 4, 96, 80, 64, seed=9)
    got = eager.bmm(layout, a.cuda(), b[0].cuda())
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), oracle.torch_bmm(layout, a, b[:1]).half().float(), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("B,M,N,K,d1", [(24, 80, 88, 64, 12), (10240, 88, 88, 64, 10), (100, 88, 88, 64, 10)])
def test_bmm_rrr_permute(B, M, N, K, d1):       # tests/unittest/ops/test_bmm_permute.py:66-71
    print(f"case bmm_rrr_permute B={B} M={M} N={N} K={K} d1={d1}", flush=True)
    a, b = _operands("rrr", B, M, N, K)
    got = eager.bmm("rrr", a.cuda(), b.cuda(), d1=d1)
    plain = eager.bmm("rrr", a.cuda(), b.cuda())
    torch.cuda.synchronize()
    assert tuple(got.shape) == (B // d1, M, d1, N)
    assert torch.equal(got.cpu(), plain.cpu().reshape(B // d1, d1, M, N).permute(0, 2, 1, 3))
    if B <= 1024:
        want = oracle.torch_bmm("rrr", a, b).reshape(B // d1, d1, M, N).permute(0, 2, 1, 3).half().float()
        torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)


def test_odd_pitch_takes_the_element_wide_instance():
    lib = _kernels.load()
    # B is [K, N] with N = 36: rows of 72 bytes cannot be fetched in 16-byte pieces, so only the instance with
    # element-wide loads qualifies (the reference narrows its loads the same way, backend/rocm/gemm/common.py:945-1020)
    a, b = _operands("rrr", 2, 64, 36, 64)
    algo = lib.aitamd_gemm_heuristic_algo_layout(0, 0, 1, 2, 64, 36, 64, 64, 36, 16)
    assert algo >= 0 and _kernels.gemm_algo_names(0, 0)[algo].endswith("_v1")
    got = eager.bmm("rrr", a.cuda(), b.cuda())
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), oracle.torch_bmm("rrr", a, b).half().float(), atol=1e-2, rtol=1e-2)
    # an unknown layout id is an error, not a crash
    assert lib.aitamd_bmm(7, 0, -1, None, None, None, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0, None) != 0


# ---- residual add and the rrr bias + permuted store ---------------------------------------------
@pytest.mark.parametrize("layout,B,M,N,K", [
    ("rrr", 32, 256, 512, 256), ("ccr", 32, 256, 256, 512), ("crr", 32, 256, 512, 256),   # test_bmm_add.py:286-302
    ("rcr", 6, 200, 136, 72), ("rrr", 3, 200, 136, 72), ("ccr", 5, 104, 88, 40), ("crr", 2, 520, 64, 33),
    ("rrr", 3, 23, 37, 45), ("ccr", 2, 65, 30, 7), ("crr", 2, 33, 36, 20),
])
def test_bmm_add(layout, B, M, N, K):
    print(f"case bmm_{layout}_add B={B} M={M} N={N} K={K}", flush=True)
    a, b = _operands(layout, B, M, N, K)
    d = _rand((B, M, N), 7)
    got = eager.bmm_add(layout, a.cuda(), b.cuda(), d.cuda())
    torch.cuda.synchronize()
    want = (oracle.torch_bmm(layout, a, b) + d.float()).half().float()
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)


def test_bmm_add_every_instance():
    lib = _kernels.load()
    B, M, N, K = 2, 200, 136, 72
    for layout in ("rcr", "rrr", "ccr", "crr"):
        lay = _kernels.LAYOUT_ID[layout]
        a, b = _operands(layout, B, M, N, K, seed=lay)
        d = _rand((B, M, N), 11)
        want = (oracle.torch_bmm(layout, a, b) + d.float()).half().float()
        ad, bd, dd = a.cuda(), b.cuda(), d.cuda()
        ran = 0
        for algo, name in enumerate(_kernels.gemm_algo_names(_kernels.EPI_ADD, 0)):
            if not lib.aitamd_gemm_algo_supported_layout(_kernels.EPI_ADD, 0, lay, algo, M, N, K, a.shape[2], b.shape[2], 16):
                continue
            print(f"case bmm_{layout}_add instance={name}", flush=True)
            got = eager.bmm_add(layout, ad, bd, dd, algo=algo)
            torch.cuda.synchronize()
            torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)
            ran += 1
        assert ran >= 5


@pytest.mark.parametrize("M,N,K,shape", [(4 * 32 * 128, 16 * 256, 128, (32, 128, 16)),   # test_gemm_bias_permute.py:250-280
                                         (3 * 7 * 8, 5 * 16, 24, (7, 8, 5)), (2 * 3 * 100, 4 * 72, 200, (3, 100, 4))])
def test_gemm_rrr_bias_permute(M, N, K, shape):
    print(f"case gemm_rrr_bias_permute M={M} N={N} K={K} shape={shape}", flush=True)
    x, w, bias = _rand((M, K), 1), _rand((K, N), 2, K ** -0.5), _rand((N,), 3)
    got = eager.gemm_permute("gemm_rrr_bias_permute", x.cuda(), w.cuda(), bias.cuda(), shape)
    torch.cuda.synchronize()
    t1, t2, t3 = shape
    y = oracle.torch_bmm("rrr", x, w)[0] + bias.float()
    want = oracle.permute_5d(y, "m3n2", shape).half().float()
    assert tuple(got.shape) == (t2, M // (t1 * t2), t3, t1, N // t3)
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)
