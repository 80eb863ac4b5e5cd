"""GPU parity of the persistent GEMM instances (one workgroup per CU walks its tiles, the LDS ring
runs across tile boundaries): many tiles per workgroup, fewer tiles than CUs, single-slab K, K
tails, M/N tails, the scalar-store path (N not a multiple of 8), strided views, batches, bf16,
every epilogue.  Tiles of an even number of K-slabs, 16 or more, run the slab-pair form of the kernel
where the instance has one: the shapes below cover both forms and the switch between them."""
import pytest
import torch

from aitemplate_amd import _kernels, eager
from oracle import oracle

pytestmark = pytest.mark.gpu


def _persist_names(epi=1, dtype=0):
    return [n for n in _kernels.gemm_algo_names(epi, dtype) if "_persist" in n]


def _algo(op, name, dtype=0):
    a = _kernels.load().aitamd_gemm_find_algo(_kernels.EPILOGUE_OF_OP[op], dtype, name.encode())
    assert a >= 0, (op, name)
    return a


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _check(op, name, M, N, K, dtype=torch.float16, seed=0):
    print(f"case op={op} instance={name} M={M} N={N} K={K} dtype={dtype}", flush=True)
    x = _rand((M, K), dtype, seed)
    w = _rand((N, K), dtype, seed + 1, scale=max(K, 1) ** -0.5)
    b = _rand((N,), dtype, seed + 2)
    d0 = _rand((M, N), dtype, seed + 3)
    d1 = _rand((M, N), dtype, seed + 4)
    want = oracle.torch_gemm(op, x, w, b, d0, d1).to(dtype).float()
    nres = _kernels.NUM_RESIDUALS_OF_EPILOGUE[_kernels.EPILOGUE_OF_OP[op]]
    dname = name.replace("_f16_", "_bf16_") if dtype == torch.bfloat16 else name
    got = eager.gemm(op, x.cuda(), w.cuda(), None if op == "gemm_rcr" else b.cuda(),
                     d0.cuda() if nres >= 1 else None, d1.cuda() if nres >= 2 else None,
                     algo=_algo(op, dname, 0 if dtype == torch.float16 else 1))
    torch.cuda.synchronize()
    tol = 1e-2 if dtype == torch.float16 else 3e-2
    torch.testing.assert_close(got.cpu().float(), want, atol=tol, rtol=tol)


def test_persist_instances_exist():
    assert _persist_names(), "no persistent instance compiled in"
    assert [n for n in _kernels.gemm_algo_names(5, 0) if "_persist" in n]
    # a tile is written when its last K-slab has been multiplied: K = 0 is not for these instances
    lib = _kernels.load()
    for name in _persist_names():
        a = _algo("gemm_rcr_bias", name)
        assert lib.aitamd_gemm_algo_supported(1, 0, a, 64, 64, 0, 0, 0, 16) == 0
        assert lib.aitamd_gemm_algo_supported(1, 0, a, 64, 64, 8, 8, 8, 16) == 1


@pytest.mark.parametrize("name", _persist_names())
@pytest.mark.parametrize("shape", [
    (256, 256, 64),      # one tile, two slabs
    (256, 256, 32),      # one tile, a single slab
    (300, 264, 200),     # M / N / K tails
    (1, 8, 8),           # smallest aligned problem
    (515, 40, 72),
    (64, 520, 1024),
    (2048, 1536, 256),   # 48 tiles < CUs
    (8192, 3072, 768),   # 384 tiles: one or two per workgroup
    (12608, 1024, 96),   # unaligned M, three slabs
    (4000, 4352, 64),    # 272 tiles on 256 CUs: the 16 leftover tiles are split in halves; M tail of 160 rows
    (3900, 4352, 64),    # same, M tail of 60 rows: some lower halves lie wholly below M
    (24576, 768, 128),   # 288 tiles: one full round plus 32 split tiles
    (1000, 392, 512),    # 16 slabs: the shortest tile of the slab-pair form
    (515, 264, 1000),    # 32 slabs, the last one ragged (K tail inside a pair)
    (300, 264, 520),     # 17 slabs: odd, the one-slab form
    (4000, 4352, 576),   # 18 slabs, 272 tiles: pairs across tile boundaries, leftover tiles split in halves
    (3900, 4352, 512),   # same with lower halves wholly below M (waves that load but do not multiply)
    (2048, 1536, 2048),  # 48 tiles of 64 slabs
])
def test_persist_shapes(name, shape):
    M, N, K = shape
    _check("gemm_rcr_bias_gelu", name, M, N, K, seed=sum(shape))
    _check("gemm_rcr_bias_add_add", name, M, N, K, seed=sum(shape) + 1)


@pytest.mark.parametrize("name", _persist_names())
@pytest.mark.parametrize("op", sorted(set(_kernels.EPILOGUE_OF_OP) - {"bmm_rcr"}))
def test_persist_every_epilogue(name, op):
    _check(op, name, 1000, 392, 320, seed=7)
    _check(op, name, 1000, 392, 640, seed=8)   # 20 slabs: the slab-pair form


@pytest.mark.parametrize("name", _persist_names())
def test_persist_scalar_store_path(name):
    # N not a multiple of 8 -> element-wise stores and bias reads
    _check("gemm_rcr_bias_gelu", name, 333, 100, 64, seed=3)
    _check("gemm_rcr_bias_add", name, 700, 250, 160, seed=4)
    _check("gemm_rcr_bias_add", name, 700, 250, 1024, seed=5)


@pytest.mark.parametrize("name", _persist_names())
def test_persist_bf16(name):
    _check("gemm_rcr_bias_gelu", name, 1024, 768, 512, dtype=torch.bfloat16, seed=11)


@pytest.mark.parametrize("name", _persist_names())
def test_persist_full_headline_shape(name):
    inp = oracle.config_inputs("c2a")
    want = oracle.config_expected("c2a", inp).half().float()
    got = eager.gemm("gemm_rcr_bias_gelu", inp["x"].cuda(), inp["w"].cuda(), inp["bias"].cuda(),
                     algo=_algo("gemm_rcr_bias_gelu", name))
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("name", _persist_names())
def test_persist_bmm_batches_and_views(name):
    # batch folded into the persistent tile walk; output and operand pitches larger than the rows
    a = _rand((6, 300, 64), torch.float16, 1, 0.25).cuda()
    b = _rand((6, 200, 64), torch.float16, 2, 0.25).cuda()
    want = oracle.torch_bmm_rcr(a.cpu(), b.cpu()).half().float()
    got = eager.bmm_rcr(a, b, algo=_algo("gemm_rcr", name))
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)
    # the same with 18 K-slabs per tile: the slab-pair form, pairs handed over from one batch entry to the next
    a = _rand((5, 300, 576), torch.float16, 3, 0.25).cuda()
    b = _rand((5, 264, 576), torch.float16, 4, 0.25).cuda()
    want = oracle.torch_bmm_rcr(a.cpu(), b.cpu()).half().float()
    got = eager.bmm_rcr(a, b, algo=_algo("gemm_rcr", name))
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)
    wide = _rand((300, 2048), torch.float16, 8).cuda()
    xv = wide[:, 256:256 + 1024]                 # row pitch 2048, offset 256, 32 slabs
    wv = _rand((264, 1024), torch.float16, 9, 1024 ** -0.5).cuda()
    bv = _rand((264,), torch.float16, 10).cuda()
    want = oracle.torch_gemm("gemm_rcr_bias", xv.cpu(), wv.cpu(), bv.cpu()).half().float()
    got = eager.gemm("gemm_rcr_bias", xv, wv, bv, algo=_algo("gemm_rcr_bias", name))
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)
    big = _rand((500, 512), torch.float16, 5).cuda()
    x = big[:, 64:64 + 256]                      # row pitch 512, offset 64
    w = _rand((264, 256), torch.float16, 6, 256 ** -0.5).cuda()
    bias = _rand((264,), torch.float16, 7).cuda()
    want = oracle.torch_gemm("gemm_rcr_bias", x.cpu(), w.cpu(), bias.cpu()).half().float()
    got = eager.gemm("gemm_rcr_bias", x, w, bias, algo=_algo("gemm_rcr_bias", name))
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-2, rtol=1e-2)
