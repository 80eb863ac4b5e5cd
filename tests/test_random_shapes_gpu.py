"""Seeded random-shape parity sweeps on the GPU: every case draws an op, a dtype and ragged sizes (1 ... 1024, most
of them not multiples of any tile edge or load width) and compares the C-ABI result with the CPU oracle at the
tolerance of the reference's own tests (atol = rtol = 1e-2 for fp16 GEMMs, tests/unittest/ops/test_gemm_bias.py:69;
2e-2 on the softmax path, test_bmm_softmax_bmm.py:114; bf16 three / two times that).  The fixed-shape tests cover
the reference's shapes and every instance; these cover what nobody thought of."""
import random

import pytest
import torch

from aitemplate_amd import _kernels, eager
from oracle import oracle

pytestmark = pytest.mark.gpu

DIMS = [1, 3, 8, 15, 16, 17, 31, 32, 33, 40, 64, 65, 72, 100, 128, 130, 200, 256, 264, 300, 512, 520, 768, 1000, 1024]


def _close(got, want, tol):
    err = (got.cpu().float() - want).abs()
    return bool((err <= tol + tol * want.abs()).all()), float(err.max())


def _dev(t):
    return None if t is None else t.cuda()


def test_gemm_rcr_family_random_shapes():
    rng = random.Random(7)
    ops = [o for o in sorted(_kernels.EPILOGUE_OF_OP) if o.startswith("gemm_rcr")]
    for i in range(150):
        op = rng.choice(ops)
        epi = _kernels.EPILOGUE_OF_OP[op]
        nres = _kernels.NUM_RESIDUALS_OF_EPILOGUE[epi]
        M, N, K = rng.choice(DIMS + [2048, 4096]), rng.choice(DIMS), rng.choice(DIMS)
        dtype = torch.float16 if rng.random() < 0.7 else torch.bfloat16
        g = torch.Generator().manual_seed(i)
        x = torch.randn(M, K, generator=g).to(dtype)
        w = (torch.randn(N, K, generator=g) * K ** -0.5).to(dtype)
        bias = (torch.rand(N, generator=g) * 0.2 - 0.1).to(dtype) if epi not in (0, _kernels.EPI_ADD) else None
        d0 = torch.randn(M, N, generator=g).to(dtype) if nres >= 1 else None
        d1 = torch.randn(M, N, generator=g).to(dtype) if nres >= 2 else None
        print(f"case {i} {op} M={M} N={N} K={K} {dtype}", flush=True)
        want = oracle.torch_gemm(op, x, w, bias, d0, d1).to(dtype).float()
        got = eager.gemm(op, x.cuda(), w.cuda(), _dev(bias), _dev(d0), _dev(d1))
        torch.cuda.synchronize()
        ok, err = _close(got, want, 1e-2 if dtype == torch.float16 else 3e-2)
        assert ok, f"case {i} {op} M={M} N={N} K={K} {dtype}: max error {err}"


def test_bmm_layouts_random_shapes():
    rng = random.Random(99)
    dims = [1, 2, 3, 7, 8, 15, 16, 17, 31, 33, 40, 63, 64, 65, 72, 100, 127, 128, 130, 200, 255, 256, 264, 300, 520]
    for i in range(150):
        layout = rng.choice(["rcr", "rrr", "ccr", "crr"])
        B = rng.choice([1, 2, 3, 5])
        M, N, K = rng.choice(dims), rng.choice(dims), rng.choice(dims)
        dtype = torch.float16 if rng.random() < 0.7 else torch.bfloat16
        add = rng.random() < 0.4
        g = torch.Generator().manual_seed(i)
        a = torch.randn((B, K, M) if layout[0] == "c" else (B, M, K), generator=g).to(dtype)
        b = (torch.randn((B, N, K) if layout[1] == "c" else (B, K, N), generator=g) * K ** -0.5).to(dtype)
        d = torch.randn(B, M, N, generator=g).to(dtype)
        print(f"case {i} bmm_{layout} B={B} M={M} N={N} K={K} {dtype} add={add}", flush=True)
        want = oracle.torch_bmm(layout, a, b)
        if add:
            want = want + d.float()
            got = eager.bmm_add(layout, a.cuda(), b.cuda(), d.cuda())
        elif layout == "rcr":
            got = eager.bmm_rcr(a.cuda(), b.cuda())
        else:
            got = eager.bmm(layout, a.cuda(), b.cuda())
        torch.cuda.synchronize()
        ok, err = _close(got, want.to(dtype).float(), 1e-2 if dtype == torch.float16 else 3e-2)
        assert ok, f"case {i} bmm_{layout} B={B} M={M} N={N} K={K} {dtype} add={add}: max error {err}"


def test_attention_random_shapes(attn_variant):
    rng = random.Random(1234)
    for i in range(150):
        G = rng.choice([1, 2, 4, 8])
        B = G * rng.choice([1, 2, 3, 8])
        M = rng.choice([1, 7, 31, 32, 33, 100, 128, 129, 255, 256, 257, 300, 511, 700])
        N = rng.choice([1, 5, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 256, 300, 383, 384, 500, 777, 1024])
        K = rng.choice([8, 16, 24, 32, 40, 48, 64, 72, 96, 128, 160])
        O = rng.choice([8, 16, 32, 40, 64, 96, 128, 160])
        causal = rng.random() < 0.4
        dtype = torch.float16 if rng.random() < 0.7 else torch.bfloat16
        scale = rng.choice([K ** -0.5, K ** -0.5, 0.3, -0.2, 1.0 / 8])
        mode = rng.choice([None, 0, 1, 2, 3])  # kernel variant, where the head dims allow the choice
        if mode is None:
            attn_variant(-1)
        else:
            attn_variant(mode)
        g = torch.Generator().manual_seed(i)
        q = torch.randn(B, M, K, generator=g).to(dtype)
        k = torch.randn(B, N, K, generator=g).to(dtype)
        v = torch.randn(B, N, O, generator=g).to(dtype)
        print(f"case {i} attention B={B} M={M} N={N} K={K} O={O} G={G} causal={causal} {dtype} scale={scale:.4f} "
              f"mode={mode}", flush=True)
        want = oracle.torch_bmm_softmax_bmm_permute(q, k, v, scale, G, causal).to(dtype).float()
        got = eager.bmm_softmax_bmm_permute(q.cuda(), k.cuda(), v.cuda(), (G,), scale=scale, causal=causal)
        torch.cuda.synchronize()
        ok, err = _close(got, want, 2e-2 if dtype == torch.float16 else 4e-2)
        assert ok, f"case {i}: max error {err}"


def test_mem_eff_attention_random_shapes_and_key_lengths(attn_variant):
    rng = random.Random(4321)
    for i in range(100):
        heads = rng.choice([1, 2, 4, 8])
        batch = rng.choice([1, 2, 3, 5])
        S = rng.choice([1, 31, 33, 100, 128, 129, 256, 300, 511])
        Skv = rng.choice([1, 5, 33, 64, 77, 127, 128, 129, 200, 256, 300, 383, 500, 777, 1024])
        d = rng.choice([8, 16, 20, 32, 40, 64, 96, 128, 160])
        dv = rng.choice([8, 16, 24, 40, 64, 128, 160])
        causal = rng.random() < 0.3
        dtype = torch.float16 if rng.random() < 0.7 else torch.bfloat16
        mode = rng.choice([None, 0, 1, 2, 3])
        if mode is None:
            attn_variant(-1)
        else:
            attn_variant(mode)
        lens = None
        if rng.random() < 0.8:
            lens = torch.tensor([rng.choice([0, 1, Skv, Skv // 2, rng.randint(0, Skv)]) for _ in range(batch)],
                                dtype=torch.int32)
        g = torch.Generator().manual_seed(1000 + i)
        q = torch.randn(batch, heads, S, d, generator=g).to(dtype)
        k = torch.randn(batch, heads, Skv, d, generator=g).to(dtype)
        v = torch.randn(batch, heads, Skv, dv, generator=g).to(dtype)
        print(f"case {i} mem_eff_attention batch={batch} heads={heads} S={S} Skv={Skv} d={d} dv={dv} causal={causal} "
              f"{dtype} mode={mode} lens={None if lens is None else lens.tolist()}", flush=True)
        want = oracle.torch_mem_eff_attention(q, k, v, causal, lens).to(dtype).float()
        if lens is not None:
            for b in range(batch):  # rows past the length must not be read
                k[b, :, int(lens[b]):] = float("nan")
                v[b, :, int(lens[b]):] = float("nan")
        got = eager.mem_eff_attention(q.cuda(), k.cuda(), v.cuda(), causal=causal,
                                      lengths_kv=None if lens is None else lens.cuda())
        torch.cuda.synchronize()
        ok, err = _close(got, want, 2e-2 if dtype == torch.float16 else 4e-2)
        assert ok, f"case {i}: max error {err}"
