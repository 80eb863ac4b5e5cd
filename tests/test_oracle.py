"""Pins of the CPU oracle (no GPU).  The reference holds no golden vectors for the
GEMM path, so the oracle is pinned by what the mathematics fixes: brute force on
tiny inputs, special cases that reduce to library routines, and invariants chosen
so that a dropped term, a transposed operand or a wrong permute fails one of them."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle


def _rand(shape, dtype=torch.float16, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


# ---- number formats ---------------------------------------------------------
def test_c_half_conversion_matches_numpy_for_every_half_and_random_floats():
    lib = oracle.c_lib()
    # identity GEMM with K=1: c = fp16(a * 1) exercises half->float->half on every finite half
    bits = np.arange(0, 1 << 16, dtype=np.uint16)
    finite = bits[((bits & 0x7C00) != 0x7C00) & (bits != 0x8000)]  # 0 + (-0) is +0: skip -0
    x = torch.from_numpy(finite.view(np.float16).copy()).reshape(-1, 1)
    one = torch.ones(1, 1, dtype=torch.float16)
    y = oracle.c_gemm("gemm_rcr", x, one)
    assert np.array_equal(y.numpy().view(np.uint16).ravel(), finite)
    # rounding: sums of two halves need a real float->half rounding; numpy is the library routine
    rng = np.random.default_rng(0)
    a = rng.standard_normal((512, 2)).astype(np.float16)
    a[:, 0] *= np.float16(1000.0)
    ones = torch.ones(1, 2, dtype=torch.float16)
    got = oracle.c_gemm("gemm_rcr", torch.from_numpy(a), ones).numpy().ravel()
    want = (a[:, 0].astype(np.float32) + a[:, 1].astype(np.float32)).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # tiny values -> subnormal halves
    tiny = (rng.standard_normal((512, 2)) * 1e-6).astype(np.float16)
    got = oracle.c_gemm("gemm_rcr", torch.from_numpy(tiny), ones).numpy().ravel()
    want = (tiny[:, 0].astype(np.float32) + tiny[:, 1].astype(np.float32)).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_c_bf16_rounding_matches_torch():
    a = _rand((257, 2), torch.bfloat16, seed=3, scale=50.0)
    ones = torch.ones(1, 2, dtype=torch.bfloat16)
    got = oracle.c_gemm("gemm_rcr", a, ones).ravel()
    want = (a[:, 0].float() + a[:, 1].float()).to(torch.bfloat16)
    assert torch.equal(got, want)


# ---- GEMM: brute force and invariants --------------------------------------
def _brute_gemm(x, w, bias):
    M, K = x.shape
    N = w.shape[0]
    out = [[0.0] * N for _ in range(M)]
    for m in range(M):
        for n in range(N):
            s = 0.0
            for k in range(K):
                s += float(x[m, k]) * float(w[n, k])
            out[m][n] = s + (float(bias[n]) if bias is not None else 0.0)
    return torch.tensor(out, dtype=torch.float64)


@pytest.mark.parametrize("M,N,K", [(3, 5, 7), (16, 16, 16), (1, 9, 4), (8, 1, 3)])
def test_gemm_matches_brute_force(M, N, K):
    x, w, b = _rand((M, K), seed=1), _rand((N, K), seed=2), _rand((N,), seed=3)
    want = _brute_gemm(x, w, b)
    got_t = oracle.torch_gemm("gemm_rcr_bias", x, w, b).double()
    got_c = oracle.c_gemm("gemm_rcr_bias", x, w, b).double()
    assert torch.allclose(got_t, want, atol=1e-4, rtol=1e-5)
    assert torch.allclose(got_c, want, atol=1e-2, rtol=1e-3)  # rounded to fp16
    # a transposed W would fail here: W is not square and not symmetric
    want_nb = _brute_gemm(x, w, None)
    assert torch.allclose(oracle.torch_gemm("gemm_rcr", x, w).double(), want_nb, atol=1e-4, rtol=1e-5)


def test_gemm_identity_weight_and_zero_input():
    x, b = _rand((12, 32), seed=4), _rand((32,), seed=5)
    eye = torch.eye(32, dtype=torch.float16)
    for f in (oracle.torch_gemm, oracle.c_gemm):
        y = f("gemm_rcr_bias", x, eye, b).float()
        assert torch.allclose(y, (x.float() + b.float()), atol=2e-3, rtol=1e-3)
        z = f("gemm_rcr_bias", torch.zeros_like(x), _rand((8, 32), seed=6), b[:8]).float()
        assert torch.allclose(z, b[:8].float().expand(12, 8), atol=0, rtol=0)


def test_gelu_closed_form_and_identities():
    x = torch.linspace(-8, 8, 4001)
    u = math.sqrt(2 / math.pi) * (x + 0.044715 * x ** 3)
    closed = 0.5 * x * (1 + torch.tanh(u))
    lib = torch.nn.functional.gelu(x, approximate="tanh")
    assert torch.allclose(closed, lib, atol=1e-6)
    # sigmoid form with the reference's rounded constants (custom_math.cuh:828-851)
    sig = x / (1 + torch.exp(-2 * x * (0.797885 + 0.035677 * x * x)))
    assert (sig - lib).abs().max() < 2e-5
    # erf GELU (what the reference's ROCm test compares against) is within 5e-4 of it... loosely 1e-3
    assert (torch.nn.functional.gelu(x) - lib).abs().max() < 1e-3


EPILOGUE_CASES = ["gemm_rcr", "gemm_rcr_bias", "gemm_rcr_bias_relu", "gemm_rcr_bias_gelu", "gemm_rcr_bias_add",
                  "gemm_rcr_bias_add_add", "gemm_rcr_bias_add_relu", "gemm_rcr_bias_add_add_relu",
                  "gemm_rcr_bias_sigmoid", "gemm_rcr_bias_tanh", "gemm_rcr_bias_swish", "gemm_rcr_bias_hardswish",
                  "gemm_rcr_bias_mul", "gemm_rcr_bias_mul_add", "gemm_rcr_bias_sigmoid_mul",
                  "gemm_rcr_bias_sigmoid_mul_tanh", "gemm_rcr_bias_mul_tanh"]


@pytest.mark.parametrize("op", EPILOGUE_CASES)
def test_c_and_torch_restatements_agree(op):
    M, N, K = 33, 20, 48
    x, w, b = _rand((M, K), seed=7), _rand((N, K), seed=8, scale=K ** -0.5), _rand((N,), seed=9)
    d0, d1 = _rand((M, N), seed=10), _rand((M, N), seed=11)
    want = oracle.torch_gemm(op, x, w, b, d0, d1)
    got = oracle.c_gemm(op, x, w, b, d0, d1).float()
    assert torch.allclose(got, want, atol=2e-3, rtol=2e-3), (got - want).abs().max()
    # the reference's rounding points move the result by a few fp16 ulps only
    got_ref = oracle.c_gemm(op, x, w, b, d0, d1, ref_rounding=True).float()
    assert torch.allclose(got_ref, want, atol=1e-2, rtol=1e-2)


def test_epilogue_terms_are_all_present():
    # each residual / bias term changes the output: a dropped term fails
    M, N, K = 4, 8, 8
    x, w = _rand((M, K), seed=1), _rand((N, K), seed=2)
    b = torch.full((N,), 2.0, dtype=torch.float16)
    d0 = torch.full((M, N), 16.0, dtype=torch.float16)
    d1 = torch.full((M, N), 128.0, dtype=torch.float16)
    base = oracle.torch_gemm("gemm_rcr", x, w)
    for f in (oracle.torch_gemm, lambda *a: oracle.c_gemm(*a).float()):
        assert torch.allclose(f("gemm_rcr_bias", x, w, b) - base, torch.full((M, N), 2.0), atol=3e-2)
        assert torch.allclose(f("gemm_rcr_bias_add", x, w, b, d0) - base, torch.full((M, N), 18.0), atol=3e-2)
        assert torch.allclose(f("gemm_rcr_bias_add_add", x, w, b, d0, d1) - base, torch.full((M, N), 146.0),
                              atol=2e-1)


# ---- bmm --------------------------------------------------------------------
def test_bmm_rcr_brute_force_and_broadcast():
    q, k = _rand((3, 4, 6), seed=1), _rand((3, 5, 6), seed=2)
    want = torch.einsum("bmk,bnk->bmn", q.double(), k.double())
    assert torch.allclose(oracle.torch_bmm_rcr(q, k).double(), want, atol=1e-5)
    assert torch.allclose(oracle.c_bmm_rcr(q, k).double(), want, atol=1e-2, rtol=1e-2)
    # broadcast of a batch-1 / 2-D operand
    k1 = k[:1]
    want_b = torch.einsum("bmk,nk->bmn", q.double(), k1[0].double())
    assert torch.allclose(oracle.torch_bmm_rcr(q, k1).double(), want_b, atol=1e-5)
    assert torch.allclose(oracle.c_bmm_rcr(q, k1[0]).double(), want_b, atol=1e-2, rtol=1e-2)


# ---- attention --------------------------------------------------------------
def _brute_attention(q, k, v, scale, G, causal=False):
    B, M, K = q.shape
    N, O = v.shape[1], v.shape[2]
    out = torch.zeros(B // G, M, G, O, dtype=torch.float64)
    for b in range(B):
        for m in range(M):
            n_end = min(m + 1, N) if causal else N
            s = [sum(float(q[b, m, kk]) * float(k[b, n, kk]) for kk in range(K)) * scale for n in range(n_end)]
            mx = max(s)
            e = [math.exp(t - mx) for t in s]
            z = sum(e)
            for o in range(O):
                out[b // G, m, b % G, o] = sum(e[n] * float(v[b, n, o]) for n in range(n_end)) / z
    return out


@pytest.mark.parametrize("causal", [False, True])
def test_attention_brute_force(causal):
    B, M, N, K, O, G = 4, 5, 7, 3, 6, 2
    if causal:
        N = M
    q, k, v = _rand((B, M, K), seed=1), _rand((B, N, K), seed=2), _rand((B, N, O), seed=3)
    want = _brute_attention(q, k, v, 0.37, G, causal)
    got_t = oracle.torch_bmm_softmax_bmm_permute(q, k, v, 0.37, G, causal).double()
    got_c = oracle.c_bmm_softmax_bmm_permute(q, k, v, 0.37, G, causal).double()
    assert got_t.shape == (B // G, M, G, O)
    assert torch.allclose(got_t, want, atol=1e-5)
    assert torch.allclose(got_c, want, atol=2e-3, rtol=2e-3)


def test_attention_invariants():
    B, M, N, K, O, G = 8, 16, 24, 40, 40, 4
    q, k, v = _rand((B, M, K), seed=1), _rand((B, N, K), seed=2), _rand((B, N, O), seed=3)
    for f in (oracle.torch_bmm_softmax_bmm_permute, lambda *a: oracle.c_bmm_softmax_bmm_permute(*a).float()):
        # rows of P sum to one: constant V -> constant output
        vc = torch.full_like(v, 0.75)
        assert torch.allclose(f(q, k, vc, 0.2, G), torch.full((B // G, M, G, O), 0.75), atol=1e-3)
        # Q = 0 -> uniform attention -> column mean of V
        out = f(torch.zeros_like(q), k, v, 0.2, G)
        mean = v.float().mean(dim=1)  # [B, O]
        want = mean.reshape(B // G, G, 1, O).permute(0, 2, 1, 3).expand(B // G, M, G, O)
        assert torch.allclose(out, want, atol=2e-3)
        # permutation: V[b] = b (one value per batch) lands at [b // G, :, b % G, :]
        vb = torch.arange(B, dtype=torch.float32).reshape(B, 1, 1).expand(B, N, O).to(torch.float16)
        out = f(q, k, vb, 0.2, G)
        for b in range(B):
            assert torch.allclose(out[b // G, :, b % G, :], torch.full((M, O), float(b)), atol=1e-2)


def test_config_generators_and_work_counts():
    inp = oracle.config_inputs("c1")
    assert inp["x"].shape == (256, 1024) and inp["w"].shape == (1024, 1024) and inp["bias"].shape == (1024,)
    assert float(inp["x"].float().abs().max()) <= 1.0
    # determinism
    again = oracle.config_inputs("c1")
    assert torch.equal(inp["x"], again["x"])
    assert oracle.config_flops_bytes("c1") == (536870912, 3147776)
    assert oracle.config_flops_bytes("c2a") == (115964116992, 193468416)
    assert oracle.config_flops_bytes("c2b") == (115964116992, 231212544)
    assert oracle.config_flops_bytes("c3") == (105763569664, 189138944)
    assert oracle.config_flops_bytes("c4") == (14495514624, 301989888)
    assert oracle.config_flops_bytes("c5") == (42949672960, 20971520)
    small = oracle.config_inputs("c3", m_override=200)
    assert small["x"].shape == (200, 4096) and small["d1"].shape == (200, 1024)


# ---- permuting GEMMs and the attention block ------------------------------------------------
@pytest.mark.parametrize("layout,dims", [("m2n3", (3, 5, 2, 4, 6)), ("m3n2", (3, 4, 5, 2, 6)),
                                         ("m2n3", (1, 7, 3, 1, 8)), ("m3n2", (2, 1, 3, 4, 1))])
def test_permute_5d_matches_the_reference_stride_tables(layout, dims):
    """Element by element against the destination strides the reference hands to its kernels
    (python/aitemplate/backend/rocm/gemm/permute_common.py:84-91 for m2n3, :124-125 for m3n2): an
    independent statement of the same permutation.  Unique values make any wrong index visible."""
    if layout == "m2n3":
        M0, M1, N0, N1, N2 = dims
        M, N, shape = M0 * M1, N0 * N1 * N2, (M1, N0, N1)
    else:
        M0, M1, M2, N0, N1 = dims
        M, N, shape = M0 * M1 * M2, N0 * N1, (M1, M2, N0)
    y = torch.arange(M * N, dtype=torch.float32).reshape(M, N)
    got = oracle.permute_5d(y, layout, shape).reshape(-1)
    want = torch.full((M * N,), -1.0)
    for m in range(M):
        for n in range(N):
            if layout == "m2n3":
                m0, m1 = divmod(m, M1)
                n0, r = divmod(n, N1 * N2)
                n1, n2 = divmod(r, N2)
                dst = m0 * (N1 * M1 * N2) + m1 * N2 + n0 * (M0 * N1 * M1 * N2) + n1 * (M1 * N2) + n2
            else:
                m0, r = divmod(m, M1 * M2)
                m1, m2 = divmod(r, M2)
                n0, n1 = divmod(n, N1)
                dst = m0 * (N0 * M1 * N1) + m1 * N1 + m2 * (M0 * N0 * M1 * N1) + n0 * (M1 * N1) + n1
            want[dst] = y[m, n]
    assert torch.equal(got, want)


def test_gemm_permute_for_packed_qkv_gives_per_head_projections():
    """shape = (seq, 3, heads) on a packed projection must give [3, B, heads, S, d] with
    out[j, b, h] = x[b] @ w[j*D + h*d : j*D + (h+1)*d].T + bias[...]: the layout the attention op reads."""
    B, S, D, H = 2, 5, 12, 3
    d = D // H
    x, w, bias = _rand((B, S, D), seed=1), _rand((3 * D, D), seed=2), _rand((3 * D,), seed=3)
    out = oracle.torch_gemm_permute("gemm_rcr_bias_permute_m2n3", x, w, bias, (S, 3, H))
    assert tuple(out.shape) == (3, B, H, S, d)
    for j in range(3):
        for b in range(B):
            for h in range(H):
                rows = slice(j * D + h * d, j * D + (h + 1) * d)
                want = x[b].float() @ w[rows].float().T + bias[rows].float()
                assert torch.allclose(out[j, b, h], want, atol=1e-5)
    no_bias = oracle.torch_gemm_permute("gemm_rcr_permute_m2n3", x, w, None, (S, 3, H))
    assert torch.allclose(out - no_bias, bias.float().reshape(3, 1, H, 1, d).expand_as(out), atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_block_matches_torch_nn_multiheadattention(causal):
    """The block reduces to the library's nn.MultiheadAttention (packed in_proj, batch_first) plus a residual."""
    B, S, D, H = 2, 7, 16, 4
    mha = torch.nn.MultiheadAttention(D, H, bias=True, batch_first=True).eval()
    x, res = _rand((B, S, D), torch.float32, seed=4), _rand((B * S, D), torch.float32, seed=5)
    mask = torch.triu(torch.ones(S, S, dtype=torch.bool), diagonal=1) if causal else None
    with torch.no_grad():
        want, _ = mha(x, x, x, attn_mask=mask, need_weights=False)
        got = oracle.torch_multihead_attention(x, mha.in_proj_weight, mha.in_proj_bias, mha.out_proj.weight,
                                               mha.out_proj.bias, res, H, causal)
    assert torch.allclose(got, want + res.reshape(B, S, D), atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_cross_attention_block_matches_torch_nn_multiheadattention(causal):
    """Separate q / k / v projections are the three row blocks of the library module's packed in_proj."""
    B, S, Skv, D, H = 2, 7, 7 if causal else 5, 16, 4
    mha = torch.nn.MultiheadAttention(D, H, bias=True, batch_first=True).eval()
    q, k, v = (_rand((B, n, D), torch.float32, seed=6 + i) for i, n in enumerate((S, Skv, Skv)))
    res = _rand((B * S, D), torch.float32, seed=9)
    wq, wk, wv = mha.in_proj_weight.chunk(3)
    bq, bk, bv = mha.in_proj_bias.chunk(3)
    mask = torch.triu(torch.ones(S, Skv, dtype=torch.bool), diagonal=1) if causal else None
    with torch.no_grad():
        want, _ = mha(q, k, v, attn_mask=mask, need_weights=False)
        got = oracle.torch_cross_attention(q, k, v, wq, wk, wv, bq, bk, bv, mha.out_proj.weight, mha.out_proj.bias,
                                           res, H, causal)
    assert torch.allclose(got, want + res.reshape(B, S, D), atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_mem_eff_attention_key_lengths(causal):
    """Three pins: without lengths it is the pinned bmm_softmax_bmm_permute on [batch * heads] operands; with
    lengths every batch entry equals the fixed-length result on its truncated keys (rows past the length may hold
    anything, NaN included); and it agrees with the library's scaled_dot_product_attention under a padding mask."""
    batch, heads, S, Skv, d, dv = 3, 2, 9, 11, 8, 6
    q, k, v = (_rand(sh, torch.float32, seed=20 + i)
               for i, sh in enumerate(((batch, heads, S, d), (batch, heads, Skv, d), (batch, heads, Skv, dv))))
    flat = oracle.torch_bmm_softmax_bmm_permute(q.reshape(-1, S, d), k.reshape(-1, Skv, d), v.reshape(-1, Skv, dv),
                                                d ** -0.5, heads, causal)
    assert torch.allclose(oracle.torch_mem_eff_attention(q, k, v, causal), flat, atol=1e-6)
    lens = torch.tensor([[11], [4], [1]], dtype=torch.int32)
    k2, v2 = k.clone(), v.clone()
    for b in range(batch):
        k2[b, :, int(lens[b]):] = float("nan")
        v2[b, :, int(lens[b]):] = float("nan")
    got = oracle.torch_mem_eff_attention(q, torch.nan_to_num(k2, nan=7.0), v2, causal, lens)
    for b in range(batch):
        n = int(lens[b])
        want = oracle.torch_mem_eff_attention(q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n], causal)
        assert torch.allclose(got[b:b + 1], want, atol=1e-6)
    keep = torch.arange(Skv)[None, :] < lens.long()                       # [batch, Skv]
    mask = keep[:, None, None, :].expand(batch, 1, S, Skv)
    if causal:
        mask = mask & torch.tril(torch.ones(S, Skv, dtype=torch.bool))
    sdpa = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask).permute(0, 2, 1, 3)
    assert torch.allclose(oracle.torch_mem_eff_attention(q, k, v, causal, lens), sdpa, atol=1e-5)
    # query lengths only blank rows: everything before them is untouched
    lq = torch.tensor([9, 3, 0], dtype=torch.int32)
    with_q = oracle.torch_mem_eff_attention(q, k, v, causal, lens, lq)
    base = oracle.torch_mem_eff_attention(q, k, v, causal, lens)
    for b in range(batch):
        assert torch.equal(with_q[b, :int(lq[b])], base[b, :int(lq[b])])
        assert torch.count_nonzero(with_q[b, int(lq[b]):]) == 0
    # no keys at all: zeros by this library's convention
    zero = oracle.torch_mem_eff_attention(q, k, v, causal, torch.zeros(batch, 1, dtype=torch.int32))
    assert torch.count_nonzero(zero) == 0


def test_bmm_rcr_permute_places_each_batch_as_a_head():
    """out[g, m, h, n] must be (Q[g*d1 + h] @ K[g*d1 + h]^T)[m, n]: brute force over the batch index."""
    B, M, N, K, d1 = 6, 5, 7, 4, 3
    q, k = _rand((B, M, K), seed=1), _rand((B, N, K), seed=2)
    out = oracle.torch_bmm_rcr_permute(q, k, d1)
    assert tuple(out.shape) == (B // d1, M, d1, N)
    for b in range(B):
        want = q[b].float() @ k[b].float().T
        assert torch.allclose(out[b // d1, :, b % d1, :], want, atol=1e-5)


@pytest.mark.parametrize("layout", ["rcr", "rrr", "ccr", "crr"])
def test_bmm_layouts_brute_force(layout):
    """C[b, m, n] = sum_k A(b, m, k) B(b, k, n) with the operands indexed as each layout stores them."""
    B, M, N, K = 2, 3, 4, 5
    a = _rand((B, K, M) if layout[0] == "c" else (B, M, K), seed=1)
    b = _rand((B, N, K) if layout[1] == "c" else (B, K, N), seed=2)
    got = oracle.torch_bmm(layout, a, b)
    for bi in range(B):
        for m in range(M):
            for n in range(N):
                acc = 0.0
                for k in range(K):
                    av = a[bi, k, m] if layout[0] == "c" else a[bi, m, k]
                    bv = b[bi, n, k] if layout[1] == "c" else b[bi, k, n]
                    acc += float(av) * float(bv)
                assert abs(got[bi, m, n].item() - acc) < 1e-4
    if layout == "rcr":
        assert torch.equal(got, oracle.torch_bmm_rcr(a, b))


def test_attention_nan_scores_count_as_minus_infinity():
    """A NaN score leaves its key out of the row's softmax (the reference's ScaleAndResetNaNToMinusInfinity functor,
    python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:106): against a loop that says `isnan -> -inf`
    explicitly, and against plain attention over the keys that are left."""
    B, M, N, K, O, G = 4, 5, 9, 3, 6, 2
    q, k, v = _rand((B, M, K), seed=1), _rand((B, N, K), seed=2), _rand((B, N, O), seed=3)
    k[1, 4, 2] = float("nan")      # one key of batch entry 1 is bad for every query
    q[2, 3, 0] = float("nan")      # one query row of batch entry 2 is bad for every key
    scale = 0.37
    want = torch.zeros(B // G, M, G, O, dtype=torch.float64)
    for b in range(B):
        for m in range(M):
            s = []
            for n in range(N):
                t = sum(float(q[b, m, kk]) * float(k[b, n, kk]) for kk in range(K)) * scale
                s.append(-math.inf if math.isnan(t) else t)
            mx = max(s)
            if mx == -math.inf:
                want[b // G, m, b % G, :] = float("nan")  # every score reset: 0 / 0, pinned by nothing
                continue
            e = [math.exp(t - mx) for t in s]
            for o in range(O):
                want[b // G, m, b % G, o] = sum(e[n] * float(v[b, n, o]) for n in range(N)) / sum(e)
    got_t = oracle.torch_bmm_softmax_bmm_permute(q, k, v, scale, G).double()
    got_c = oracle.c_bmm_softmax_bmm_permute(q, k, v, scale, G).double()
    live = ~torch.isnan(want)
    assert not live[1, 3, 0].any() and live.sum() == want.numel() - O  # only the all-NaN query row is left open
    assert torch.allclose(got_t[live], want[live], atol=1e-5)
    assert torch.allclose(got_c[live], want[live], atol=2e-3, rtol=2e-3)
    # the same as attention without the bad key
    keep = [n for n in range(N) if n != 4]
    ref = oracle.torch_bmm_softmax_bmm_permute(q[1:2], k[1:2, keep], v[1:2, keep], scale, 1).double()
    assert torch.allclose(got_t[0, :, 1, :], ref[0, :, 0, :], atol=1e-6)
    # a NaN in V is not a score: it reaches the output of every query of its batch entry
    v2 = v.clone()
    v2[0, 2, 1] = float("nan")
    out = oracle.torch_bmm_softmax_bmm_permute(q, k, v2, scale, G)
    assert torch.isnan(out[0, :, 0, 1]).all() and not torch.isnan(out[0, :, 0, 0]).any()


def test_elementwise_nan_conventions_and_function_table():
    """torch_elementwise against the reference's device functions written out by hand: MAX / MIN return NaN when
    either operand is NaN (fmaxf_nan / fminf_nan, backend/rocm/elementwise/custom_math.h:282-310), RELU is
    `a > 0 ? a : 0`, which sends NaN to 0 (custom_math.h:117), LRELU is `a > 0 ? a : a * slope`."""
    nan, inf = float("nan"), float("inf")
    a = torch.tensor([1.0, nan, -2.0, nan, 0.5, -inf, 3.0])
    b = torch.tensor([nan, 2.0, -3.0, nan, 0.5, 1.0, -inf])

    def by_hand(f):
        return [f(float(x), float(y)) for x, y in zip(a, b)]

    def same(got, want):
        want = torch.tensor(want, dtype=torch.float32)
        return bool((torch.isnan(got) == torch.isnan(want)).all()) and \
            bool(torch.equal(torch.nan_to_num(got, nan=0.0), torch.nan_to_num(want, nan=0.0)))

    assert same(oracle.torch_elementwise("MAX", a, b),
                by_hand(lambda x, y: nan if (math.isnan(x) or math.isnan(y)) else max(x, y)))
    assert same(oracle.torch_elementwise("MIN", a, b),
                by_hand(lambda x, y: nan if (math.isnan(x) or math.isnan(y)) else min(x, y)))
    assert same(oracle.torch_elementwise("RELU", a), [x if x > 0 else 0.0 for x in a.tolist()])
    assert oracle.torch_elementwise("RELU", torch.tensor([nan])).item() == 0.0
    assert same(oracle.torch_elementwise("LRELU", a, 0.1),
                [float(torch.tensor(x if x > 0 else x * 0.1, dtype=torch.float32)) for x in a.tolist()])
    # the rest of the table against the math library on a few points, constants as the second operand included
    x = torch.tensor([0.25, 1.5, 2.0])
    y = torch.tensor([2.0, 0.5, 3.0])
    for name, f in (("ADD", lambda p, q: p + q), ("SUB", lambda p, q: p - q), ("MUL", lambda p, q: p * q),
                    ("DIV", lambda p, q: p / q), ("POW", lambda p, q: p ** q)):
        want = torch.tensor([f(float(p), float(q)) for p, q in zip(x, y)])
        assert torch.allclose(oracle.torch_elementwise(name, x, y), want, rtol=1e-6), name
        assert torch.allclose(oracle.torch_elementwise(name, x, 2.0),
                              torch.tensor([f(float(p), 2.0) for p in x]), rtol=1e-6), name
    for name, f in (("TANH", math.tanh), ("ABS", abs), ("EXP", math.exp), ("SQRT", math.sqrt),
                    ("SIGMOID", lambda t: 1 / (1 + math.exp(-t))), ("SILU", lambda t: t / (1 + math.exp(-t))),
                    ("GELU", lambda t: 0.5 * t * (1 + math.erf(t / math.sqrt(2)))),
                    ("FASTGELU", lambda t: 0.5 * t * (1 + math.tanh(0.7978845608 * (t + 0.044715 * t ** 3)))),
                    ("COS", math.cos), ("SIN", math.sin), ("SIGN", lambda t: (t > 0) - (t < 0)), ("LOGE", math.log),
                    ("LOG1P", math.log1p), ("SOFTSIGN", lambda t: t / (1 + abs(t))), ("FLOOR", math.floor),
                    ("RECIPROCAL", lambda t: 1 / t)):
        pts = torch.tensor([-1.25, 0.25, 1.5]) if name not in ("SQRT", "LOGE", "LOG1P") else x
        want = torch.tensor([float(f(float(t))) for t in pts])
        assert torch.allclose(oracle.torch_elementwise(name, pts), want, rtol=2e-6, atol=1e-7), name
