"""GPU parity of bmm_softmax_bmm_permute through the C ABI against the CPU oracle.
Tolerance atol = rtol = 2e-2 (softmax path, fp16 out / fp32 accumulate)."""
import pytest
import torch

from aitemplate_amd import eager
from oracle import oracle

pytestmark = pytest.mark.gpu

TOL = 2e-2


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def _check(B, M, N, K, O, G, causal=False, dtype=torch.float16, scale=None, seed=0, tol=TOL):
    print(f"case attention B={B} M={M} N={N} K={K} O={O} G={G} causal={causal} {dtype}", flush=True)
    q, k, v = _rand((B, M, K), dtype, seed), _rand((B, N, K), dtype, seed + 1), _rand((B, N, O), dtype, seed + 2)
    scale = K ** -0.5 if scale is None else scale
    want = oracle.torch_bmm_softmax_bmm_permute(q, k, v, scale, G, causal).to(dtype).float()
    got = eager.bmm_softmax_bmm_permute(q.cuda(), k.cuda(), v.cuda(), (G,), scale=scale, causal=causal)
    torch.cuda.synchronize()
    assert got.shape == (B // G, M, G, O)
    torch.testing.assert_close(got.cpu().float(), want, atol=tol, rtol=tol)


# the shapes of the reference's ROCm test (tests/unittest/ops/test_bmm_softmax_bmm.py:174-205)
@pytest.mark.parametrize("B,M,N,K,O,G,causal", [
    (24, 256, 256, 64, 64, 12, False),
    (24, 196, 196, 64, 64, 12, False),
    (24, 128, 1024, 64, 128, 12, False),
    (24, 128, 49, 64, 128, 12, False),
    (24, 49, 49, 64, 64, 12, False),
    (24, 1020, 1020, 64, 128, 12, False),
    (32, 49, 49, 64, 64, 4, False),
    (16, 4096, 64, 40, 40, 8, False),
    (12, 64, 64, 64, 64, 12, True),
])
def test_reference_shapes(B, M, N, K, O, G, causal):
    _check(B, M, N, K, O, G, causal)


@pytest.mark.parametrize("B,M,N,K,O,G,causal", [
    (4, 130, 70, 40, 40, 2, False),     # ragged M and N, head_dim 40
    (2, 33, 200, 16, 24, 1, False),     # small head dims
    (2, 65, 65, 128, 128, 2, True),     # largest head dims, causal with ragged edge
    (4, 300, 300, 96, 80, 4, True),
    (2, 17, 9, 20, 12, 2, False),       # K, O not multiples of 8 -> element-wise loads
    (3, 5, 1, 8, 8, 3, False),          # a single key: softmax == 1
])
def test_ragged_and_odd_shapes(B, M, N, K, O, G, causal):
    _check(B, M, N, K, O, G, causal, seed=3)


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("B,M,N,K,O,G,causal,scale", [
    (8, 300, 1000, 40, 40, 4, False, None),    # 8 key tiles: both wave groups busy
    (8, 300, 900, 40, 40, 4, True, None),      # causal: workgroups stop at different tiles
    (4, 100, 130, 40, 40, 2, False, -0.2),     # 2 tiles, the second ragged; negative scale
    (4, 70, 384, 32, 32, 4, False, None),      # 3 tiles: the second group is short of one
    (2, 40, 50, 40, 40, 2, True, None),        # a single tile: the second group has nothing to merge
    (2, 260, 0, 40, 40, 2, False, None),       # no keys at all
])
def test_every_variant_of_the_small_head_dims(attn_variant, mode, B, M, N, K, O, G, causal, scale):
    # aitamd_attention_set_variant picks the variant where the shape allows it: 0 four waves, 1 eight waves, 2 (3) two groups of
    # eight (four) waves that take alternate key tiles and merge their running sums at the end
    attn_variant(mode)
    print(f"case attention mode={mode} B={B} M={M} N={N} K={K} causal={causal} scale={scale}", flush=True)
    _check(B, M, N, K, O, G, causal=causal, scale=scale, seed=mode + N)


@pytest.mark.parametrize("B,M,N,K,O,G,causal", [
    (16, 256, 256, 160, 160, 8, False),     # the deepest attention of Stable Diffusion v1: 1280 channels, 8 heads
    (8, 100, 77, 160, 160, 8, False),       # its cross-attention over 77 text tokens
    (4, 130, 200, 136, 160, 2, True),
    (4, 64, 300, 160, 40, 4, False),
])
def test_head_dim_160(B, M, N, K, O, G, causal):
    _check(B, M, N, K, O, G, causal, seed=11)


def test_bf16():
    _check(8, 200, 136, 64, 64, 4, dtype=torch.bfloat16, tol=4e-2)
    _check(8, 100, 100, 40, 40, 8, causal=True, dtype=torch.bfloat16, tol=4e-2)


@pytest.mark.parametrize("scale", [-0.3, 0.0])
@pytest.mark.parametrize("causal", [False, True])
def test_negative_and_zero_scale(scale, causal):
    # the running maximum is kept on raw scores: a negative scale is moved into the Q fragments
    _check(8, 200, 200, 40, 40, 4, causal=causal, scale=scale, seed=9)


def test_large_scores_do_not_overflow():
    # scores of magnitude ~60: exp() of the raw score would overflow fp16/fp32 ranges without the running max
    _check(4, 64, 256, 64, 64, 4, scale=1.0, seed=5, tol=3e-2)


def test_invariants_on_gpu():
    B, M, N, K, O, G = 8, 100, 150, 40, 40, 4
    q, k = _rand((B, M, K), torch.float16, 1).cuda(), _rand((B, N, K), torch.float16, 2).cuda()
    vc = torch.full((B, N, O), 0.75, dtype=torch.float16, device="cuda")
    out = eager.bmm_softmax_bmm_permute(q, k, vc, (G,), scale=0.2)
    assert torch.allclose(out.float().cpu(), torch.full((B // G, M, G, O), 0.75), atol=2e-3)
    vb = torch.arange(B, dtype=torch.float32).reshape(B, 1, 1).expand(B, N, O).to(torch.float16).cuda().contiguous()
    out = eager.bmm_softmax_bmm_permute(q, k, vb, (G,), scale=0.2).cpu().float()
    for b in range(B):
        assert torch.allclose(out[b // G, :, b % G, :], torch.full((M, O), float(b)), atol=1e-2)


def test_empty_keys_give_zero_and_empty_batch_is_noop():
    q = torch.randn(2, 8, 16, dtype=torch.float16, device="cuda")
    k = torch.empty(2, 0, 16, dtype=torch.float16, device="cuda")
    v = torch.empty(2, 0, 8, dtype=torch.float16, device="cuda")
    out = torch.full((1, 8, 2, 8), 7.0, dtype=torch.float16, device="cuda")
    eager.bmm_softmax_bmm_permute(q, k, v, (2,), out=out)
    torch.cuda.synchronize()
    assert float(out.abs().max()) == 0.0
    with pytest.raises(RuntimeError):
        eager.bmm_softmax_bmm_permute(q, k, v, (3,))  # batch 2 is not a multiple of 3 heads


def _check_mem_eff(batch, heads, S, Skv, d, dv, lens, causal=False, dtype=torch.float16, seed=0, lens_q=None):
    print(f"case mem_eff_attention batch={batch} heads={heads} S={S} Skv={Skv} d={d} dv={dv} lens={lens} "
          f"causal={causal} {dtype}", flush=True)
    q, k, v = (_rand(sh, dtype, seed + i)
               for i, sh in enumerate(((batch, heads, S, d), (batch, heads, Skv, d), (batch, heads, Skv, dv))))
    lengths = None if lens is None else torch.tensor(lens, dtype=torch.int32).reshape(batch, 1)
    lengths_q = None if lens_q is None else torch.tensor(lens_q, dtype=torch.int32)
    want = oracle.torch_mem_eff_attention(q, k, v, causal, lengths, lengths_q).to(dtype).float()
    if lengths is not None:
        # rows past a batch entry's length must not be read: poison them
        for b in range(batch):
            k[b, :, max(0, min(Skv, int(lens[b]))):] = float("nan")
            v[b, :, max(0, min(Skv, int(lens[b]))):] = float("nan")
    got = eager.mem_eff_attention(q.cuda(), k.cuda(), v.cuda(), causal=causal,
                                  lengths_kv=None if lengths is None else lengths.cuda(),
                                  lengths_q=None if lengths_q is None else lengths_q.cuda(),
                                  out=torch.full((batch, S, heads, dv), 3.0, dtype=dtype, device="cuda"))
    torch.cuda.synchronize()
    assert got.shape == (batch, S, heads, dv)
    torch.testing.assert_close(got.cpu().float(), want, atol=TOL, rtol=TOL)


@pytest.mark.parametrize("mode", [None, 0, 1, 2, 3])
@pytest.mark.parametrize("batch,heads,S,Skv,d,dv,lens,causal", [
    (4, 2, 300, 1000, 40, 40, [1000, 517, 128, 1], False),   # whole tiles, a ragged last tile, one key
    (4, 2, 300, 900, 40, 40, [900, 300, 77, 0], True),       # causal bound and key length, whichever is shorter
    (3, 4, 70, 384, 32, 32, [384, 129, 0], False),           # a batch entry without keys is zeros
    (2, 2, 40, 50, 40, 40, [50, 49], False),                 # single tile
    (2, 3, 64, 200, 64, 128, [1200, -3], False),             # lengths are clamped to [0, Skv]
])
def test_mem_eff_attention_key_lengths(attn_variant, mode, batch, heads, S, Skv, d, dv, lens, causal):
    """Key lengths through the C ABI for every kernel variant (as in test_attention.py:504-523 of the reference)."""
    if mode is not None:
        attn_variant(mode)
    _check_mem_eff(batch, heads, S, Skv, d, dv, lens, causal=causal, seed=Skv)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch,heads,S,Skv,d,dv,lens", [
    (2, 8, 1024, 77, 40, 40, None),                          # fixed length: the cross-attention of a diffusion UNet
    (2, 4, 197, 197, 64, 64, [197, 50]),
    (3, 2, 50, 333, 20, 24, [333, 100, 7]),                  # head dims that are no multiple of 8: element-wise loads
    (2, 2, 128, 256, 160, 160, [256, 65]),
])
def test_mem_eff_attention_shapes_and_dtypes(dtype, batch, heads, S, Skv, d, dv, lens):
    _check_mem_eff(batch, heads, S, Skv, d, dv, lens, dtype=dtype, seed=d)


@pytest.mark.parametrize("mode", [None, 0, 1, 2, 3])
@pytest.mark.parametrize("causal", [False, True])
def test_mem_eff_attention_query_lengths(attn_variant, mode, causal):
    """Rows past a query length are zeros (whole blocks of them visit no keys), the rows before are unchanged."""
    if mode is not None:
        attn_variant(mode)
    _check_mem_eff(5, 2, 700, 640, 40, 40, [640, 300, 640, 1, 640], causal=causal, seed=mode or 9,
                   lens_q=[700, 130, 0, 257, 9000])


def test_mem_eff_attention_argument_checks():
    q = torch.randn(2, 2, 8, 16, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        eager.mem_eff_attention(q, q, q, lengths_kv=torch.zeros(2, dtype=torch.int64, device="cuda"))
    with pytest.raises(ValueError):
        eager.mem_eff_attention(q, q, q, lengths_kv=torch.zeros(3, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError):
        eager.mem_eff_attention(q, q[:, :1], q)


def test_config_c5_full_size():
    print("case config=c5 full size", flush=True)
    inp = oracle.config_inputs("c5")
    want = oracle.config_expected("c5", inp).half().float()
    got = eager.bmm_softmax_bmm_permute(inp["q"].cuda(), inp["k"].cuda(), inp["v"].cuda(), (oracle.C5_HEADS,),
                                        scale=oracle.C5_SCALE)
    torch.cuda.synchronize()
    assert got.shape == (2, 4096, 8, 40)
    torch.testing.assert_close(got.cpu().float(), want, atol=TOL, rtol=TOL)


def test_nan_in_a_key_leaves_that_key_out():
    """A NaN score counts as -inf, as in the reference, whose kernel takes ScaleAndResetNaNToMinusInfinity between the
    first product and the softmax (python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:106): every query of
    the batch entry that holds the bad key row comes out finite and equal to attention without that key; a NaN in a
    query row resets all of that row's scores, which the reference leaves as 0 / 0 and nothing pins (finite or NaN
    is accepted there); a NaN in V reaches the output as a NaN."""
    B, M, N, K, O, G = 4, 96, 200, 64, 64, 2
    print(f"case attention NaN key B={B} M={M} N={N} K={K}", flush=True)
    q, k, v = _rand((B, M, K), torch.float16, 11), _rand((B, N, K), torch.float16, 12), _rand((B, N, O), torch.float16, 13)
    k[1, 77, 5] = float("nan")
    k[1, 199, 0] = float("nan")   # in the masked tail tile as well
    q[2, 40, 3] = float("nan")
    v[3, 10, 7] = float("nan")
    want = oracle.torch_bmm_softmax_bmm_permute(q, k, v, K ** -0.5, G, False).half().float()   # [B/G, M, G, O]
    got = eager.bmm_softmax_bmm_permute(q.cuda(), k.cuda(), v.cuda(), (G,), scale=K ** -0.5).cpu().float()
    assert not torch.isnan(want[0, :, 1, :]).any(), "the oracle resets NaN scores"
    assert not torch.isnan(got[0, :, 1, :]).any()
    keep = [n for n in range(N) if n not in (77, 199)]
    without = oracle.torch_bmm_softmax_bmm_permute(q[1:2], k[1:2, keep], v[1:2, keep], K ** -0.5, 1, False)
    torch.testing.assert_close(got[0, :, 1, :], without[0, :, 0, :].half().float(), atol=TOL, rtol=TOL)
    open_rows = torch.zeros(B // G, M, G, dtype=torch.bool)
    open_rows[1, 40, 0] = True   # the query row whose scores are all NaN
    assert torch.isnan(got[1, :, 1, 7]).all() and torch.isnan(want[1, :, 1, 7]).all()
    sel = ~open_rows[..., None].expand_as(got)
    torch.testing.assert_close(got[sel], want[sel], atol=TOL, rtol=TOL, equal_nan=True)


# ---- head dims that leave padding columns in the LDS tiles (K = 16 KS - 8: 24, 40, 56, 88, 120, 152; O = 32 OT - 24)
@pytest.mark.parametrize("B,M,N,K,O,G,causal,scale", [
    (8, 300, 700, 40, 40, 4, False, None),
    (8, 300, 300, 40, 40, 4, True, None),
    (4, 130, 1000, 40, 64, 2, False, -0.2),     # negative scale: changes sides into Q
    (6, 64, 77, 24, 24, 3, False, None),
    (6, 200, 200, 24, 32, 3, True, None),
    (4, 100, 520, 56, 56, 2, False, None),
    (4, 257, 257, 88, 88, 2, True, None),
    (2, 96, 300, 120, 120, 2, False, None),
    (2, 64, 200, 152, 152, 1, False, None),
    # K = 16 KS - 8 with O = 32 OT - 24
    (6, 100, 333, 24, 8, 3, False, None),
    (4, 200, 520, 56, 40, 2, True, None),
    (4, 130, 300, 88, 72, 2, False, None),
    (2, 96, 260, 120, 104, 2, True, None),
    (2, 64, 200, 152, 136, 1, False, None),
    (70000, 8, 40, 40, 40, 7, False, None),    # more batch entries than the grid's y range: a workgroup takes two
])
def test_head_dims_with_padding_columns(B, M, N, K, O, G, causal, scale):
    _check(B, M, N, K, O, G, causal, scale=scale, seed=K + M)


def test_large_small_and_all_negative_logits():
    """Logits of about 100 (a sharply peaked softmax), rows whose scores are all far below zero (the running maximum
    must not start at 0: the sum would underflow) and tiny logits; fp16 and bf16."""
    B, M, N, K, G = 8, 256, 600, 40, 4
    for mult, shift, tol in ((4.0, 0.0, 2e-2), (1.0, -30.0, 2e-2), (0.01, 0.0, 2e-3)):
        print(f"case attention logits x{mult} shift {shift}", flush=True)
        q, k, v = _rand((B, M, K), torch.float16, 31) * mult, _rand((B, N, K), torch.float16, 32) * mult, \
            _rand((B, N, K), torch.float16, 33)
        if shift:
            # every score of a row about `shift`: q gets a constant component that k answers with a negative one
            q[..., 0] = 8.0
            k[..., 0] = shift / 8.0 * K ** 0.5
        want = oracle.torch_bmm_softmax_bmm_permute(q, k, v, K ** -0.5, G, False).half().float()
        got = eager.bmm_softmax_bmm_permute(q.cuda(), k.cuda(), v.cuda(), (G,), scale=K ** -0.5).cpu().float()
        assert torch.isfinite(got).all()
        torch.testing.assert_close(got, want, atol=tol, rtol=tol)
    # (3e-2 is the bf16 tolerance of the other tests)
    q, k, v = _rand((B, M, K), torch.bfloat16, 34) * 4, _rand((B, N, K), torch.bfloat16, 35) * 4, \
        _rand((B, N, K), torch.bfloat16, 36)
    want = oracle.torch_bmm_softmax_bmm_permute(q, k, v, K ** -0.5, G, False).bfloat16().float()
    got = eager.bmm_softmax_bmm_permute(q.cuda(), k.cuda(), v.cuda(), (G,), scale=K ** -0.5).cpu().float()
    torch.testing.assert_close(got, want, atol=3e-2, rtol=3e-2)


def test_nan_key_and_lengths_at_head_dim_40(attn_variant):
    """The NaN reset and the length masks at head dim 40 (padded to 48 / 64 inside LDS), every variant."""
    B, M, N, K, O, G = 4, 96, 700, 40, 40, 2
    q, k, v = _rand((B, M, K), torch.float16, 41), _rand((B, N, K), torch.float16, 42), _rand((B, N, O), torch.float16, 43)
    k[1, 77, 5] = float("nan")
    k[1, 650, 1] = float("nan")
    want = oracle.torch_bmm_softmax_bmm_permute(q, k, v, K ** -0.5, G, False).half().float()
    assert not torch.isnan(want).any()
    for mode in (-1, 0, 1, 2, 3):
        attn_variant(mode)
        print(f"case attention NaN reset head dim 40 variant {mode}", flush=True)
        got = eager.bmm_softmax_bmm_permute(q.cuda(), k.cuda(), v.cuda(), (G,), scale=K ** -0.5).cpu().float()
        torch.testing.assert_close(got, want, atol=TOL, rtol=TOL)
        _check_mem_eff(3, 4, 150, 333, 40, 40, [333, 1, 200], causal=False)
        _check_mem_eff(3, 4, 150, 150, 40, 40, [150, 0, 77], causal=True, lens_q=[150, 10, 0])
