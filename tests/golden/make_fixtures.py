"""Writes tests/golden/gemm_family.npz: small seeded inputs and expected outputs for every op of the path.

The reference holds no stored vectors for this path (its unit tests compare against PyTorch on a GPU),
and its arithmetic lives in a library that is not part of its tree, so these vectors are NOT produced by
the reference.  Expected values come from plain float64 numpy written here independently of oracle/
(matrix products, the tanh-GELU closed form, an explicit softmax) - they pin both the oracle (CPU test)
and the HIP path (GPU test) to the mathematics.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def h(a):
    return a.astype(np.float16)


def gelu_tanh(x):
    return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    # GEMM family: ragged M/N, K multiple of 8
    M, N, K = 77, 52, 72
    x, w = h(rng.standard_normal((M, K))), h(rng.standard_normal((N, K)) * K ** -0.5)
    b, d0, d1 = h(rng.uniform(-1, 1, N)), h(rng.standard_normal((M, N))), h(rng.standard_normal((M, N)))
    x64, w64, b64, d064, d164 = (t.astype(np.float64) for t in (x, w, b, d0, d1))
    acc = x64 @ w64.T
    out.update(gemm_x=x, gemm_w=w, gemm_bias=b, gemm_d0=d0, gemm_d1=d1)
    out["gemm_rcr"] = acc
    out["gemm_rcr_bias"] = acc + b64
    out["gemm_rcr_bias_relu"] = np.maximum(acc + b64, 0.0)
    out["gemm_rcr_bias_gelu"] = gelu_tanh(acc + b64)
    out["gemm_rcr_bias_add"] = acc + b64 + d064
    out["gemm_rcr_bias_add_add"] = acc + b64 + d064 + d164
    # bmm_rcr
    B, M, N, K = 5, 33, 47, 24
    q, k = h(rng.standard_normal((B, M, K)) / 4), h(rng.standard_normal((B, N, K)) / 4)
    out.update(bmm_q=q, bmm_k=k)
    out["bmm_rcr"] = np.einsum("bmk,bnk->bmn", q.astype(np.float64), k.astype(np.float64))
    # bmm_softmax_bmm_permute: 2 x 3 heads, ragged key count, head dim 40
    G, B, M, N, D = 3, 6, 70, 49, 40
    q, k, v = (h(rng.standard_normal(s)) for s in ((B, M, D), (B, N, D), (B, N, D)))
    scale = D ** -0.5  # exact; the op's rounding of the scale to the element type is below the test tolerance
    s = np.einsum("bmk,bnk->bmn", q.astype(np.float64), k.astype(np.float64)) * scale
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    o = np.einsum("bmn,bno->bmo", p, v.astype(np.float64))
    out.update(attn_q=q, attn_k=k, attn_v=v, attn_heads=np.int64(G), attn_scale=np.float64(D ** -0.5))
    out["bmm_softmax_bmm_permute"] = o.reshape(B // G, G, M, D).transpose(0, 2, 1, 3)
    for key, val in list(out.items()):
        if isinstance(val, np.ndarray) and val.dtype == np.float64 and val.ndim > 0:
            out[key] = val.astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "gemm_family.npz"), **out)
    print("wrote", os.path.join(HERE, "gemm_family.npz"))


if __name__ == "__main__":
    main()
