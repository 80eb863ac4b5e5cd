"""TEST INFRASTRUCTURE ONLY — CPU oracle of the AITemplate ROCm GEMM family.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; nothing under ``aitemplate_amd/`` does.

Two independent restatements are kept side by side:

* ``torch_*`` — the fp32 PyTorch expressions the reference's own unit tests use
  as their oracle, evaluated on the CPU:
  ``F.linear`` (tests/unittest/ops/test_gemm_bias.py:69, test_gemm.py),
  ``relu`` (test_gemm_bias_relu.py:64-65), GELU (test_gemm_rcr_bias_fast_gelu.py:96;
  the kernel implements the tanh form, see backend/cuda/elementwise/custom_math.cuh:828-851),
  ``linear + D0 (+ D1)`` (test_gemm_bias_broadcast.py:213-216,372-376),
  ``bmm(Q, K^T)`` (test_bmm.py:50-51),
  ``softmax(Q K^T * scale) V`` with the 0213 permute (test_bmm_softmax_bmm.py:90,111-114), and the
  5-D output permutations of the permuting GEMMs (test_gemm_bias_permute.py:73-75,138-140), and
  attention on [batch, heads, seq, head_dim] operands with an optional key-padding mask from per-batch key
  lengths (test_attention.py:504-523,593).
* ``c_*`` — the plain-C triple loops of ``oracle/gemm_oracle.c`` (fp32 accumulate,
  optional reference rounding points), loaded through ctypes.

Parity status: the reference ships no golden vectors for this path (its tests
compare against PyTorch on a GPU), so every function here is pinned by closed
forms, invariants and brute force in ``tests/test_oracle.py`` rather than by
fixtures of the reference.  One convention is pinned by nothing in the reference
("parity unpinned"): ``torch_mem_eff_attention`` returns zeros for a batch entry
whose key length is 0, where PyTorch's softmax gives NaN, and zeros for query
rows past a query length, which the reference leaves unspecified.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Dict, Optional, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_C_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_c_lib: Optional[ctypes.CDLL] = None

EPILOGUE_ID = {
    "gemm_rcr": 0, "bmm_rcr": 0, "gemm_rcr_bias": 1, "gemm_rcr_bias_relu": 2, "gemm_rcr_bias_gelu": 3,
    "gemm_rcr_bias_fast_gelu": 3, "gemm_rcr_bias_add": 4, "gemm_rcr_bias_add_add": 5,
    "gemm_rcr_bias_add_relu": 6, "gemm_rcr_bias_add_add_relu": 7, "gemm_rcr_bias_sigmoid": 8,
    "gemm_rcr_bias_tanh": 9, "gemm_rcr_bias_swish": 10, "gemm_rcr_bias_hardswish": 11,
    "gemm_rcr_bias_mul": 12, "gemm_rcr_bias_mul_add": 13, "gemm_rcr_bias_sigmoid_mul": 14,
    "gemm_rcr_bias_sigmoid_mul_tanh": 15, "gemm_rcr_bias_mul_tanh": 16,
}


def build_c_oracle() -> str:
    """Compile oracle/gemm_oracle.c with gcc (a second or two)."""
    import subprocess

    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _C_LIB_PATH


def c_lib() -> ctypes.CDLL:
    global _c_lib
    if _c_lib is None:
        if not os.path.exists(_C_LIB_PATH):
            build_c_oracle()
        lib = ctypes.CDLL(_C_LIB_PATH)
        i64, i32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
        lib.oracle_gemm_rcr.restype = i32
        lib.oracle_gemm_rcr.argtypes = [i32, i32, i32, vp, vp, vp, vp, vp, vp, i64, i64, i64]
        lib.oracle_bmm_rcr_epilogue.restype = i32
        lib.oracle_bmm_rcr_epilogue.argtypes = [i32, i32, i32, vp, vp, vp, vp, vp, vp] + [i64] * 12
        lib.oracle_bmm_softmax_bmm_permute.restype = i32
        lib.oracle_bmm_softmax_bmm_permute.argtypes = [i32, i32, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64,
                                                       ctypes.c_float, i32]
        _c_lib = lib
    return _c_lib


# ---------------------------------------------------------------------------
# torch fp32 expressions (the reference tests' oracle, on the CPU)
# ---------------------------------------------------------------------------
def _f(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if t is None else t.detach().to("cpu", torch.float32)


def torch_epilogue(op: str, y: torch.Tensor, d0=None, d1=None) -> torch.Tensor:
    """Apply the epilogue named by the reference op to y = X W^T + b (fp32)."""
    F = torch.nn.functional
    if op in ("gemm_rcr", "bmm_rcr", "gemm_rcr_bias"):
        return y
    if op == "gemm_rcr_bias_relu":
        return F.relu(y)
    if op in ("gemm_rcr_bias_gelu", "gemm_rcr_bias_fast_gelu"):
        return F.gelu(y, approximate="tanh")
    if op == "gemm_rcr_bias_add":
        return y + d0
    if op == "gemm_rcr_bias_add_add":
        return y + d0 + d1
    if op == "gemm_rcr_bias_add_relu":
        return F.relu(y + d0)
    if op == "gemm_rcr_bias_add_add_relu":
        return F.relu(y + d0 + d1)
    if op == "gemm_rcr_bias_sigmoid":
        return torch.sigmoid(y)
    if op == "gemm_rcr_bias_tanh":
        return torch.tanh(y)
    if op == "gemm_rcr_bias_swish":
        return y * torch.sigmoid(y)
    if op == "gemm_rcr_bias_hardswish":
        return F.hardswish(y)
    if op == "gemm_rcr_bias_mul":
        return y * d0
    if op == "gemm_rcr_bias_mul_add":
        return y * d0 + d1
    if op == "gemm_rcr_bias_sigmoid_mul":
        return torch.sigmoid(y) * d0
    if op == "gemm_rcr_bias_sigmoid_mul_tanh":
        return torch.tanh(torch.sigmoid(y) * d0)
    if op == "gemm_rcr_bias_mul_tanh":
        return torch.tanh(y * d0)
    raise KeyError(op)


def torch_elementwise(func: str, a, b=None) -> torch.Tensor:
    """f(a, b) in fp32 for the reference's FuncEnum name `func`, operands broadcast numpy-style
    (python/aitemplate/compiler/ops/common/elementwise.py:68-87; the function table is
    python/aitemplate/backend/backend_spec.py:117-330).  MAX / MIN return NaN when either operand is NaN
    (fmaxf_nan / fminf_nan, backend/rocm/elementwise/custom_math.h:282-310), RELU maps NaN to 0
    (custom_math.h:117), GELU is the erf form and FASTGELU the tanh form (hgelu / h_fast_gelu of
    backend/cuda/elementwise/custom_math.cuh)."""
    F = torch.nn.functional
    x = _f(a) if isinstance(a, torch.Tensor) else torch.tensor(float(a))
    y = None if b is None else (_f(b) if isinstance(b, torch.Tensor) else torch.tensor(float(b)))
    table = {
        "ADD": lambda: x + y, "SUB": lambda: x - y, "MUL": lambda: x * y, "DIV": lambda: x / y,
        "MAX": lambda: torch.maximum(x, y), "MIN": lambda: torch.minimum(x, y),
        "TANH": lambda: torch.tanh(x), "ABS": lambda: torch.abs(x), "EXP": lambda: torch.exp(x),
        "SQRT": lambda: torch.sqrt(x), "SIGMOID": lambda: torch.sigmoid(x),
        "RELU": lambda: torch.where(x > 0, x, torch.zeros_like(x)), "SILU": lambda: x * torch.sigmoid(x),
        "GELU": lambda: F.gelu(x), "FASTGELU": lambda: F.gelu(x, approximate="tanh"),
        "COS": lambda: torch.cos(x), "SIN": lambda: torch.sin(x), "SIGN": lambda: torch.sign(x),
        "LOGE": lambda: torch.log(x), "LOG1P": lambda: torch.log1p(x), "POW": lambda: torch.pow(x, y),
        "LRELU": lambda: torch.where(x > 0, x, x * y), "SOFTSIGN": lambda: x / (1 + torch.abs(x)),
        "FLOOR": lambda: torch.floor(x), "RECIPROCAL": lambda: 1.0 / x,
    }
    return table[func]()


def torch_gemm(op: str, x, w, bias=None, d0=None, d1=None) -> torch.Tensor:
    """fp32 result of reference op `op`; cast to the input dtype by the caller."""
    y = torch.nn.functional.linear(_f(x), _f(w), _f(bias) if op != "gemm_rcr" else None)
    return torch_epilogue(op, y, _f(d0), _f(d1))


PERMUTE_OPS = {  # op -> (op that names the epilogue, layout)
    "gemm_rcr_permute_m2n3": ("gemm_rcr", "m2n3"),
    "gemm_rcr_bias_permute_m2n3": ("gemm_rcr_bias", "m2n3"),
    "gemm_rcr_bias_permute_m3n2": ("gemm_rcr_bias", "m3n2"),
    "gemm_rcr_bias_permute": ("gemm_rcr_bias", "m3n2"),  # layout "20314" on ROCm
}


def permute_5d(y: torch.Tensor, layout: str, shape) -> torch.Tensor:
    """The 5-D output permutation of the permuting GEMMs applied to a [M, N] result, as the reference's
    tests state it: m2n3 = reshape(M0, M1, N0, N1, N2).permute(2, 0, 3, 1, 4) with shape = (M1, N0, N1)
    (tests/unittest/ops/test_gemm_bias_permute.py:34-42,73-75); m3n2 = reshape(M0, M1, M2, N0, N1)
    .permute(2, 0, 3, 1, 4) with shape = (M1, M2, N0) (:100-108,138-140).  Returns a contiguous tensor."""
    M, N = y.shape
    t1, t2, t3 = (int(t) for t in shape)
    if layout == "m2n3":
        r = y.reshape(M // t1, t1, t2, t3, N // (t2 * t3))
    elif layout == "m3n2":
        r = y.reshape(M // (t1 * t2), t1, t2, t3, N // t3)
    else:
        raise KeyError(layout)
    return r.permute(2, 0, 3, 1, 4).contiguous()


def torch_gemm_permute(op: str, x, w, bias, shape) -> torch.Tensor:
    base, layout = PERMUTE_OPS[op]
    return permute_5d(torch_gemm(base, x.reshape(-1, x.shape[-1]), w, bias), layout, shape)


def torch_multihead_attention(x, qkv_w, qkv_b, proj_w, proj_b, residual, num_heads: int,
                              causal: bool = False) -> torch.Tensor:
    """fp32 self-attention block as the reference's module test states it
    (tests/unittest/ops/test_attention.py / frontend/nn/attention.py:150-290): packed QKV projection,
    softmax(q k^T / sqrt(d)) v per head, output projection (+ residual).  x: [B, S, D]."""
    B, S, D = x.shape
    d = D // num_heads
    qkv = torch.nn.functional.linear(_f(x), _f(qkv_w), _f(qkv_b))
    q, k, v = qkv.reshape(B, S, 3, num_heads, d).permute(2, 0, 3, 1, 4)
    s = torch.matmul(q, k.transpose(-1, -2)) * (d ** -0.5)
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), diagonal=1), float("-inf"))
    o = torch.matmul(torch.softmax(s, dim=-1), v).permute(0, 2, 1, 3).reshape(B * S, D)
    y = torch.nn.functional.linear(o, _f(proj_w), _f(proj_b))
    if residual is not None:
        y = y + _f(residual).reshape(B * S, D)
    return y.reshape(B, S, D)


def torch_mem_eff_attention(q, k, v, causal: bool = False, lengths_kv=None, lengths_q=None) -> torch.Tensor:
    """fp32 attention on [batch, heads, seq, head_dim] operands, result [batch, seq_q, heads, head_dim_v], scale
    head_dim ** -0.5 (python/aitemplate/compiler/ops/attention/mem_eff_attention.py:49-263).  `lengths_kv` is the
    key-padding mask of the reference's test (tests/unittest/ops/test_attention.py:504-523: key n of batch entry b
    counts iff n < lengths_kv[b]).  A batch entry without keys is all zeros here, the kernel library's convention;
    PyTorch's softmax gives NaN for it and the reference's test accepts either side's NaN only if both have it, so
    that case is pinned by nothing in the reference.  `lengths_q`: query rows m >= lengths_q[b] are zeros, again the
    library's convention for rows the reference leaves unspecified (its test blanks them, test_attention.py:661-664)."""
    q, k, v = _f(q), _f(k), _f(v)
    batch, heads, seq_q, d = q.shape
    seq_kv = k.shape[2]
    s = torch.matmul(q, k.transpose(-1, -2)) * (d ** -0.5)
    dead = torch.zeros(batch, 1, seq_q, seq_kv, dtype=torch.bool)
    if lengths_kv is not None:
        lens = lengths_kv.detach().to("cpu").reshape(batch).long()
        dead = dead | (torch.arange(seq_kv)[None, None, None, :] >= lens[:, None, None, None])
    if causal:
        dead = dead | torch.triu(torch.ones(seq_q, seq_kv, dtype=torch.bool), diagonal=1)[None, None]
    s = s.masked_fill(dead, float("-inf"))
    p = torch.softmax(s, dim=-1)
    p = torch.where(torch.isnan(p), torch.zeros_like(p), p)  # rows with every key masked
    v = torch.where(torch.isnan(v) | torch.isinf(v), torch.zeros_like(v), v)  # masked rows may hold anything
    out = torch.matmul(p, v).permute(0, 2, 1, 3).contiguous()  # [batch, seq_q, heads, head_dim_v]
    if lengths_q is not None:
        lq = lengths_q.detach().to("cpu").reshape(batch).long()
        out = out.masked_fill((torch.arange(seq_q)[None, :] >= lq[:, None])[:, :, None, None], 0.0)
    return out


def torch_cross_attention(q_in, k_in, v_in, wq, wk, wv, bq, bk, bv, proj_w, proj_b, residual, num_heads: int,
                          causal: bool = False) -> torch.Tensor:
    """fp32 cross-attention block (python/aitemplate/frontend/nn/attention.py:289-400): separate q, k and v
    projections, softmax(q k^T / sqrt(d)) v per head, output projection (+ residual).
    q_in: [B, S, D]; k_in, v_in: [B, Skv, D]."""
    B, S, D = q_in.shape
    Skv = k_in.shape[1]
    d = D // num_heads
    lin = torch.nn.functional.linear
    q = lin(_f(q_in), _f(wq), _f(bq)).reshape(B, S, num_heads, d).permute(0, 2, 1, 3)
    k = lin(_f(k_in), _f(wk), _f(bk)).reshape(B, Skv, num_heads, d).permute(0, 2, 1, 3)
    v = lin(_f(v_in), _f(wv), _f(bv)).reshape(B, Skv, num_heads, d).permute(0, 2, 1, 3)
    s = torch.matmul(q, k.transpose(-1, -2)) * (d ** -0.5)
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(S, Skv, dtype=torch.bool), diagonal=1), float("-inf"))
    o = torch.matmul(torch.softmax(s, dim=-1), v).permute(0, 2, 1, 3).reshape(B * S, D)
    y = lin(o, _f(proj_w), _f(proj_b))
    if residual is not None:
        y = y + _f(residual).reshape(B * S, D)
    return y.reshape(B, S, D)


def torch_bmm_rcr(q, k) -> torch.Tensor:
    q, k = _f(q), _f(k)
    if q.dim() == 2:
        q = q.unsqueeze(0)
    if k.dim() == 2:
        k = k.unsqueeze(0)
    return torch.matmul(q, k.transpose(-1, -2))


def torch_bmm(layout: str, a, b) -> torch.Tensor:
    """fp32 batched product for the reference's operand layouts, as its tests state them
    (tests/unittest/ops/test_bmm.py:46-50 rcr, :87-89 crr, :120-122 rrr, :153-155 ccr):
    first letter c = A is [B, K, M] and enters transposed, second letter c = B is [B, N, K] and enters transposed."""
    a, b = _f(a), _f(b)
    if a.dim() == 2:
        a = a.unsqueeze(0)
    if b.dim() == 2:
        b = b.unsqueeze(0)
    if layout[0] == "c":
        a = a.transpose(-1, -2)
    if layout[1] == "c":
        b = b.transpose(-1, -2)
    return torch.matmul(a, b)


def torch_bmm_rcr_permute(q, k, d1: int) -> torch.Tensor:
    """bmm(Q, K^T).reshape(B // d1, d1, M, N).permute(0, 2, 1, 3), as the reference's op states it
    (python/aitemplate/compiler/ops/gemm_universal/bmm_rcr_permute.py:36-45, tests/unittest/ops/test_bmm_permute.py)."""
    y = torch_bmm_rcr(q, k)
    B, M, N = y.shape
    return y.reshape(B // d1, d1, M, N).permute(0, 2, 1, 3).contiguous()


def torch_bmm_softmax_bmm_permute(q, k, v, scale: float, num_heads: int, causal: bool = False,
                                  chunk: int = 4) -> torch.Tensor:
    """softmax(Q K^T * scale) V, output [B/G, M, G, O]; chunked over the batch to bound memory.  A NaN score
    counts as -inf (its key is left out): the reference's kernel takes ScaleAndResetNaNToMinusInfinity as the
    functor between the first product and the softmax
    (python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:106, bmm_softmax_bmm.py:99).  A row whose
    scores are all NaN is left to PyTorch's softmax here (NaN) and is pinned by nothing."""
    q, k, v = _f(q), _f(k), _f(v)
    B, M, _ = q.shape
    N, O = v.shape[1], v.shape[2]
    out = torch.empty(B, M, O, dtype=torch.float32)
    for s in range(0, B, chunk):
        att = torch.bmm(q[s:s + chunk], k[s:s + chunk].transpose(1, 2)) * scale
        att = torch.where(torch.isnan(att), torch.full_like(att, float("-inf")), att)
        if causal:
            mask = torch.ones(M, N, dtype=torch.bool).tril()
            att = att.masked_fill(~mask, float("-inf"))
        att = torch.softmax(att, dim=-1)
        out[s:s + chunk] = torch.bmm(att, v[s:s + chunk])
    G = num_heads
    return out.reshape(B // G, G, M, O).permute(0, 2, 1, 3).contiguous()


# ---------------------------------------------------------------------------
# C restatement through ctypes (inputs: fp16 / bf16 torch CPU tensors)
# ---------------------------------------------------------------------------
def _dtype_id(t: torch.Tensor) -> int:
    return {torch.float16: 0, torch.bfloat16: 1}[t.dtype]


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def c_gemm(op: str, x, w, bias=None, d0=None, d1=None, ref_rounding: bool = False) -> torch.Tensor:
    x, w = x.cpu().contiguous(), w.cpu().contiguous()
    bias = None if bias is None else bias.cpu().contiguous()
    d0 = None if d0 is None else d0.cpu().contiguous()
    d1 = None if d1 is None else d1.cpu().contiguous()
    M, K = x.shape
    N = w.shape[0]
    out = torch.empty(M, N, dtype=x.dtype)
    rc = c_lib().oracle_gemm_rcr(EPILOGUE_ID[op], _dtype_id(x), int(ref_rounding), _ptr(x), _ptr(w), _ptr(bias),
                                 _ptr(d0), _ptr(d1), _ptr(out), M, N, K)
    assert rc == 0, rc
    return out


def c_bmm_rcr(q, k, ref_rounding: bool = False) -> torch.Tensor:
    q, k = q.cpu().contiguous(), k.cpu().contiguous()
    if q.dim() == 2:
        q = q.unsqueeze(0)
    if k.dim() == 2:
        k = k.unsqueeze(0)
    B = max(q.shape[0], k.shape[0])
    M, K = q.shape[1], q.shape[2]
    N = k.shape[1]
    sa = 0 if q.shape[0] == 1 and B > 1 else M * K
    sb = 0 if k.shape[0] == 1 and B > 1 else N * K
    out = torch.empty(B, M, N, dtype=q.dtype)
    rc = c_lib().oracle_bmm_rcr_epilogue(0, _dtype_id(q), int(ref_rounding), _ptr(q), _ptr(k), None, None, None,
                                         _ptr(out), B, M, N, K, K, K, N, N, sa, sb, M * N, 0)
    assert rc == 0, rc
    return out


def c_bmm_softmax_bmm_permute(q, k, v, scale: float, num_heads: int, causal: bool = False,
                              ref_rounding: bool = False) -> torch.Tensor:
    q, k, v = q.cpu().contiguous(), k.cpu().contiguous(), v.cpu().contiguous()
    B, M, K = q.shape
    N, O = v.shape[1], v.shape[2]
    G = num_heads
    out = torch.empty(B // G, M, G, O, dtype=q.dtype)
    rc = c_lib().oracle_bmm_softmax_bmm_permute(_dtype_id(q), int(ref_rounding), _ptr(q), _ptr(k), _ptr(v),
                                                _ptr(out), B, M, N, K, O, G, float(scale), int(causal))
    assert rc == 0, rc
    return out


# ---------------------------------------------------------------------------
# Seeded synthetic inputs of the five benchmark configurations.
# Generated on the CPU in fp32 with torch.manual_seed(seed), cast to `dtype`;
# draw order = order listed.  `scale_down` shrinks M (and the batch) for quick
# parity cases while keeping every other dimension.
# ---------------------------------------------------------------------------
def _u(shape, lo, hi):
    return torch.rand(*shape) * (hi - lo) + lo


def config_inputs(cfg: str, dtype=torch.float16, m_override: Optional[int] = None,
                  batch_override: Optional[int] = None) -> Dict[str, torch.Tensor]:
    if cfg == "c1":
        torch.manual_seed(0)
        M = m_override or 256
        d = {"x": _u((M, 1024), -1, 1), "w": _u((1024, 1024), -1, 1), "bias": _u((1024,), -1, 1)}
    elif cfg == "c2a":
        torch.manual_seed(1)
        M = m_override or 24576
        d = {"x": torch.randn(M, 768), "w": torch.randn(3072, 768) * 768 ** -0.5, "bias": _u((3072,), -0.1, 0.1)}
    elif cfg == "c2b":
        torch.manual_seed(2)
        M = m_override or 24576
        d = {"x": torch.randn(M, 3072), "w": torch.randn(768, 3072) * 3072 ** -0.5,
             "bias": _u((768,), -0.1, 0.1), "d0": torch.randn(M, 768)}
    elif cfg == "c3":
        torch.manual_seed(3)
        M = m_override or 12608
        d = {"x": torch.randn(M, 4096), "w": torch.randn(1024, 4096) * 4096 ** -0.5, "bias": torch.randn(1024),
             "d0": torch.randn(M, 1024), "d1": torch.randn(M, 1024)}
    elif cfg == "c4":
        torch.manual_seed(4)
        B = batch_override or 768
        d = {"q": torch.randn(B, 384, 64) / 8.0, "k": torch.randn(B, 384, 64) / 8.0}
    elif cfg == "c5":
        torch.manual_seed(5)
        B = batch_override or 16
        S = m_override or 4096
        d = {"q": torch.randn(B, S, 40), "k": torch.randn(B, S, 40), "v": torch.randn(B, S, 40)}
    else:
        raise KeyError(cfg)
    return {k: v.to(dtype) for k, v in d.items()}


CONFIG_OP = {
    "c1": "gemm_rcr_bias",
    "c2a": "gemm_rcr_bias_gelu",
    "c2b": "gemm_rcr_bias_add",
    "c3": "gemm_rcr_bias_add_add",
    "c4": "bmm_rcr",
    "c5": "bmm_softmax_bmm_permute",
}
C5_HEADS = 8
C5_SCALE = 40 ** -0.5


def config_expected(cfg: str, inp: Dict[str, torch.Tensor]) -> torch.Tensor:
    """fp32 torch oracle of a configuration (not yet cast to fp16)."""
    op = CONFIG_OP[cfg]
    if cfg in ("c1", "c2a", "c2b", "c3"):
        return torch_gemm(op, inp["x"], inp["w"], inp.get("bias"), inp.get("d0"), inp.get("d1"))
    if cfg == "c4":
        return torch_bmm_rcr(inp["q"], inp["k"])
    return torch_bmm_softmax_bmm_permute(inp["q"], inp["k"], inp["v"], C5_SCALE, C5_HEADS)


def config_flops_bytes(cfg: str) -> Tuple[int, int]:
    """Algorithmic FLOPs and bytes (fp16, every tensor once) of a full-size configuration."""
    if cfg == "c1":
        M, N, K, r = 256, 1024, 1024, 0
    elif cfg == "c2a":
        M, N, K, r = 24576, 3072, 768, 0
    elif cfg == "c2b":
        M, N, K, r = 24576, 768, 3072, 1
    elif cfg == "c3":
        M, N, K, r = 12608, 1024, 4096, 2
    elif cfg == "c4":
        B, M, N, K = 768, 384, 384, 64
        return 2 * B * M * N * K, 2 * B * (M * K + N * K + M * N)
    elif cfg == "c5":
        B, M, N, K, O = 16, 4096, 4096, 40, 40
        return 2 * B * M * N * K + 2 * B * M * N * O, 2 * B * (M * K + N * K + N * O + M * O)
    else:
        raise KeyError(cfg)
    return 2 * M * N * K, 2 * (M * K + N * K + N + (1 + r) * M * N)
