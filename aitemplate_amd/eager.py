"""Direct launches of the GEMM-family kernels on torch device tensors.

Each helper hands raw device pointers, sizes and the current HIP stream to the
C ABI of the kernel library (``include/aitemplate_amd_kernels.h``); torch is
used for memory and streams only.  The names and argument order follow the
reference frontend ops (``ops.gemm_rcr_bias()(a, b, bias)`` etc.,
python/aitemplate/compiler/ops/gemm_universal/).  There is no fallback path:
a missing library or a CPU tensor raises.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _kernels

_TORCH_DTYPE_ID = {torch.float16: 0, torch.bfloat16: 1}


def _check(t: Optional[torch.Tensor], name: str, dtype=None):
    if t is None:
        return
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor (no CPU path exists)")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name}: dtype {t.dtype} differs from {dtype}")


def _stream_ptr() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t: Optional[torch.Tensor]) -> Optional[ctypes.c_void_p]:
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _row_pitch(t: torch.Tensor, name: str) -> int:
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise ValueError(f"{name} must be 2-D with a contiguous last dimension")
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], t.stride(0))


def gemm_workspace_bytes(op: str, algo: int, M: int, N: int, K: int, dtype=torch.float16, batch: int = 1) -> int:
    """Bytes of scratch memory instance `algo` of `op` needs for this problem (0 for all but the split-K ones)."""
    lib = _kernels.load()
    return int(lib.aitamd_gemm_workspace_bytes(_kernels.EPILOGUE_OF_OP[op], _TORCH_DTYPE_ID[dtype], algo, batch, M, N, K))


def new_workspace(nbytes: int, device="cuda") -> torch.Tensor:
    """A scratch buffer for `gemm(..., workspace=)`: zeroed once (the kernels leave its counters zero again)."""
    return torch.zeros(max(int(nbytes), 16), dtype=torch.uint8, device=device)


def gemm(op: str, a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None,
         d0: Optional[torch.Tensor] = None, d1: Optional[torch.Tensor] = None,
         out: Optional[torch.Tensor] = None, algo: int = -1,
         workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Run reference op `op` (e.g. "gemm_rcr_bias_gelu"): out = epilogue(a @ b.T, bias, d0, d1).

    `a` may have more than 2 dims; leading dims are flattened into M as the
    reference does (gemm_rcr.py:51-77).  `algo` = -1 uses the library heuristic,
    otherwise the instance index (see `_kernels.gemm_algo_names`).  `workspace`: a buffer from
    `new_workspace` for the instances that split K between workgroups (the reference ops' `workspace`
    attribute, gemm_common.py:201-215); without it those instances are not chosen.
    """
    lib = _kernels.load()
    epi = _kernels.EPILOGUE_OF_OP[op]
    dtype = a.dtype
    if dtype not in _TORCH_DTYPE_ID:
        raise ValueError(f"unsupported dtype {dtype}")
    for t, n in ((a, "a"), (b, "b"), (bias, "bias"), (d0, "d0"), (d1, "d1"), (out, "out")):
        _check(t, n, dtype)
    lead = a.shape[:-1]
    K = a.shape[-1]
    M = 1
    for d in lead:
        M *= d
    a2 = a.reshape(M, K)
    N = b.shape[0]
    if b.dim() != 2 or b.shape[1] != K:
        raise ValueError(f"b must be [N, K={K}], got {tuple(b.shape)}")
    if out is None:
        out = torch.empty(*lead, N, dtype=dtype, device=a.device)
    if out.dim() == 2 and out.shape == (M, N) and out.stride(1) == 1 and out.stride(0) >= N:
        out2 = out  # a row-pitched view (rows of a wider buffer) is written in place with ldc = its pitch
    else:
        _check_out(out, M * N, "M*N")
        out2 = out.view(M, N)
    nres = _kernels.NUM_RESIDUALS_OF_EPILOGUE[epi]
    if epi != 0 and (bias is None or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous 1-D tensor of size N")
    d0_2 = d0.reshape(M, N) if d0 is not None else None
    d1_2 = d1.reshape(M, N) if d1 is not None else None
    if nres >= 1 and (d0_2 is None or d0_2.shape != out2.shape):
        raise ValueError("d0 must have the output's shape")
    if nres >= 2 and (d1_2 is None or d1_2.shape != out2.shape):
        raise ValueError("d1 must have the output's shape")
    ldd = _row_pitch(d0_2, "d0") if nres >= 1 else N
    if nres >= 2 and _row_pitch(d1_2, "d1") != ldd:
        raise ValueError("d0 and d1 must share a row pitch")
    if workspace is not None and (not workspace.is_cuda or not workspace.is_contiguous()
                                  or workspace.dtype != torch.uint8):
        raise ValueError("workspace must be a contiguous uint8 GPU tensor (see new_workspace)")
    rc = lib.aitamd_gemm_rcr_ws(epi, _TORCH_DTYPE_ID[dtype], algo, _p(a2), _p(b), _p(bias), _p(d0_2), _p(d1_2),
                                _p(out2), M, N, K, _row_pitch(a2, "a"), _row_pitch(b, "b"), _row_pitch(out2, "out"),
                                ldd, _p(workspace), 0 if workspace is None else workspace.numel(), _stream_ptr())
    _kernels.check(rc, op)
    return out


def _check_out(out: torch.Tensor, numel: int, what: str) -> None:
    """A caller's output buffer is written in place through its raw pointer: it has to be dense and of the
    result's size, or the kernel would write past it (or into a temporary copy)."""
    if not out.is_contiguous() or out.numel() != numel:
        raise ValueError(f"out must be contiguous with {what} = {numel} elements, got shape {tuple(out.shape)} "
                         f"strides {tuple(out.stride())}")


def gemm_permute(op: str, a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor], shape,
                 out: Optional[torch.Tensor] = None, algo: int = -1) -> torch.Tensor:
    """Run a permuting op (`_kernels.PERMUTE_OPS`): linear(a, b, bias) written through the op's 5-D permutation.

    `shape` = (t1, t2, t3) as in the reference ops (gemm_rcr_bias_permute.py:28-76, gemm_rcr_permute.py:33-70).
    Returns [t2, M/t1, t3, t1, N/(t2*t3)] for the m2n3 ops and [t2, M/(t1*t2), t3, t1, N/t3] for the others.
    """
    lib = _kernels.load()
    epi, layout = _kernels.PERMUTE_OPS[op]
    dtype = a.dtype
    if dtype not in _TORCH_DTYPE_ID:
        raise ValueError(f"unsupported dtype {dtype}")
    for t, n in ((a, "a"), (b, "b"), (bias, "bias"), (out, "out")):
        _check(t, n, dtype)
    operands = _kernels.LAYOUT_ID[_kernels.PERMUTE_OPERANDS.get(op, "rcr")]
    K = a.shape[-1]
    a2 = a.reshape(-1, K)
    b_k, b_n = (0, 1) if operands & 1 else (1, 0)  # gemm_rrr_bias_permute takes B as [K, N]
    if b.dim() != 2 or b.shape[b_k] != K:
        raise ValueError(f"b does not match K={K}: got {tuple(b.shape)}")
    M, N = a2.shape[0], b.shape[b_n]
    if epi != 0 and (bias is None or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous 1-D tensor of size N")
    t1, t2, t3 = (int(t) for t in shape)
    if layout == _kernels.PERMUTE_M2N3:
        if M % t1 or N % (t2 * t3):
            raise ValueError(f"[{M}, {N}] does not split by shape {tuple(shape)}")
        out_shape = (t2, M // t1, t3, t1, N // (t2 * t3))
    else:
        if M % (t1 * t2) or N % t3:
            raise ValueError(f"[{M}, {N}] does not split by shape {tuple(shape)}")
        out_shape = (t2, M // (t1 * t2), t3, t1, N // t3)
    if out is None:
        out = torch.empty(out_shape, dtype=dtype, device=a.device)
    elif not out.is_contiguous() or out.numel() != M * N:
        raise ValueError("out must be contiguous with M*N elements")
    rc = lib.aitamd_gemm_permute(operands, epi, _TORCH_DTYPE_ID[dtype], algo, _p(a2), _p(b), _p(bias), _p(out), M, N, K,
                                 _row_pitch(a2, "a"), _row_pitch(b, "b"), layout, t1, t2, t3, _stream_ptr())
    _kernels.check(rc, op)
    return out


def bmm_rcr(a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None, algo: int = -1) -> torch.Tensor:
    """out[b] = a[b] @ b[b].T with batch broadcast when one operand is 2-D or has batch 1
    (python/aitemplate/compiler/ops/gemm_universal/bmm.py:72-90)."""
    lib = _kernels.load()
    dtype = a.dtype
    for t, n in ((a, "a"), (b, "b"), (out, "out")):
        _check(t, n, dtype)
    a3 = a if a.dim() == 3 else a.unsqueeze(0)
    b3 = b if b.dim() == 3 else b.unsqueeze(0)
    if not (a3.is_contiguous() and b3.is_contiguous()):
        raise ValueError("bmm_rcr operands must be contiguous")
    B = max(a3.shape[0], b3.shape[0])
    if a3.shape[0] not in (1, B) or b3.shape[0] not in (1, B):
        raise ValueError("batch sizes must match or be 1")
    M, K = a3.shape[1], a3.shape[2]
    N = b3.shape[1]
    if b3.shape[2] != K:
        raise ValueError("K mismatch")
    if out is None:
        out = torch.empty(B, M, N, dtype=dtype, device=a.device)
    else:
        _check_out(out, B * M * N, "B*M*N")
    sa = 0 if (a3.shape[0] == 1 and B > 1) else M * K
    sb = 0 if (b3.shape[0] == 1 and B > 1) else N * K
    rc = lib.aitamd_bmm_rcr(_TORCH_DTYPE_ID[dtype], algo, _p(a3), _p(b3), _p(out), B, M, N, K, K, K, N, sa, sb,
                            M * N, _stream_ptr())
    _kernels.check(rc, "bmm_rcr")
    return out


def bmm(layout: str, a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None, d1: int = 0,
        algo: int = -1) -> torch.Tensor:
    """Batched GEMM for the operand layouts "rcr", "rrr", "ccr", "crr" of the reference
    (python/aitemplate/compiler/ops/gemm_universal/bmm_xxx.py): first letter r = A is [B, M, K], c = A is
    [B, K, M]; second letter r = B is [B, K, N], c = B is [B, N, K]; the result is [B, M, N], or
    [B // d1, M, d1, N] when d1 > 0 (the *_permute ops).  2-D or batch-1 operands broadcast."""
    lib = _kernels.load()
    lay = _kernels.LAYOUT_ID[layout]
    dtype = a.dtype
    for t, n in ((a, "a"), (b, "b"), (out, "out")):
        _check(t, n, dtype)
    a3 = a if a.dim() == 3 else a.unsqueeze(0)
    b3 = b if b.dim() == 3 else b.unsqueeze(0)
    if not (a3.is_contiguous() and b3.is_contiguous()):
        raise ValueError("bmm operands must be contiguous")
    B = max(a3.shape[0], b3.shape[0])
    if a3.shape[0] not in (1, B) or b3.shape[0] not in (1, B):
        raise ValueError("batch sizes must match or be 1")
    M, K = (a3.shape[2], a3.shape[1]) if lay & 2 else (a3.shape[1], a3.shape[2])
    N, Kb = (b3.shape[2], b3.shape[1]) if lay & 1 else (b3.shape[1], b3.shape[2])
    if Kb != K:
        raise ValueError("K mismatch")
    if d1 and (d1 < 0 or B % d1):
        raise ValueError(f"batch {B} is not a multiple of d1 = {d1}")
    if out is None:
        out = torch.empty((B // d1, M, d1, N) if d1 else (B, M, N), dtype=dtype, device=a.device)
    elif not out.is_contiguous() or out.numel() != B * M * N:
        raise ValueError("out must be contiguous with B*M*N elements")
    sa = 0 if (a3.shape[0] == 1 and B > 1) else M * K
    sb = 0 if (b3.shape[0] == 1 and B > 1) else N * K
    rc = lib.aitamd_bmm(lay, _TORCH_DTYPE_ID[dtype], algo, _p(a3), _p(b3), _p(out), B, M, N, K, a3.shape[2],
                        b3.shape[2], N, sa, sb, M * N, d1, _stream_ptr())
    _kernels.check(rc, f"bmm_{layout}")
    return out


def bmm_add(layout: str, a: torch.Tensor, b: torch.Tensor, d0: torch.Tensor, out: Optional[torch.Tensor] = None,
            algo: int = -1) -> torch.Tensor:
    """bmm(layout, a, b) + d0 with d0 of the result's shape [B, M, N]: the bmm_rrr_add / bmm_ccr_add / bmm_crr_add
    ops (python/aitemplate/compiler/ops/gemm_universal/bmm_xxx_add.py)."""
    lib = _kernels.load()
    lay = _kernels.LAYOUT_ID[layout]
    dtype = a.dtype
    for t, n in ((a, "a"), (b, "b"), (d0, "d0"), (out, "out")):
        _check(t, n, dtype)
    if a.dim() != 3 or b.dim() != 3 or not (a.is_contiguous() and b.is_contiguous() and d0.is_contiguous()):
        raise ValueError("bmm_add operands must be contiguous 3-D tensors")
    B = a.shape[0]
    M, K = (a.shape[2], a.shape[1]) if lay & 2 else (a.shape[1], a.shape[2])
    N, Kb = (b.shape[2], b.shape[1]) if lay & 1 else (b.shape[1], b.shape[2])
    if Kb != K or b.shape[0] != B:
        raise ValueError("A and B do not match")
    if tuple(d0.shape) != (B, M, N):
        raise ValueError(f"d0 must be [{B}, {M}, {N}], got {tuple(d0.shape)}")
    if out is None:
        out = torch.empty(B, M, N, dtype=dtype, device=a.device)
    else:
        _check_out(out, B * M * N, "B*M*N")
    rc = lib.aitamd_bmm_add(lay, _TORCH_DTYPE_ID[dtype], algo, _p(a), _p(b), _p(d0), _p(out), B, M, N, K, a.shape[2],
                            b.shape[2], N, N, M * K, N * K, M * N, M * N, _stream_ptr())
    _kernels.check(rc, f"bmm_{layout}_add")
    return out


def bmm_rcr_permute(a: torch.Tensor, b: torch.Tensor, shape, out: Optional[torch.Tensor] = None,
                    algo: int = -1) -> torch.Tensor:
    """bmm_rcr stored as [B // d1, M, d1, N] with shape = (d1,)
    (python/aitemplate/compiler/ops/gemm_universal/bmm_rcr_permute.py:28-116)."""
    lib = _kernels.load()
    dtype = a.dtype
    for t, n in ((a, "a"), (b, "b"), (out, "out")):
        _check(t, n, dtype)
    a3 = a if a.dim() == 3 else a.unsqueeze(0)
    b3 = b if b.dim() == 3 else b.unsqueeze(0)
    if not (a3.is_contiguous() and b3.is_contiguous()):
        raise ValueError("bmm_rcr_permute operands must be contiguous")
    B = max(a3.shape[0], b3.shape[0])
    if a3.shape[0] not in (1, B) or b3.shape[0] not in (1, B):
        raise ValueError("batch sizes must match or be 1")
    M, K = a3.shape[1], a3.shape[2]
    N = b3.shape[1]
    if b3.shape[2] != K:
        raise ValueError("K mismatch")
    d1 = int(shape[0])
    if d1 <= 0 or B % d1:
        raise ValueError(f"batch {B} is not a multiple of d1 = {d1}")
    if out is None:
        out = torch.empty(B // d1, M, d1, N, dtype=dtype, device=a.device)
    elif not out.is_contiguous() or out.numel() != B * M * N:
        raise ValueError("out must be contiguous with B*M*N elements")
    sa = 0 if (a3.shape[0] == 1 and B > 1) else M * K
    sb = 0 if (b3.shape[0] == 1 and B > 1) else N * K
    rc = lib.aitamd_bmm_rcr_permute(_TORCH_DTYPE_ID[dtype], algo, _p(a3), _p(b3), _p(out), B, M, N, K, K, K, sa, sb,
                                    d1, _stream_ptr())
    _kernels.check(rc, "bmm_rcr_permute")
    return out


def bmm_softmax_bmm_permute(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, shape, scale: float = 1.0,
                            causal: bool = False, layout: str = "0213",
                            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(scale * q @ k^T) @ v with the [B, M, O] result written as [B / G, M, G, O], G = shape[0]
    (python/aitemplate/compiler/ops/gemm_universal/bmm_softmax_bmm_permute.py:30-194)."""
    lib = _kernels.load()
    if layout != "0213":
        raise NotImplementedError(f"{layout} is not implemented!")
    dtype = q.dtype
    for t, n in ((q, "q"), (k, "k"), (v, "v"), (out, "out")):
        _check(t, n, dtype)
    if not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
        raise ValueError("bmm_softmax_bmm_permute operands must be contiguous")
    B, M, K = q.shape
    N, O = v.shape[1], v.shape[2]
    if k.shape != (B, N, K) or v.shape[0] != B:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    G = int(shape[0])
    if out is None:
        out = torch.empty(B // G, M, G, O, dtype=dtype, device=q.device)
    else:
        _check_out(out, B * M * O, "B*M*O")
    rc = lib.aitamd_bmm_softmax_bmm_permute(_TORCH_DTYPE_ID[dtype], _p(q), _p(k), _p(v), _p(out), B, M, N, K, O, G,
                                            float(scale), int(bool(causal)), _stream_ptr())
    _kernels.check(rc, "bmm_softmax_bmm_permute")
    return out


def mem_eff_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, causal: bool = False,
                      lengths_kv: Optional[torch.Tensor] = None, lengths_q: Optional[torch.Tensor] = None,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(q k^T / sqrt(head_dim)) v on [batch, heads, seq, head_dim] operands, written as
    [batch, seq_q, heads, head_dim_v]; `lengths_kv` ([batch] or [batch, 1], int32, on the device) limits batch entry b
    to its first lengths_kv[b] keys; `lengths_q`, same form, zeroes the query rows past lengths_q[b]
    (python/aitemplate/compiler/ops/attention/mem_eff_attention.py:49-263)."""
    lib = _kernels.load()
    dtype = q.dtype
    for t, n in ((q, "q"), (k, "k"), (v, "v"), (out, "out")):
        _check(t, n, dtype)
    if not (q.dim() == k.dim() == v.dim() == 4):
        raise ValueError("mem_eff_attention operands must be [batch, heads, seq, head_dim]")
    if not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
        raise ValueError("mem_eff_attention operands must be contiguous")
    batch, heads, seq_q, head_dim = q.shape
    seq_kv, head_dim_v = v.shape[2], v.shape[3]
    if k.shape != (batch, heads, seq_kv, head_dim) or v.shape[:2] != (batch, heads):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    for lengths, name in ((lengths_kv, "lengths_kv"), (lengths_q, "lengths_q")):
        if lengths is not None and (lengths.dtype != torch.int32 or lengths.numel() != batch
                                    or not lengths.is_contiguous() or lengths.device != q.device):
            raise ValueError(f"{name} must be a contiguous int32 tensor with one entry per batch on the operands' device")
    if out is None:
        out = torch.empty(batch, seq_q, heads, head_dim_v, dtype=dtype, device=q.device)
    else:
        _check_out(out, batch * seq_q * heads * head_dim_v, "batch*seq_q*heads*head_dim_v")
    rc = lib.aitamd_mem_eff_attention(_TORCH_DTYPE_ID[dtype], _p(q), _p(k), _p(v), _p(out), batch, heads, seq_q, seq_kv,
                                      head_dim, head_dim_v, float(head_dim) ** -0.5, int(bool(causal)),
                                      _p(lengths_kv), _p(lengths_q), _stream_ptr())
    _kernels.check(rc, "mem_eff_attention")
    return out


def elementwise(func: str, a: torch.Tensor, b=None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Stand-alone element-wise op `func` (a FuncEnum name, e.g. "ADD", "FASTGELU"): f(a, b) with b a tensor whose
    shape is a's or a suffix of it (leading 1s allowed), a number, or None for the unary functions.  A number or a
    broadcast tensor as the FIRST operand: pass it as `a` and the full-shape tensor as `b`."""
    from .compiler.ops.common.epilogue import FuncEnum

    lib = _kernels.load()
    fid = FuncEnum[func].value
    swap = 0
    if not isinstance(a, torch.Tensor) or (isinstance(b, torch.Tensor) and b.numel() > a.numel()):
        a, b, swap = b, a, 1
    _check(a, "a", None)
    if a.dtype not in _TORCH_DTYPE_ID or not a.is_contiguous():
        raise ValueError("a must be a contiguous fp16 / bf16 GPU tensor")
    b_ptr, b_period, b_value = None, 1, 0.0
    if isinstance(b, torch.Tensor):
        _check(b, "b", a.dtype)
        if not b.is_contiguous():
            raise ValueError("b must be contiguous")
        shape = list(b.shape)
        while shape and shape[0] == 1:
            shape.pop(0)
        if shape != list(a.shape)[len(a.shape) - len(shape):]:
            raise ValueError(f"b of shape {tuple(b.shape)} does not broadcast over the leading dims of {tuple(a.shape)}")
        b_ptr, b_period = _p(b), max(1, b.numel())
    elif b is not None:
        b_value = float(b)
    if out is None:
        out = torch.empty_like(a)
    else:
        _check(out, "out", a.dtype)
        _check_out(out, a.numel(), "a.numel()")
    rc = lib.aitamd_elementwise(fid, _TORCH_DTYPE_ID[a.dtype], _p(a), b_ptr, _p(out), a.numel(), b_period, b_value, swap,
                                _stream_ptr())
    _kernels.check(rc, f"elementwise({func})")
    return out


def split(x: torch.Tensor, sizes, dim: int) -> Tuple[torch.Tensor, ...]:
    """torch.split(x, sizes, dim) with every piece a new contiguous tensor, one strided row copy per piece
    (python/aitemplate/compiler/ops/tensor/split.py:31-170)."""
    lib = _kernels.load()
    if not x.is_cuda or not x.is_contiguous():
        raise ValueError("x must be a contiguous GPU tensor")
    dim %= x.dim()
    if sum(sizes) != x.shape[dim]:
        raise ValueError(f"split sizes {list(sizes)} do not add up to {x.shape[dim]}")
    rows = 1
    for d in x.shape[:dim]:
        rows *= d
    inner = x.element_size()
    for d in x.shape[dim + 1:]:
        inner *= d
    outs, start = [], 0
    for n in sizes:
        o = torch.empty(*x.shape[:dim], n, *x.shape[dim + 1:], dtype=x.dtype, device=x.device)
        rc = lib.aitamd_copy_rows(ctypes.c_void_p(x.data_ptr() + start * inner), _p(o), rows, n * inner, x.shape[dim] * inner, n * inner,
                                  _stream_ptr())
        _kernels.check(rc, "split")
        outs.append(o)
        start += n
    return tuple(outs)


def concatenate(tensors, dim: int) -> torch.Tensor:
    """torch.cat(tensors, dim) as one strided row copy per input
    (python/aitemplate/compiler/ops/tensor/concatenate.py:31-170)."""
    lib = _kernels.load()
    first = tensors[0]
    dim %= first.dim()
    for t in tensors:
        if not t.is_cuda or not t.is_contiguous() or t.dtype != first.dtype:
            raise ValueError("inputs must be contiguous GPU tensors of one dtype")
        if list(t.shape[:dim]) + list(t.shape[dim + 1:]) != list(first.shape[:dim]) + list(first.shape[dim + 1:]):
            raise ValueError("inputs differ in a dim other than the concatenated one")
    total = sum(t.shape[dim] for t in tensors)
    out = torch.empty(*first.shape[:dim], total, *first.shape[dim + 1:], dtype=first.dtype, device=first.device)
    rows = 1
    for d in first.shape[:dim]:
        rows *= d
    inner = first.element_size()
    for d in first.shape[dim + 1:]:
        inner *= d
    start = 0
    for t in tensors:
        n = t.shape[dim]
        rc = lib.aitamd_copy_rows(_p(t), ctypes.c_void_p(out.data_ptr() + start * inner), rows, n * inner, n * inner, total * inner,
                                  _stream_ptr())
        _kernels.check(rc, "concatenate")
        start += n
    return out
