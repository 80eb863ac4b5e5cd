"""nn.MultiheadAttention: packed QKV projection, fused attention, output projection.

Counterpart of the ROCm branch of python/aitemplate/frontend/nn/attention.py:95-290:

    qkv  = Linear(dim, 3*dim, specialization="permute", shape=(seq_len, 3, heads), layout="m2n3")
           [B, S, dim] -> [3, B, heads, S, head_dim]        (gemm_rcr[_bias]_permute_m2n3)
    q, k, v = split(qkv, 1, dim=0), each viewed as [B*heads, S, head_dim]
    attn = bmm_softmax_bmm_permute(shape=(heads,), scale=head_dim**-0.5, causal)(q, k, v)
           -> [B, S, heads, head_dim]
    out  = Linear(dim, dim, specialization="add" if has_residual else None)(attn.reshape(B*S, dim)[, residual])
           -> [B, S, dim]

Three kernels per block: two GEMMs and one attention launch; the split and every reshape are views.
The CUDA-only pieces of the reference module (flash attention on a packed tensor, cu_length) have no
counterpart here; `mask_seq` needs dynamic_slice / concatenate, which this backend does not have.

nn.CrossAttention (python/aitemplate/frontend/nn/attention.py:289-400): separate Q / K / V projections of three
inputs, mem_eff_attention on [B, heads, S, head_dim] operands, output projection.  The reference permutes the
projected tensors with a stand-alone permute op; here each projection writes the permuted layout itself
(Linear specialization="permute", shape=(seq, 1, heads), layout="m2n3": [B*S, dim] -> [1, B, heads, S, head_dim]),
so the block is four GEMMs and one attention launch."""
from ...compiler import ops
from .dropout import Dropout
from .linear import Linear
from .module import Module


class MultiheadAttention(Module):
    r"""Multi-Head Attention: MultiHead(Q, K, V) = Concat(head_1, ..., head_h) W^O.

    Args mirror the reference: dim, batch_size, seq_len, num_heads=8, qkv_bias=False, attn_drop=0.0,
    proj_drop=0.0, has_residual=True, causal=False, mask_seq=0, use_mem_eff=False, dtype="float16".
    Dropout probabilities are accepted and ignored (inference)."""

    def __init__(self, dim, batch_size, seq_len, num_heads=8, qkv_bias=False, attn_drop=0.0, proj_drop=0.0,
                 has_residual=True, causal=False, mask_seq=0, use_mem_eff=False, dtype="float16"):
        super().__init__()
        assert dim % num_heads == 0, f"dim {dim} should be divisible by num_heads {num_heads}"
        if mask_seq:
            raise NotImplementedError("mask_seq needs dynamic_slice and concatenate, which this backend lacks")
        if use_mem_eff:
            raise NotImplementedError("use_mem_eff is the CUDA branch of the reference module; ROCm uses "
                                      "bmm_softmax_bmm_permute")
        self.num_heads = num_heads
        self.scale = (dim // num_heads) ** -0.5
        self.causal = causal
        self.has_residual = has_residual
        self.qkv = Linear(dim, dim * 3, bias=qkv_bias, specialization="permute", shape=(seq_len, 3, num_heads),
                          layout="m2n3", dtype=dtype)
        self.attn_drop = Dropout(attn_drop, dtype=dtype)
        self.proj = Linear(dim, dim, specialization="add" if has_residual else None, dtype=dtype)
        self.proj_drop = Dropout(proj_drop, dtype=dtype)

    @staticmethod
    def get_shape(x):
        return [it.value() for it in x._attrs["shape"]]

    def qkv_proj(self, x):
        return self.qkv(x)

    def attention(self, x):
        """x: [3, B, heads, S, head_dim] -> [B, S, heads, head_dim]"""
        q, k, v = ops.split()(x, 1, dim=0)
        _, _, _, seqlen, d = self.get_shape(q)
        op = ops.bmm_softmax_bmm_permute(shape=(self.num_heads,), scale=self.scale, causal=self.causal)
        return op(ops.reshape()(q, [-1, seqlen, d]), ops.reshape()(k, [-1, seqlen, d]),
                  ops.reshape()(v, [-1, seqlen, d]))

    def forward(self, *args):
        assert len(args) >= 1
        x = args[0]
        batch, seq, hidden = self.get_shape(x)
        attn_output = self.attention(self.qkv_proj(x))
        attn_output = ops.reshape()(attn_output, [batch * seq, -1])
        if self.has_residual:
            assert len(args) == 2
            x = self.proj(attn_output, args[1])
        else:
            x = self.proj(attn_output)
        x = self.proj_drop(x)
        return ops.reshape()(x, [batch, seq, hidden])


class CrossAttention(Module):
    r"""Cross Multi-head Attention: queries from one sequence, keys and values from another.

    Args mirror the reference: dim, seq_len, seq_len_kv, num_heads, qkv_bias=False, attn_drop=0.0, proj_drop=0.0,
    has_residual=True, causal=False, dtype="float16".  forward(q, k, v[, residual]) with q: [B, seq_len, dim] and
    k, v: [B, seq_len_kv, dim]; returns [B, seq_len, dim]."""

    def __init__(self, dim, seq_len, seq_len_kv, num_heads, qkv_bias=False, attn_drop=0.0, proj_drop=0.0,
                 has_residual=True, causal=False, dtype="float16"):
        super().__init__()
        assert dim % num_heads == 0, f"dim {dim} should be divisible by num_heads {num_heads}"
        self.num_heads = num_heads
        self.causal = causal
        self.has_residual = has_residual
        self.dim = dim
        self.op = ops.mem_eff_attention(causal=causal)

        def permuting(seq):
            return Linear(dim, dim, bias=qkv_bias, specialization="permute", shape=(seq, 1, num_heads), layout="m2n3",
                          dtype=dtype)

        self.proj_q = permuting(seq_len)
        self.proj_k = permuting(seq_len_kv)
        self.proj_v = permuting(seq_len_kv)
        self.attn_drop = Dropout(attn_drop, dtype=dtype)
        self.proj = Linear(dim, dim, specialization="add" if has_residual else None, dtype=dtype)
        self.proj_drop = Dropout(proj_drop, dtype=dtype)

    def attention(self, q, k, v):
        """[B, S, dim] inputs -> [B, S, heads, head_dim]"""
        head_dim = self.dim // self.num_heads

        def heads_first(proj, x):
            batch, seq, _ = [d.value() for d in x._attrs["shape"]]
            return ops.reshape()(proj(x), [batch, self.num_heads, seq, head_dim])  # [1, B, H, S, D] viewed as 4-D

        return self.op(heads_first(self.proj_q, q), heads_first(self.proj_k, k), heads_first(self.proj_v, v))

    def forward(self, *args):
        assert len(args) >= 3
        x = args[0]
        batch, seq, _ = [d.value() for d in x._attrs["shape"]]
        attn_output = ops.reshape()(self.attention(args[0], args[1], args[2]), [batch * seq, self.dim])
        if self.has_residual:
            assert len(args) == 4
            x = self.proj(attn_output, args[3])
        else:
            x = self.proj(attn_output)
        x = self.proj_drop(x)
        return ops.reshape()(x, [batch, seq, self.dim])


class ScaledDotProductAttention(Module):
    """softmax(q k^T / sqrt(head_dim)) v on [batch, heads, seq, head_dim] operands, result [batch, seq, heads, head_dim]
    (python/aitemplate/frontend/nn/attention.py:403-410)."""

    def __init__(self) -> None:
        super().__init__()

    def forward(self, q, k, v):
        return ops.mem_eff_attention(causal=False)(q, k, v)
