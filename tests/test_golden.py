"""Committed vectors (tests/golden/gemm_family.npz, float64 numpy closed forms) against the CPU
oracle (no GPU) and against the HIP path through the C ABI (GPU)."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemm_family.npz"))
GEMM_OPS = ["gemm_rcr", "gemm_rcr_bias", "gemm_rcr_bias_relu", "gemm_rcr_bias_gelu", "gemm_rcr_bias_add",
            "gemm_rcr_bias_add_add"]


def _t(name):
    return torch.from_numpy(GOLD[name])


def _gemm_args(op):
    args = [_t("gemm_x"), _t("gemm_w")]
    if op != "gemm_rcr":
        args.append(_t("gemm_bias"))
    if "add" in op:
        args.append(_t("gemm_d0"))
    if op.endswith("add_add"):
        args.append(_t("gemm_d1"))
    return args


@pytest.mark.parametrize("op", GEMM_OPS)
def test_oracle_gemm_matches_golden(op):
    want = _t(op)
    # fp32 oracle vs float64 closed form: only accumulation-order noise
    torch.testing.assert_close(oracle.torch_gemm(op, *_gemm_args(op)), want, atol=2e-5, rtol=2e-5)
    # the C oracle rounds its result to fp16
    torch.testing.assert_close(oracle.c_gemm(op, *_gemm_args(op)).float(), want.half().float(), atol=2e-3, rtol=2e-3)


def test_oracle_bmm_and_attention_match_golden():
    torch.testing.assert_close(oracle.torch_bmm_rcr(_t("bmm_q"), _t("bmm_k")), _t("bmm_rcr"), atol=2e-5, rtol=2e-5)
    heads, scale = int(GOLD["attn_heads"]), float(GOLD["attn_scale"])
    got = oracle.torch_bmm_softmax_bmm_permute(_t("attn_q"), _t("attn_k"), _t("attn_v"), scale, heads)
    torch.testing.assert_close(got, _t("bmm_softmax_bmm_permute"), atol=2e-5, rtol=2e-5)
    got = oracle.c_bmm_softmax_bmm_permute(_t("attn_q"), _t("attn_k"), _t("attn_v"), scale, heads)
    torch.testing.assert_close(got.float(), _t("bmm_softmax_bmm_permute"), atol=2e-3, rtol=2e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("op", GEMM_OPS)
def test_hip_gemm_matches_golden(op):
    from aitemplate_amd import eager

    got = eager.gemm(op, *[a.cuda() for a in _gemm_args(op)])
    torch.testing.assert_close(got.float().cpu(), _t(op), atol=1e-2, rtol=1e-2)


@pytest.mark.gpu
def test_hip_bmm_and_attention_match_golden():
    from aitemplate_amd import eager

    got = eager.bmm_rcr(_t("bmm_q").cuda(), _t("bmm_k").cuda())
    torch.testing.assert_close(got.float().cpu(), _t("bmm_rcr"), atol=1e-2, rtol=1e-2)
    heads, scale = int(GOLD["attn_heads"]), float(GOLD["attn_scale"])
    got = eager.bmm_softmax_bmm_permute(_t("attn_q").cuda(), _t("attn_k").cuda(), _t("attn_v").cuda(),
                                        shape=(heads,), scale=scale)
    torch.testing.assert_close(got.float().cpu(), _t("bmm_softmax_bmm_permute"), atol=2e-2, rtol=2e-2)
