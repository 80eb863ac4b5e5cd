"""GPU parity of the strided row copy and of the splits / concatenates that become one.

The reference's own tests for these ops: tests/unittest/ops/test_split.py, test_concatenate.py (torch.split /
torch.cat as the expectation, as here).  Byte copies: every comparison is exact."""
import ctypes
import itertools
import os

import pytest
import torch

from aitemplate_amd import _kernels, eager
from aitemplate_amd.compiler import compile_model, ops
from aitemplate_amd.frontend import IntImm, Tensor
from aitemplate_amd.testing import detect_target
from aitemplate_amd.utils import shape_utils
from oracle import oracle

pytestmark = pytest.mark.gpu

WORKDIR = os.environ.get("AIT_TEST_WORKDIR", "/tmp/aitemplate_amd_tests")
_counter = itertools.count()


def _rand(shape, seed, dtype=torch.float16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _mark_output(y, name):
    y._attrs["name"] = name
    y._attrs["is_output"] = True
    return y


@pytest.mark.parametrize("shape,dim,sizes", [
    ((4, 10, 8), 1, [3, 7]),           # 16-byte rows and pitches: the widest path
    ((5, 9, 6), 1, [2, 3, 4]),         # 4-byte granularity
    ((3, 7, 5), 1, [1, 6]),            # 2-byte granularity
    ((6, 33), 1, [32, 1]),             # last dim
    ((12, 7), 0, [5, 7]),              # first dim: one row per piece
    ((2, 3, 4, 16), 2, [1, 1, 2]),
    ((70000, 4, 8), 1, [1, 3]),        # more rows than one grid dimension holds
    ((4, 6, 8), 1, [6, 0]),            # an empty piece
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_split_and_concatenate_through_the_c_abi(shape, dim, sizes, dtype):
    print(f"case copy_rows split/concatenate shape={shape} dim={dim} sizes={sizes} {dtype}", flush=True)
    x = _rand(shape, 1, dtype).cuda()
    pieces = eager.split(x, sizes, dim)
    for got, want in zip(pieces, torch.split(x, sizes, dim)):
        assert got.is_contiguous() and torch.equal(got, want)
    back = eager.concatenate(pieces, dim)
    assert torch.equal(back, x)


def test_copy_rows_leaves_the_gaps_alone_and_refuses_bad_arguments():
    print("case copy_rows gaps and errors", flush=True)
    lib = _kernels.load()
    src = torch.arange(8 * 24, dtype=torch.int16, device="cuda").reshape(8, 24)
    dst = torch.full((8, 40), -1, dtype=torch.int16, device="cuda")
    s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # columns 3 .. 13 of src into columns 5 .. 15 of dst
    rc = lib.aitamd_copy_rows(ctypes.c_void_p(src.data_ptr() + 6), ctypes.c_void_p(dst.data_ptr() + 10), 8, 22, 48, 80, s)
    assert rc == 0
    want = torch.full((8, 40), -1, dtype=torch.int16)
    want[:, 5:16] = src.cpu()[:, 3:14]
    assert torch.equal(dst.cpu(), want)
    assert lib.aitamd_copy_rows(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), 8, 64, 48, 80, s) != 0
    assert "pitch" in _kernels.last_error()
    assert lib.aitamd_copy_rows(None, ctypes.c_void_p(dst.data_ptr()), 8, 16, 48, 80, s) != 0
    assert lib.aitamd_copy_rows(None, None, 0, 16, 48, 80, s) == 0  # nothing to do
    assert lib.aitamd_copy_rows(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), -1, 16, 48, 80, s) != 0


@pytest.mark.parametrize("Ms,K,N,dtype", [([4, 33], 32, 24, "float16"), ([128], 72, 40, "bfloat16")])
def test_middle_dim_split_and_first_dim_concatenate_around_gemms(Ms, K, N, dtype):
    """x[m, 2, K] split along dim 1 (copies: the pieces are rows K elements long, 2 K apart), each half through its
    own GEMM, the results interleaved along dim 1 again (copies into the output's rows; m is dynamic)."""
    print(f"case compile_model copies around GEMMs Ms={Ms} K={K} N={N} {dtype}", flush=True)
    tdt = {"float16": torch.float16, "bfloat16": torch.bfloat16}[dtype]
    m = shape_utils.gen_int_var_min_max(Ms, name="m")
    X = Tensor([m, IntImm(2), IntImm(K)], dtype=dtype, name="x", is_input=True)
    W0, W1 = Tensor([N, K], dtype=dtype, name="w0", is_input=True), Tensor([N, K], dtype=dtype, name="w1", is_input=True)
    B = Tensor([N], dtype=dtype, name="b", is_input=True)
    xa, xb = ops.split()(X, 1, dim=1)                                   # [m, 1, K] each
    y0, y1 = ops.gemm_rcr_bias()(xa, W0, B), ops.gemm_rcr_bias()(xb, W1, B)  # [m, 1, N] each
    Y = _mark_output(ops.concatenate()([y0, y1], dim=1), "y")           # [m, 2, N]
    module = compile_model(Y, detect_target(), WORKDIR, f"copy_views_{next(_counter)}")
    for M in Ms:
        x = _rand((M, 2, K), 1, tdt)
        w0, w1, b = _rand((N, K), 2, tdt, K ** -0.5), _rand((N, K), 3, tdt, K ** -0.5), _rand((N,), 4, tdt)
        want = torch.stack([oracle.torch_gemm("gemm_rcr_bias", x[:, 0].contiguous(), w0, b),
                            oracle.torch_gemm("gemm_rcr_bias", x[:, 1].contiguous(), w1, b)], dim=1)
        y = torch.full((M, 2, N), float("nan"), dtype=tdt, device="cuda")
        module.run_with_tensors({"x": x.cuda(), "w0": w0.cuda(), "w1": w1.cuda(), "b": b.cuda()}, [y])
        torch.testing.assert_close(y.cpu().float(), want.to(tdt).float(), atol=1e-2, rtol=1e-2)
    module.close()


def test_concatenate_of_a_gemm_output_and_a_graph_input_and_a_split_piece_as_output():
    """Last-dim concatenate of [GEMM output | graph input]: the GEMM writes its columns through its accessor, the
    input is copied into its own; a piece of a last-dim split of a graph input leaves the graph as an output."""
    print("case compile_model fused and copied columns", flush=True)
    M, K, N, Z = 48, 64, 40, 24
    X = Tensor([M, K], name="x", is_input=True)
    W, B = Tensor([N, K], name="w", is_input=True), Tensor([N], name="b", is_input=True)
    S = Tensor([M, Z + 8], name="s", is_input=True)
    z, tail = ops.split()(S, [Z, 8], dim=1)
    Y = _mark_output(ops.concatenate()([ops.gemm_rcr_bias()(X, W, B), z], dim=1), "y")
    T = _mark_output(tail, "t")
    module = compile_model([Y, T], detect_target(), WORKDIR, f"copy_cat_{next(_counter)}")
    x, w, b, s = _rand((M, K), 1), _rand((N, K), 2, scale=K ** -0.5), _rand((N,), 3), _rand((M, Z + 8), 4)
    y = torch.full((M, N + Z), float("nan"), dtype=torch.float16, device="cuda")
    t = torch.full((M, 8), float("nan"), dtype=torch.float16, device="cuda")
    module.run_with_tensors({"x": x.cuda(), "w": w.cuda(), "b": b.cuda(), "s": s.cuda()}, {"y": y, "t": t})
    torch.testing.assert_close(y.cpu().float()[:, :N], oracle.torch_gemm("gemm_rcr_bias", x, w, b).half().float(),
                               atol=1e-2, rtol=1e-2)
    assert torch.equal(y.cpu()[:, N:], s[:, :Z]) and torch.equal(t.cpu(), s[:, Z:])
    module.close()
