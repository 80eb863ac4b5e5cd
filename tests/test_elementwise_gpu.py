"""GPU parity of the stand-alone element-wise kernel through the C ABI, against the fp32 oracle at atol = rtol = 1e-2
(the reference's tolerance, tests/unittest/ops/test_fused_elementwise.py:169,268,309), and of element-wise ops that
compile_model leaves outside the GEMM epilogues.  Covers every function of the kernel, both element types, the
16-byte and the element-wide path (odd sizes, pointers that are only element-aligned), an operand that broadcasts
over leading dims, a constant operand on either side, and the NaN rules of MAX / MIN / RELU
(test_fused_elementwise.py:440-475)."""
import itertools

import pytest
import torch

from aitemplate_amd import eager
from aitemplate_amd.compiler import compile_model, ops
from aitemplate_amd.compiler.ops.common.elementwise import _BINARY_FUNCS, STANDALONE_FUNCS
from aitemplate_amd.frontend import IntVar, Tensor, nn
from aitemplate_amd.testing import detect_target
from oracle import oracle

pytestmark = pytest.mark.gpu
WORKDIR = "/tmp/aitamd_test_elementwise"
_counter = itertools.count()
DTYPES = {"float16": torch.float16, "bfloat16": torch.bfloat16}
# inputs inside every function's domain: LOGE, LOG1P, SQRT, POW need positive values
POSITIVE = {"LOGE", "LOG1P", "SQRT", "POW", "RECIPROCAL", "DIV"}


def _rand(shape, seed, dtype=torch.float16, positive=False):
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(*shape, generator=g) * 1.5
    if positive:
        t = t.abs() + 0.25
    return t.to(dtype)


def _close(got, want, dtype):
    torch.testing.assert_close(got.cpu().float(), want.to(dtype).float(), atol=1e-2, rtol=1e-2, equal_nan=True)


@pytest.mark.parametrize("dtype", list(DTYPES.values()))
@pytest.mark.parametrize("func", sorted(f.name for f in STANDALONE_FUNCS))
def test_every_function_on_both_paths(func, dtype):
    binary = ops.FuncEnum[func] in _BINARY_FUNCS
    for shape in [(64, 1024), (3, 7, 11), (1,), (5, 48)]:  # 16-byte path, element path, one element, broadcast row
        print(f"case elementwise {func} {dtype} shape={shape}", flush=True)
        a = _rand(shape, 1, dtype, func in POSITIVE)
        if not binary:
            _close(eager.elementwise(func, a.cuda()), oracle.torch_elementwise(func, a), dtype)
            continue
        b = _rand(shape, 2, dtype, func in POSITIVE)
        _close(eager.elementwise(func, a.cuda(), b.cuda()), oracle.torch_elementwise(func, a, b), dtype)
        row = _rand((1,) * (len(shape) - 1) + shape[-1:], 3, dtype, func in POSITIVE)
        _close(eager.elementwise(func, a.cuda(), row.cuda()), oracle.torch_elementwise(func, a, row), dtype)
        _close(eager.elementwise(func, row.cuda(), a.cuda()), oracle.torch_elementwise(func, row, a), dtype)
        one = _rand((1,), 4, dtype, func in POSITIVE)
        _close(eager.elementwise(func, a.cuda(), one.cuda()), oracle.torch_elementwise(func, a, one), dtype)
        _close(eager.elementwise(func, a.cuda(), 1.25), oracle.torch_elementwise(func, a, 1.25), dtype)
        _close(eager.elementwise(func, 1.25, a.cuda()), oracle.torch_elementwise(func, 1.25, a), dtype)
    torch.cuda.synchronize()


def test_element_aligned_pointers_large_sizes_and_out_argument():
    # views that start one element into a buffer: the kernel must fall back to element-wide accesses
    base_a, base_b = _rand((4096 * 33 + 1,), 5), _rand((4096 * 33 + 1,), 6)
    da, db = base_a.cuda(), base_b.cuda()
    out = torch.full((4096 * 33 + 1,), float("nan"), dtype=torch.float16, device="cuda")
    eager.elementwise("ADD", da[1:], db[1:], out=out[1:])
    _close(out[1:], oracle.torch_elementwise("ADD", base_a[1:], base_b[1:]), torch.float16)
    assert torch.isnan(out[0]).item()  # nothing before the view was written
    # more elements than one pass of the grid covers (the grid-stride loop), with a row that tiles them
    a, row = _rand((9000, 4096), 7), _rand((4096,), 8)
    got = eager.elementwise("MUL", a.cuda(), row.cuda())
    assert torch.equal(got.cpu(), (a.float() * row.float()).half())  # one rounding of the fp32 product
    # a broadcast period that is not a multiple of 8 takes the element path and still tiles correctly
    a, row = _rand((33, 12), 9), _rand((12,), 10)
    _close(eager.elementwise("SUB", row.cuda(), a.cuda()), oracle.torch_elementwise("SUB", row, a), torch.float16)
    assert eager.elementwise("RELU", torch.empty(0, 8, dtype=torch.float16, device="cuda")).numel() == 0


def test_nan_rules_and_argument_checks():
    nan = float("nan")
    a = torch.tensor([1.0, nan, -2.0, nan, 3.0, -1.0, 0.0, 5.0], dtype=torch.float16)
    b = torch.tensor([nan, 1.0, 4.0, nan, 2.0, -3.0, 0.0, nan], dtype=torch.float16)
    for func in ("MAX", "MIN"):  # NaN if either operand is (torch.maximum / minimum do the same)
        got = eager.elementwise(func, a.cuda(), b.cuda()).cpu()
        want = oracle.torch_elementwise(func, a, b).half()
        assert torch.equal(torch.isnan(got), torch.isnan(want)) and torch.equal(got.nan_to_num(7), want.nan_to_num(7))
    assert eager.elementwise("RELU", a.cuda()).cpu().tolist() == [1.0, 0.0, 0.0, 0.0, 3.0, 0.0, 0.0, 5.0]
    with pytest.raises(ValueError, match="does not broadcast"):
        eager.elementwise("ADD", torch.zeros(4, 6, dtype=torch.float16, device="cuda"),
                          torch.zeros(4, 1, dtype=torch.float16, device="cuda"))
    with pytest.raises(KeyError):
        eager.elementwise("NO_SUCH_FUNC", a.cuda())
    with pytest.raises(RuntimeError, match="not supported"):
        eager.elementwise("ELU", a.cuda())
    with pytest.raises(ValueError, match="GPU tensor"):
        eager.elementwise("RELU", a)


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_compile_model_runs_leftover_elementwise_ops(dtype):
    """A graph whose element-wise ops cannot fold into a GEMM epilogue (the GEMM output is a graph output too, a
    function no epilogue has, a broadcast row, constants on either side) runs them as stand-alone launches, with a
    dynamic batch dim (the reference: test_fused_elementwise.py:180-268, a chain of element-wise ops end to end)."""
    print(f"case compile_model leftover elementwise {dtype}", flush=True)
    tdt = DTYPES[dtype]
    batch = IntVar([1, 6], name="batch")
    X = Tensor([batch, 40, 32], dtype=dtype, name="x", is_input=True)
    row = Tensor([1, 48], dtype=dtype, name="row", is_input=True)
    lin = nn.Linear(32, 48, dtype=dtype)
    lin.name_parameter_tensor("fc")
    h = lin(X)
    h._attrs["is_output"], h._attrs["name"] = True, "h"
    e = ops.elementwise(ops.FuncEnum.EXP)(h * 0.25)
    s = 2.0 - e
    r = ops.elementwise(ops.FuncEnum.MAX)(row, s)
    y = ops.elementwise(ops.FuncEnum.TANH)(r / (ops.elementwise(ops.FuncEnum.ABS)(h) + 1.0))
    y._attrs["is_output"], y._attrs["name"] = True, "y"
    module = compile_model([h, y], detect_target(), WORKDIR, f"leftover_{dtype}_{next(_counter)}")
    for B in (1, 6, 3):
        x, rw = _rand((B, 40, 32), B, tdt), _rand((1, 48), 20, tdt)
        w, bias = _rand((48, 32), 21, tdt) * 0.2, _rand((48,), 22, tdt)
        want_h = oracle.torch_gemm("gemm_rcr_bias", x.reshape(-1, 32), w, bias).reshape(B, 40, 48).to(tdt)
        q = lambda t: t.to(tdt).float()  # every op of the chain rounds its result to the element type
        hh = want_h.float()
        ee = q(torch.exp(q(hh * 0.25)))
        rr = q(torch.maximum(rw.float(), q(2.0 - ee)))
        want_y = q(torch.tanh(q(rr / q(q(hh.abs()) + 1.0))))
        out_h = torch.full((B, 40, 48), float("nan"), dtype=tdt, device="cuda")
        out_y = torch.full((B, 40, 48), float("nan"), dtype=tdt, device="cuda")
        module.set_many_constants_with_tensors({"fc_weight": w.cuda(), "fc_bias": bias.cuda()})
        module.run_with_tensors({"x": x.cuda(), "row": rw.cuda()}, {"h": out_h, "y": out_y})
        torch.testing.assert_close(out_h.cpu().float(), want_h.float(), atol=1e-2, rtol=1e-2)
        torch.testing.assert_close(out_y.cpu().float(), want_y, atol=2e-2, rtol=2e-2)  # seven chained roundings
    module.close()
