"""C-ABI behaviour of a compiled model library, mirroring the reference's
tests/unittest/backend/test_model_api.py (:132-216 error handling, :540-610 dynamic-shape
bounds, :1033-1055 benchmark with threads, :1142-1168 closed model, :1397-1436 allocators,
constants API) on a one-GEMM graph."""
import ctypes
import json
import os

import pytest
import torch

from aitemplate_amd.compiler import AITData, AITemplateAllocatorKind, Model, compile_model, ops
from aitemplate_amd.compiler.model import torch_to_ait_data
from aitemplate_amd.frontend import IntImm, IntVar, Tensor
from aitemplate_amd.testing import detect_target
from oracle import oracle

pytestmark = pytest.mark.gpu
WORKDIR = os.environ.get("AIT_TEST_WORKDIR", "/tmp/aitemplate_amd_tests")
M_MAX, N, K = 64, 72, 40


def _graph(weight_as_constant=False, name="api"):
    m = IntVar([1, M_MAX], name="m")
    X = Tensor(shape=[m, IntImm(K)], name="input_0", is_input=True)
    W = Tensor(shape=[N, K], name="weight", is_input=not weight_as_constant)
    B = Tensor(shape=[N], name="bias", is_input=not weight_as_constant)
    Y = ops.gemm_rcr_bias()(X, W, B)
    Y._attrs["name"] = "output_0"
    Y._attrs["is_output"] = True
    return Y


@pytest.fixture(scope="module")
def module():
    mod = compile_model(_graph(), detect_target(), WORKDIR, "model_api_simple", num_runtimes=2)
    yield mod
    mod.close()


def _data(M=16, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).half()
    w = (torch.randn(N, K, generator=g) * K ** -0.5).half()
    b = torch.randn(N, generator=g).half()
    return x, w, b, oracle.torch_gemm("gemm_rcr_bias", x, w, b).half().float()


def test_names_shapes_dtypes(module):
    assert module.get_input_name_to_index_map() == {"input_0": 0, "weight": 1, "bias": 2}
    assert module.get_output_name_to_index_map() == {"output_0": 0}
    assert module.get_output_maximum_shape(0) == [M_MAX, N]
    assert module.get_output_maximum_shape("output_0") == [M_MAX, N]
    assert module.get_input_maximum_shape(0) == [M_MAX, K]
    assert module.get_output_dtype(0) == 1 and module.get_input_dtype(1) == 1  # kHalf
    assert module.get_num_runtimes() == 2
    with pytest.raises(ValueError):
        module.get_output_maximum_shape("nope")


def test_run_with_dict_list_and_dynamic_shape(module):
    for M in (1, 16, M_MAX):
        x, w, b, want = _data(M, seed=M)
        y = torch.empty(M_MAX, N, dtype=torch.float16, device="cuda")  # maximum-size output buffer
        out = module.run_with_tensors({"bias": b.cuda(), "input_0": x.cuda(), "weight": w.cuda()}, {"output_0": y})
        assert tuple(out["output_0"].shape) == (M, N)
        torch.testing.assert_close(out["output_0"].cpu().float(), want, atol=1e-2, rtol=1e-2)


def test_wrong_number_of_inputs_outputs(module):
    x, w, b, _ = _data()
    y = torch.empty(16, N, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        module.run([], [torch_to_ait_data(y)])
    with pytest.raises(RuntimeError):
        module.run_with_tensors([x.cuda(), w.cuda(), b.cuda()], [])
    with pytest.raises(ValueError):
        module.run_with_tensors({"input_0": x.cuda()}, {"output_0": y})


def test_null_pointers_and_wrong_dtypes(module):
    x, w, b, _ = _data()
    xc, wc, bc = x.cuda(), w.cuda(), b.cuda()
    y = torch.empty(16, N, dtype=torch.float16, device="cuda")
    good = [torch_to_ait_data(t) for t in (xc, wc, bc)]
    with pytest.raises(RuntimeError):
        module.run([AITData(0, [16, K], "float16")] + good[1:], [torch_to_ait_data(y)])
    with pytest.raises(RuntimeError):
        module.run(good, [AITData(0, [16, N], "float16")])
    with pytest.raises(RuntimeError):
        module.run([AITData(xc.data_ptr(), [16, K], "float32")] + good[1:], [torch_to_ait_data(y)])
    with pytest.raises(RuntimeError):
        module.run(good, [AITData(y.data_ptr(), [16, N], "float32")])
    with pytest.raises(RuntimeError):
        module.run_with_tensors([xc, wc.float(), bc], [y])
    # a failed run must not leak the runtime: the pool still serves a good run afterwards
    out = module.run_with_tensors([xc, wc, bc], [y])
    assert tuple(out["output_0"].shape) == (16, N)


def test_dynamic_dim_out_of_range_and_wrong_rank(module):
    x, w, b, _ = _data(M_MAX)
    y = torch.empty(M_MAX + 1, N, dtype=torch.float16, device="cuda")
    big = torch.zeros(M_MAX + 1, K, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        module.run_with_tensors([big, w.cuda(), b.cuda()], [y])
    with pytest.raises(RuntimeError):
        module.run_with_tensors([torch.zeros(0, K, dtype=torch.float16, device="cuda"), w.cuda(), b.cuda()], [y])
    with pytest.raises(RuntimeError):
        module.run_with_tensors([torch.zeros(2, 2, K, dtype=torch.float16, device="cuda"), w.cuda(), b.cuda()], [y])
    with pytest.raises(RuntimeError):  # static dim wrong
        module.run_with_tensors([x.cuda(), torch.zeros(N + 1, K, dtype=torch.float16, device="cuda"), b.cuda()], [y])


def test_cpu_or_noncontiguous_tensors_rejected(module):
    x, w, b, _ = _data()
    y = torch.empty(16, N, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        module.run_with_tensors([x, w.cuda(), b.cuda()], [y])
    with pytest.raises(ValueError):
        module.run_with_tensors([x.cuda(), w.cuda().t().t()[:, ::2], b.cuda()], [y])


def test_num_runtimes_zero_and_null_handle(module):
    with pytest.raises(ValueError):
        Model(module.lib_path, num_runtimes=0)
    dll = ctypes.cdll.LoadLibrary(module.lib_path)
    handle = ctypes.c_void_p()
    assert dll.AITemplateModelContainerCreate(ctypes.byref(handle), ctypes.c_size_t(0), None) == 1
    assert dll.AITemplateModelContainerCreate(None, ctypes.c_size_t(1), None) == 1
    n = ctypes.c_size_t()
    assert dll.AITemplateModelContainerGetNumInputs(None, ctypes.byref(n)) == 1
    assert dll.AITemplateModelContainerDelete(None) == 0  # deleting nothing is fine


def test_use_after_close():
    mod = Model(os.path.join(WORKDIR, "model_api_simple", "test.so"))
    mod.close()
    with pytest.raises(RuntimeError):
        mod.get_num_runtimes()
    mod.close()  # idempotent


def test_benchmark_profile_and_threads(module, tmp_path):
    x, w, b, want = _data(32)
    y = torch.empty(32, N, dtype=torch.float16, device="cuda")
    ins = [x.cuda(), w.cuda(), b.cuda()]
    mean, std, outs = module.benchmark_with_tensors(ins, [y], count=20, repeat=2)
    assert mean > 0 and tuple(outs["output_0"].shape) == (32, N)
    mean_t, _, _ = module.benchmark_with_tensors(ins, [y], count=10, num_threads=3, use_unique_stream_per_thread=True)
    assert mean_t > 0
    torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)
    report = tmp_path / "profile.json"
    module.profile_with_tensors(ins, [y], num_iters=5, filename=str(report))
    data = json.loads(report.read_text())
    assert list(data.keys()) == ["gemm_rcr_bias_0"] and data["gemm_rcr_bias_0"]["ms_per_iter"] > 0


def test_graph_mode_replays_match_eager(module):
    x, w, b, want = _data(24)
    ins = [x.cuda(), w.cuda(), b.cuda()]
    y_eager = torch.empty(24, N, dtype=torch.float16, device="cuda")
    module.run_with_tensors(ins, [y_eager])
    y = torch.empty(24, N, dtype=torch.float16, device="cuda")
    for replay in range(4):
        y.zero_()
        torch.cuda.synchronize()
        module.run_with_tensors(ins, [y], graph_mode=True)
        assert torch.equal(y, y_eager), f"replay {replay} differs from the eager run"
    # a different shape re-captures
    x2, _, _, want2 = _data(8, seed=0)
    y2 = torch.empty(8, N, dtype=torch.float16, device="cuda")
    module.run_with_tensors([x2.cuda(), w.cuda(), b.cuda()], [y2], graph_mode=True)
    want2 = oracle.torch_gemm("gemm_rcr_bias", x2, w, b).half().float()
    torch.testing.assert_close(y2.cpu().float(), want2, atol=1e-2, rtol=1e-2)


def test_outputs_on_host_and_memory_helpers(module):
    x, w, b, want = _data(16)
    y_host = torch.empty(16, N, dtype=torch.float16)
    module._run_with_tensors_outputs_on_host([x.cuda(), w.cuda(), b.cuda()], [y_host])
    torch.testing.assert_close(y_host.float(), want, atol=1e-2, rtol=1e-2)
    # numpy round trip through the library's own malloc / memcpy (no torch involved)
    import numpy as np

    arr = np.arange(24, dtype=np.float32).reshape(4, 6)
    d = module.numpy_to_ait_data(arr)
    back = module.ait_data_to_numpy(d)
    module.free_gpu_memory(d.data_ptr)
    assert np.array_equal(arr, back)


def test_tracking_allocator_counts_bytes():
    mod = compile_model(_graph(), detect_target(), WORKDIR, "model_api_alloc",
                        allocator_kind=AITemplateAllocatorKind.TRACKING)
    n = ctypes.c_size_t()
    mod.DLL.AITemplateTrackingAllocatorGetNumBytes(mod.allocator_handle, ctypes.byref(n))
    assert n.value == 0  # a one-op graph has no internal activations, workspace or constants
    mod.close()


def test_unbound_and_bound_constants():
    # weights as unbound constants: must be set before running
    mod = compile_model(_graph(weight_as_constant=True), detect_target(), WORKDIR, "model_api_unbound")
    assert sorted(mod.get_constant_names()) == ["bias", "weight"]
    x, w, b, want = _data(16)
    y = torch.empty(16, N, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        mod.run_with_tensors([x.cuda()], [y])  # constants not set
    wc, bc = w.cuda(), b.cuda()
    mod.set_many_constants_with_tensors({"weight": wc, "bias": bc})
    mod.run_with_tensors([x.cuda()], [y])
    torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)
    with pytest.raises(RuntimeError):
        mod.set_constant_with_tensor("nope", wc)
    with pytest.raises(RuntimeError):
        mod.set_constant_with_tensor("weight", torch.zeros(N, K + 8, dtype=torch.float16, device="cuda"))
    # double buffering: stage new weights, results change only after the swap
    w2 = (w * 2).cuda()
    mod.set_double_buffer_constant_with_tensor("weight", w2)
    mod.run_with_tensors([x.cuda()], [y])
    torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)
    mod.fold_constants(double_buffer=True)
    mod.swap_constants()
    mod.run_with_tensors([x.cuda()], [y])
    want2 = oracle.torch_gemm("gemm_rcr_bias", x, w * 2, b).half().float()
    torch.testing.assert_close(y.cpu().float(), want2, atol=2e-2, rtol=1e-2)
    mod.close()
    # the same weights bound at compile time: embedded in the library, nothing to set
    mod = compile_model(_graph(weight_as_constant=True), detect_target(), WORKDIR, "model_api_bound",
                        constants={"weight": w, "bias": b})
    assert mod.get_constant_names() == []
    assert sorted(mod.get_constant_names(unbound_constants_only=False)) == ["bias", "weight"]
    mod.run_with_tensors([x.cuda()], [y])
    torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)
    mod.close()


def test_graph_mode_sees_new_constants():
    """A replayed graph must not keep the weight addresses it was captured with."""
    x, w, b, want = _data(16)
    y = torch.empty(16, N, dtype=torch.float16, device="cuda")
    want2 = oracle.torch_gemm("gemm_rcr_bias", x, w * 2, b).half().float()
    # unbound constants: a new buffer through SetConstant, then through the double buffer + swap
    mod = compile_model(_graph(weight_as_constant=True), detect_target(), WORKDIR, "model_api_unbound_graph")
    wc, bc, w2 = w.cuda(), b.cuda(), (w * 2).cuda()
    mod.set_many_constants_with_tensors({"weight": wc, "bias": bc})
    for _ in range(2):
        mod.run_with_tensors([x.cuda()], [y], graph_mode=True)
        torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)
    mod.set_constant_with_tensor("weight", w2)
    for _ in range(2):
        mod.run_with_tensors([x.cuda()], [y], graph_mode=True)
        torch.testing.assert_close(y.cpu().float(), want2, atol=2e-2, rtol=1e-2)
    mod.set_double_buffer_constant_with_tensor("weight", wc)
    mod.run_with_tensors([x.cuda()], [y], graph_mode=True)
    torch.testing.assert_close(y.cpu().float(), want2, atol=2e-2, rtol=1e-2)
    mod.swap_constants()
    mod.run_with_tensors([x.cuda()], [y], graph_mode=True)
    torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)
    mod.close()


def test_bound_constant_double_buffer_takes_effect_at_the_swap():
    x, w, b, want = _data(16)
    y = torch.empty(16, N, dtype=torch.float16, device="cuda")
    want2 = oracle.torch_gemm("gemm_rcr_bias", x, w * 2, b).half().float()
    want3 = oracle.torch_gemm("gemm_rcr_bias", x, w * 2, b * 3).half().float()
    mod = compile_model(_graph(weight_as_constant=True), detect_target(), WORKDIR, "model_api_bound_swap",
                        constants={"weight": w, "bias": b})
    for graph_mode in (False, True):
        mod.run_with_tensors([x.cuda()], [y], graph_mode=graph_mode)
        torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)
    mod.set_double_buffer_constant_with_tensor("weight", (w * 2).cuda())
    for graph_mode in (False, True):  # staged only: the active weights are the compiled-in ones
        mod.run_with_tensors([x.cuda()], [y], graph_mode=graph_mode)
        torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)
    mod.swap_constants()
    for graph_mode in (False, True):  # the bias was not staged and keeps its value
        mod.run_with_tensors([x.cuda()], [y], graph_mode=graph_mode)
        torch.testing.assert_close(y.cpu().float(), want2, atol=2e-2, rtol=1e-2)
    # a second round: the blob that was active first is the staging area now
    mod.set_many_double_buffer_constants_with_tensors({"bias": (b * 3).cuda()})
    mod.run_with_tensors([x.cuda()], [y])
    torch.testing.assert_close(y.cpu().float(), want2, atol=2e-2, rtol=1e-2)
    mod.swap_constants()
    for graph_mode in (True, False):
        mod.run_with_tensors([x.cuda()], [y], graph_mode=graph_mode)
        torch.testing.assert_close(y.cpu().float(), want3, atol=2e-2, rtol=1e-2)
    # the direct call writes the active blob at once
    mod.set_constant_with_tensor("bias", b.cuda())
    mod.run_with_tensors([x.cuda()], [y], graph_mode=True)
    torch.testing.assert_close(y.cpu().float(), want2, atol=2e-2, rtol=1e-2)
    mod.close()


def test_model_library_is_self_contained(tmp_path):
    """test.so copied away from its build directory - alone - loads and runs: it carries the runtime and the kernels
    of the instance tables its ops use, and needs no other file of this package (the reference links everything into
    test.so as well, backend/builder.py:398-527)."""
    import shutil
    import subprocess

    mod = compile_model(_graph(), detect_target(), WORKDIR, "model_api_portable")
    mod.close()
    built = os.path.join(WORKDIR, "model_api_portable", "test.so")
    lone = tmp_path / "elsewhere" / "model.so"
    lone.parent.mkdir()
    shutil.copy2(built, lone)
    needed = subprocess.run(["ldd", str(lone)], capture_output=True, text=True).stdout
    assert "aitemplate_amd" not in needed, needed
    assert "not found" not in needed, needed
    assert "libamdhip64" in needed
    dynamic = subprocess.run(["readelf", "-d", str(lone)], capture_output=True, text=True).stdout
    assert "aitemplate_amd" not in dynamic, dynamic  # no run path into the source tree either
    # one (epilogue, dtype) table of kernels, not the whole 30 MB library
    assert os.path.getsize(lone) < 8 << 20
    x, w, b, want = _data(16)
    y = torch.empty(16, N, dtype=torch.float16, device="cuda")
    with Model(str(lone)) as portable:
        portable.run_with_tensors([x.cuda(), w.cuda(), b.cuda()], [y])
    torch.testing.assert_close(y.cpu().float(), want, atol=1e-2, rtol=1e-2)


def test_ait_recompile_0_loads_existing_library(module, monkeypatch):
    monkeypatch.setenv("AIT_RECOMPILE", "0")
    mod = compile_model(_graph(), detect_target(), WORKDIR, "model_api_simple")
    assert mod.get_output_maximum_shape(0) == [M_MAX, N]
    mod.close()
    with pytest.raises(RuntimeError):
        compile_model(_graph(), detect_target(), WORKDIR, "never_built")
