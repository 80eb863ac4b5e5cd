"""Host-side logic, no GPU: op construction and shape inference, exec keys and profiler command
lines (golden strings from the reference's formats), registry, naming, memory planning, code
generation, the model build and the exported C ABI, and the profiler runner with fake commands
(the latter mirrors tests/unittest/backend/test_profiler.py:48-66)."""
import copy
import ctypes
import os
import re
import stat
import subprocess
import sys
from random import random
from time import sleep

import pytest

from aitemplate_amd.backend import registry
from aitemplate_amd.backend.profiler_runner import ProfilerRunner, extract_profile_result
from aitemplate_amd.compiler import compile_model, ops, transform
from aitemplate_amd.compiler.base import DynamicProfileStrategy, IntImm, IntVar, Tensor
from aitemplate_amd.compiler.ops.gemm_universal.gemm_common import gemm_inverse_key_func
from aitemplate_amd.compiler.transform.name_graph import reset_name_counters
from aitemplate_amd.frontend import nn
from aitemplate_amd.testing import detect_target
from aitemplate_amd.utils import alignment, shape_utils

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _gemm_bias_graph(Ms=(256,), N=1024, K=1024, op="gemm_rcr_bias"):
    m = shape_utils.gen_int_var_min_max(list(Ms), name="m")
    X = Tensor(shape=[m, IntImm(K)], name="input_0", is_input=True)
    W = Tensor(shape=[IntImm(N), IntImm(K)], name="input_1", is_input=True)
    B = Tensor(shape=[IntImm(N)], name="input_2", is_input=True)
    Y = getattr(ops, op)()(X, W, B)
    Y._attrs["name"] = "output_0"
    Y._attrs["is_output"] = True
    return Y


# ---- IR -------------------------------------------------------------------------------
def test_intvar_intimm_semantics():
    assert IntImm(4) == 4 and IntImm(4) == IntImm(4) and IntImm(4) != IntImm(5)
    with pytest.raises(RuntimeError):
        IntImm(1.5)
    with pytest.raises(RuntimeError):
        IntVar([3])
    with pytest.raises(RuntimeError):
        IntVar([-1, 4])
    v = IntVar([8, 2, 4], name="b")
    assert (v.lower_bound(), v.upper_bound()) == (2, 8)
    assert IntVar([1, 9], name="b") == v  # same symbol
    assert isinstance(shape_utils.gen_int_var_min_max([7, 7]), IntImm)
    assert isinstance(shape_utils.gen_int_var_min_max([1, 7]), IntVar)
    t = Tensor([3, v])
    assert [type(d).__name__ for d in t.shape()] == ["IntImm", "IntVar"]
    assert t.size_bytes() == 3 * 8 * 2
    with pytest.raises(RuntimeError):
        Tensor(["x"])


def test_alignment_helpers():
    assert alignment.find_max_alignment(1024, "float16") == 8
    assert alignment.find_max_alignment(4, "float16") == 4
    assert alignment.find_max_alignment(81, "float16") == 1
    assert alignment.find_max_alignment(6, "float32") == 2


# ---- ops ------------------------------------------------------------------------------
def test_gemm_shape_inference_and_attrs():
    Y = _gemm_bias_graph()
    op = list(Y.src_ops())[0]
    assert [d.value() for d in Y.shape()] == [256, 1024]
    for key in ("op", "has_profiler", "f_ab_alignment", "epilogue_alignment", "epilogue", "workspace", "split_k",
                "num_sources", "alpha", "permute_shape", "inputs", "input_accessors", "outputs",
                "output_accessors"):
        assert key in op._attrs, key
    assert op._attrs["op"] == "gemm_rcr_bias" and op._attrs["epilogue_alignment"] == 8
    # leading dims of A are flattened into M
    X3 = Tensor([4, 50, 64])
    Y3 = ops.gemm_rcr()(X3, Tensor([72, 64]))
    assert [d.value() for d in Y3.shape()] == [4, 50, 72]


def test_gemm_argument_errors():
    with pytest.raises(RuntimeError, match="A/B shape mismatch"):
        ops.gemm_rcr()(Tensor([4, 8]), Tensor([4, 16]))
    with pytest.raises(RuntimeError, match="K must be static"):
        kdim = IntVar([1, 8], name="k")
        ops.gemm_rcr()(Tensor([4, kdim]), Tensor([4, kdim]))
    with pytest.raises(RuntimeError, match="Bias should be 1D"):
        ops.gemm_rcr_bias()(Tensor([4, 8]), Tensor([6, 8]), Tensor([1, 6]))
    with pytest.raises(RuntimeError, match="doesn't match"):
        ops.gemm_rcr_bias()(Tensor([4, 8]), Tensor([6, 8]), Tensor([5]))
    with pytest.raises(RuntimeError, match="doesn't match gemm_bias"):
        ops.gemm_rcr_bias_add()(Tensor([4, 8]), Tensor([6, 8]), Tensor([6]), Tensor([4, 5]))
    with pytest.raises(RuntimeError):
        ops.gemm_rcr_bias_add_add()(Tensor([4, 8]), Tensor([6, 8]), Tensor([6]), Tensor([4, 6]))  # needs d1
    with pytest.raises(RuntimeError, match="same data type"):
        ops.gemm_rcr()(Tensor([4, 8]), Tensor([6, 8], dtype="float32"))
    with pytest.raises(RuntimeError, match="2 dimensions"):
        ops.gemm_rcr()(Tensor([4, 8]), Tensor([2, 6, 8]))


def test_exec_keys_are_the_reference_format():
    op = list(_gemm_bias_graph().src_ops())[0]
    op._extract_exec_path(DynamicProfileStrategy.MAX)
    assert list(op._attrs["exec_path"]) == ["M == 256 && N == 1024 && K == 1024"]
    assert gemm_inverse_key_func("M == 256 && N == 1024 && K == 1024") == [256, 1024, 1024]
    op = list(_gemm_bias_graph(Ms=(1, 1024), N=64, K=32).src_ops())[0]
    op._extract_exec_path(DynamicProfileStrategy.MAX)
    item = list(op._attrs["exec_path"].values())[0]
    assert item.profiling_key == "M == 1024 && N == 64 && K == 32"
    assert item.exec_cond == "M >= 1 && M <= 1024 && N == 64 && K == 32"
    op._extract_exec_path(DynamicProfileStrategy.MIN)
    assert list(op._attrs["exec_path"]) == ["M == 1 && N == 64 && K == 32"]
    with pytest.raises(NotImplementedError):
        op._extract_exec_path(DynamicProfileStrategy.HINTS)
    # bmm keys are ordered B, M, N, K; attention B, M, N, K, O
    b = ops.bmm_rcr()
    b(Tensor([768, 384, 64]), Tensor([768, 384, 64]))
    b._extract_exec_path(DynamicProfileStrategy.MAX)
    assert list(b._attrs["exec_path"]) == ["B == 768 && M == 384 && N == 384 && K == 64"]
    a = ops.bmm_softmax_bmm_permute(shape=(8,), scale=0.5)
    a(Tensor([16, 4096, 40]), Tensor([16, 4096, 40]), Tensor([16, 4096, 40]))
    a._extract_exec_path(DynamicProfileStrategy.MAX)
    assert list(a._attrs["exec_path"]) == ["B == 16 && M == 4096 && N == 4096 && K == 40 && O == 40"]


def test_bmm_rules():
    y = ops.bmm_rcr()(Tensor([6, 40, 32]), Tensor([24, 32]))
    assert [d.value() for d in y.shape()] == [6, 40, 24]
    y = ops.bmm_rcr()(Tensor([1, 40, 32]), Tensor([5, 24, 32]))
    assert [d.value() for d in y.shape()] == [5, 40, 24]
    with pytest.raises(RuntimeError, match="same batch_size"):
        ops.bmm_rcr()(Tensor([2, 40, 32]), Tensor([3, 24, 32]))
    with pytest.raises(RuntimeError, match="Use gemm instead"):
        ops.bmm_rcr()(Tensor([40, 32]), Tensor([24, 32]))


def test_attention_op_output_attrs_and_copy():
    op = ops.bmm_softmax_bmm_permute(shape=(8,), scale=0.158, causal=True)
    out = op(Tensor([16, 4096, 40]), Tensor([16, 4096, 40]), Tensor([16, 4096, 40]))
    assert [d.value() for d in out.shape()] == [2, 4096, 8, 40]
    assert out._attrs["is_view_of"] is op._attrs["outputs"][0]
    assert op._attrs["op"] == "bmm_softmax_bmm_permute_causal"
    attrs = op._get_op_attributes()
    assert attrs == {"causal": True, "layout": "0213", "scale": 0.158, "shape": (8,)}
    clone = ops.bmm_softmax_bmm_permute(**attrs)
    assert clone._attrs["op"] == op._attrs["op"] and clone._attrs["layout"] == op._attrs["layout"]
    dc = copy.deepcopy(op)
    assert dc._attrs["scale"] == 0.158 and dc is not op
    with pytest.raises(NotImplementedError):
        ops.bmm_softmax_bmm_permute(shape=(8,), layout="0123")(Tensor([16, 8, 8]), Tensor([16, 8, 8]), Tensor([16, 8, 8]))


def test_nn_linear_picks_the_fused_op_by_name():
    lin = nn.Linear(64, 72, specialization="fast_gelu")
    lin.name_parameter_tensor("ffn")
    y = lin(Tensor([10, 64], name="x", is_input=True))
    assert list(y.src_ops())[0]._attrs["op"] == "gemm_rcr_bias_fast_gelu"
    assert lin.weight.tensor()._attrs["name"] == "ffn_weight"
    assert nn.Linear(8, 8, bias=False).op._attrs["op"] == "gemm_rcr"
    with pytest.raises(NotImplementedError):
        nn.Linear(8, 8, specialization="nope")


# ---- registry / target ---------------------------------------------------------------------
def test_registry_has_every_hook_for_every_op():
    detect_target()  # importing the ROCm backend registers the hooks
    for op in ("gemm_rcr", "gemm_rcr_bias", "gemm_rcr_bias_relu", "gemm_rcr_bias_gelu", "gemm_rcr_bias_fast_gelu",
               "gemm_rcr_bias_add", "gemm_rcr_bias_add_add", "bmm_rcr", "bmm_softmax_bmm_permute",
               "bmm_softmax_bmm_permute_causal", "bmm_softmax_bmm"):
        for hook in ("config", "filter", "gen_profiler", "gen_function", "func_decl", "func_call"):
            assert registry.exists(f"rocm.{op}.{hook}"), f"rocm.{op}.{hook}"
    with pytest.raises(RuntimeError):
        registry.reg("rocm.gemm_rcr.config", lambda: None)
    with pytest.raises(RuntimeError):
        registry.get("rocm.nope.config")


def test_target_properties():
    t = detect_target()
    assert t.name() == "rocm" and t.src_extension() == ".cpp" and t.dev_select_flag() == "HIP_VISIBLE_DEVICES"
    assert "{target}" in t.compile_cmd(False) and "{src}" in t.compile_cmd(True)
    names = ["gemm_rcr_f16_256x256x32_w2x2_dma4_o1_p1_m32_c0", "gemm_rcr_f16_64x64x64_w2x2_v8",
             "gemm_rcr_f16_128x128x64_w2x2_v8"]
    assert t.select_minimal_algo(names) == "gemm_rcr_f16_64x64x64_w2x2_v8"
    from aitemplate_amd.backend.rocm.target_def import ROCM

    with pytest.raises(RuntimeError):
        ROCM(arch="gfx90a")
    with t:
        from aitemplate_amd.backend.target import Target

        assert Target.current() is t
    with pytest.raises(RuntimeError):
        Target.current()


# ---- profiling plumbing ----------------------------------------------------------------
def test_profiler_command_line_and_instance_filter(tmp_path, monkeypatch):
    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    Y = _gemm_bias_graph(Ms=(4096,), N=4, K=4)
    op = list(Y.src_ops())[0]
    with detect_target():
        res = op.gen_profiler(str(tmp_path), DynamicProfileStrategy.MAX)
        assert len(res) == 1 and os.access(res[0][1], os.X_OK)
        assert res[0][1] == os.path.join(str(tmp_path), "profiler", "gemm_rcr_bias", op._get_profiler_filename())
        # K = 4 leaves only the instances that load narrower than 16-byte pieces along K
        assert op._attrs["op_instance"] and all("_v8" not in n and ("dma" not in n or "_k2" in n)
                                                for n in op._attrs["op_instance"])
        cmd = op._gen_profile_cmd(os.path.dirname(res[0][1]), op._get_profiler_filename(),
                                  "M == 4096 && N == 4 && K == 4")
        assert cmd[1:] == ["gemm", "gemm_rcr_bias", "0", "4096", "4", "4"]
        op.profile(None, str(tmp_path))
        assert op._attrs["exec_path"]["M == 4096 && N == 4 && K == 4"].algo in op._attrs["op_instance"]
    a = ops.bmm_softmax_bmm_permute(shape=(8,), scale=0.5)
    a(Tensor([16, 64, 40]), Tensor([16, 64, 40]), Tensor([16, 64, 40]))
    with detect_target():
        res = a.gen_profiler(str(tmp_path), DynamicProfileStrategy.MAX)
        key = list(a._attrs["exec_path"])[0]
        cmd = a._gen_profile_cmd(os.path.dirname(res[0][1]), a._get_profiler_filename(), key)
        assert cmd[1:] == ["attn", "bmm_softmax_bmm_permute", "0", "16", "64", "64", "40", "40", "8"]


def test_extract_profile_result():
    out = "noise\nOP:tile_a,TIME:0.25,WS:0\nOP:tile_b,TIME:0.125,WS:102400\n"
    best, failed = extract_profile_result(out)
    assert not failed and best.op_config == "tile_b" and best.duration == 0.125 and best.workspace == 102400
    both, failed = extract_profile_result(out, return_ops=["tile_a", "tile_b", "tile_c"])
    assert [r.op_config for r in both] == ["tile_a", "tile_b"]
    _, failed = extract_profile_result("segfault")
    assert failed


class _Delegate:
    def __init__(self):
        self.results = [None] * 42
        self.post = False

    def add_result(self, idx, val):
        sleep(random() * 0.005)
        self.results[idx] = val

    def postprocess_results(self):
        assert all(v is not None for v in self.results)
        self.post = True


def test_profiler_runner_with_fake_commands():
    delegate = _Delegate()
    pr = ProfilerRunner(devices=[str(i) for i in range(12)], timeout=60, postprocessing_delegate=delegate)
    for i in range(len(delegate.results)):
        pr.push(cmds=["sleep", "0"], process_result_callback=(lambda idx: (lambda result, d: d.add_result(idx, 0)))(i))
    pr.join()
    assert delegate.post


def test_profiler_runner_parses_output_and_picks_fastest(tmp_path):
    from aitemplate_amd.compiler.base import ExecItem
    from aitemplate_amd.compiler.ops.gemm_universal.gemm_common import GemmProfilerPostprocessingDelegate

    fake = tmp_path / "fake_profiler.sh"
    fake.write_text("#!/bin/sh\necho \"device=$HIP_VISIBLE_DEVICES\"\necho OP:tile_a,TIME:0.50,WS:0\necho OP:tile_b,TIME:0.25,WS:0\n"
                    "echo OP:tile_not_listed,TIME:0.01,WS:0\n")
    fake.chmod(fake.stat().st_mode | stat.S_IEXEC)
    attrs = {"op": "gemm_rcr", "exec_path": {"M == 1 && N == 2 && K == 3": ExecItem("k", "c", "")}, "workspace": 0,
             "split_k": 1, "op_instance": {"tile_a": 0, "tile_b": 1}}
    pr = ProfilerRunner(devices=["0"], postprocessing_delegate=GemmProfilerPostprocessingDelegate(), timeout=30)
    pr.push([str(fake)], func_attrs=attrs, profiler_filename="x", exec_key="M == 1 && N == 2 && K == 3", split_k=1)
    pr.join()
    assert attrs["exec_path"]["M == 1 && N == 2 && K == 3"].algo == "tile_b"
    bad = ProfilerRunner(devices=["0"], postprocessing_delegate=GemmProfilerPostprocessingDelegate(), timeout=30)
    bad.push(["false"], func_attrs=attrs, profiler_filename="x", exec_key="M == 1 && N == 2 && K == 3", split_k=1)
    with pytest.raises(RuntimeError, match="Profil"):
        bad.join()


def test_profiler_runner_does_not_rerun_a_killed_or_hung_profiler(tmp_path):
    """A profiler ended by a signal (what a GPU fault does to it) or by the time limit ran once only."""
    from aitemplate_amd.compiler.ops.gemm_universal.gemm_common import GemmProfilerPostprocessingDelegate

    log = tmp_path / "runs.log"
    killed = tmp_path / "killed.sh"
    killed.write_text(f"#!/bin/sh\necho ran >> {log}\nkill -ABRT $$\n")
    killed.chmod(killed.stat().st_mode | stat.S_IEXEC)
    pr = ProfilerRunner(devices=["0"], postprocessing_delegate=GemmProfilerPostprocessingDelegate(), timeout=30)
    pr.push([str(killed)], process_result_callback=None, return_ops=["x"])
    with pytest.raises(RuntimeError, match="killed by signal 6"):
        pr.join()
    assert log.read_text().count("ran") == 1

    log.write_text("")
    hung = tmp_path / "hung.sh"
    hung.write_text(f"#!/bin/sh\necho ran >> {log}\nexec sleep 20\n")
    hung.chmod(hung.stat().st_mode | stat.S_IEXEC)
    pr = ProfilerRunner(devices=["0"], postprocessing_delegate=GemmProfilerPostprocessingDelegate(), timeout=1)
    pr.push([str(hung)], process_result_callback=None, return_ops=["x"])
    with pytest.raises(RuntimeError, match="timed out"):
        pr.join()
    assert log.read_text().count("ran") == 1

    # an ordinary failure (exit status above 0, nothing printed) is still tried again
    log.write_text("")
    flaky = tmp_path / "flaky.sh"
    flaky.write_text(f"#!/bin/sh\necho ran >> {log}\nexit 3\n")
    flaky.chmod(flaky.stat().st_mode | stat.S_IEXEC)
    pr = ProfilerRunner(devices=["0"], postprocessing_delegate=GemmProfilerPostprocessingDelegate(), timeout=30)
    pr.push([str(flaky)], process_result_callback=None, return_ops=["x"])
    with pytest.raises(RuntimeError, match="Profiler failure"):
        pr.join()
    assert log.read_text().count("ran") == 3


# ---- passes and code generation ----------------------------------------------------------------
def test_naming_aliases_and_memory_planning():
    reset_name_counters()
    X = Tensor([8, 16], name="x", is_input=True)
    W1, W2 = Tensor([32, 16], name="w1"), Tensor([24, 32], name="w2")
    h = ops.gemm_rcr()(X, W1)
    y = ops.gemm_rcr()(h, W2)
    y._attrs["is_output"] = True
    y._attrs["name"] = "out"
    graph = transform.toposort(y)
    assert [t._attrs["name"] for t in graph][-1] == "out"
    transform.name_graph(graph)
    transform.mark_param_tensor(graph, [y])
    names = [t._attrs["name"] for t in graph]
    assert "gemm_rcr_0_0" in names and h._attrs["name"] == "gemm_rcr_0_0"
    assert [op._attrs["name"] for op in transform.get_sorted_ops(graph)] == ["gemm_rcr_0", "gemm_rcr_1"]
    assert h._attrs["shape"][0]._attrs["name"] == "x_dim_0"  # dim objects are shared and named once
    assert W1._attrs["is_param"] and not h._attrs["is_param"]
    blob, ws = transform.memory_planning(graph)
    assert h._attrs["offset"] == 0 and blob == 8 * 32 * 2 and ws == 0
    # attention: the op's [B, M, O] tensor lives in the reshaped output's buffer
    a = ops.bmm_softmax_bmm_permute(shape=(2,), scale=1.0)
    o = a(Tensor([4, 8, 16], name="q", is_input=True), Tensor([4, 8, 16], name="k", is_input=True),
          Tensor([4, 8, 16], name="v", is_input=True))
    o._attrs["is_output"] = True
    o._attrs["name"] = "o"
    g2 = transform.toposort(o)
    transform.name_graph(g2)
    transform.mark_param_tensor(g2, [o])
    inner = a._attrs["outputs"][0]
    assert inner._attrs["external_tensor"] is o and inner._attrs["has_output_aliases"]
    assert transform.memory_planning(g2) == (0, 0)


def test_compile_model_builds_a_library_exporting_the_whole_abi(tmp_path, monkeypatch):
    """No GPU here: creating the container fails cleanly, but sources are generated, the
    library links and exports every function include/model_interface.h declares."""
    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    Y = _gemm_bias_graph(Ms=(1, 128), N=64, K=1024, op="gemm_rcr_bias_fast_gelu")
    import torch

    if torch.cuda.is_available():
        compile_model(Y, detect_target(), str(tmp_path), "abi_check").close()
    else:
        with pytest.raises(RuntimeError, match="AITemplateModelContainerCreate"):
            compile_model(Y, detect_target(), str(tmp_path), "abi_check")
    build = tmp_path / "abi_check"
    src = (build / "gemm_rcr_bias_fast_gelu_0.cpp").read_text()
    assert "void gemm_rcr_bias_fast_gelu_0(void* in_ptr, void* weight_ptr, void* out_ptr, void* bias_ptr, " \
           "int64_t* a_dim0, int64_t* a_dim1, int64_t* b_dim0, int64_t* b_dim1, int64_t* c_dim0, int64_t* c_dim1, " \
           "hipStream_t stream)" in src
    assert "if (M >= 1 && M <= 128 && N == 64 && K == 1024)" in src
    assert "aitamd_gemm_rcr(3, 0, algo" in src and "Unsupported workload" in src
    model_src = (build / "model-generated.cpp").read_text()
    assert "ParamDim(1, 128, &m)" in model_src and 'OpEntry{"gemm_rcr_bias_fast_gelu_0"' in model_src
    header = open(os.path.join(ROOT, "include", "model_interface.h")).read()
    declared = sorted(set(re.findall(r"AIT_EXPORT AITemplateError\s+(AITemplate\w+)\s*\(", header)))
    assert len(declared) == 32, declared
    out = subprocess.run(["nm", "-D", "--defined-only", str(build / "test.so")], capture_output=True, text=True).stdout
    exported = sorted(set(re.findall(r" T (AITemplate\w+)", out)))
    assert exported == declared
    # nothing else leaks out of the model library except the C ABI
    others = [l.split()[-1] for l in out.splitlines() if " T " in l and "AITemplate" not in l]
    assert not [s for s in others if not s.startswith("_")], others


# ---- profiling-result cache -------------------------------------------------------------------
def test_profile_cache_db_roundtrip(tmp_path):
    from aitemplate_amd.backend.profiler_cache import ProfileCacheDB, exec_entry_sha1

    db = ProfileCacheDB("rocm", path=str(tmp_path / "rocm.db"))
    key = {"op_type": "gemm_rcr_bias", "dtype": "float16", "device": "rocm-gfx950", "instances_sha1": "abc",
           "exec_entry": "M == 256 && N == 1024 && K == 1024",
           "exec_entry_sha1": exec_entry_sha1("M == 256 && N == 1024 && K == 1024")}
    assert db.query_gemm(key) is None
    db.insert_gemm(dict(key, algo="tile_b", workspace=0, split_k=1, duration=0.25))
    assert db.query_gemm(key) == ("tile_b", 0, 1)
    db.insert_gemm(dict(key, algo="tile_c", workspace=0, split_k=1, duration=0.1))  # first writer wins
    assert db.query_gemm(key) == ("tile_b", 0, 1) and db.num_entries() == 1
    # any key component that differs is a miss: other instance list, other device, other workload
    assert db.query_gemm(dict(key, instances_sha1="other")) is None
    assert db.query_gemm(dict(key, device="rocm-gfx942")) is None
    assert db.query_gemm(dict(key, exec_entry_sha1=exec_entry_sha1("M == 1 && N == 2 && K == 3"))) is None
    with pytest.raises(KeyError):
        db.query_gemm({"op_type": "gemm_rcr"})
    db.close()
    # persisted on disk
    db2 = ProfileCacheDB("rocm", path=str(tmp_path / "rocm.db"))
    assert db2.query_gemm(key) == ("tile_b", 0, 1)
    db2.close()


def test_profile_results_are_cached_and_reused(tmp_path, monkeypatch):
    """Second profile() of the same workload takes the winner from the cache and runs no profiler
    (reference flow: gemm_common.py:618-676); FORCE_PROFILE=1 times again; CI mode has no cache."""
    from aitemplate_amd.compiler.ops.gemm_universal.gemm_common import GemmProfilerPostprocessingDelegate

    monkeypatch.delenv("CI_FLAG", raising=False)
    monkeypatch.setenv("CACHE_DIR", str(tmp_path / "cache"))
    fake = tmp_path / "fake_profiler.sh"

    def build_op():
        op = list(_gemm_bias_graph(Ms=(4096,), N=64, K=64).src_ops())[0]
        op.gen_profiler(str(tmp_path), DynamicProfileStrategy.MAX)
        exe = os.path.join(str(tmp_path), "profiler", "gemm_rcr_bias", op._get_profiler_filename())
        names = list(op._attrs["op_instance"])
        os.remove(exe)
        fake.write_text("#!/bin/sh\necho ran >> %s\n" % (tmp_path / "runs.log")
                        + "".join(f"echo OP:{n},TIME:{1.0 + i},WS:0\n" for i, n in enumerate(names[:-1]))
                        + f"echo OP:{names[-1]},TIME:0.5,WS:0\n")
        fake.chmod(fake.stat().st_mode | stat.S_IEXEC)
        os.symlink(str(fake), exe)
        return op, names

    def profile(op):
        pr = ProfilerRunner(devices=["0"], postprocessing_delegate=GemmProfilerPostprocessingDelegate(), timeout=30)
        op.profile(pr, str(tmp_path))
        pr.join()

    with detect_target() as target:
        assert target.get_profile_cache_path() == str(tmp_path / "cache" / "rocm.db")
        op, names = build_op()
        profile(op)
        key = list(op._attrs["exec_path"])[0]
        assert op._attrs["exec_path"][key].algo == names[-1]
        assert (tmp_path / "runs.log").read_text().count("ran") == 1
    with detect_target():
        op2, _ = build_op()
        profile(op2)
        assert op2._attrs["exec_path"][key].algo == names[-1]
        assert (tmp_path / "runs.log").read_text().count("ran") == 1  # served from the cache
        monkeypatch.setenv("FORCE_PROFILE", "1")
        op3, _ = build_op()
        profile(op3)
        assert (tmp_path / "runs.log").read_text().count("ran") == 2
        monkeypatch.delenv("FORCE_PROFILE")
    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    with detect_target() as target:
        assert target.get_profile_cache_path() is None


# ---- permuting GEMMs, split, nn.MultiheadAttention ------------------------------------------
def test_permuting_gemm_ops_shapes_names_and_copies():
    """Shapes as in tests/unittest/ops/test_gemm_bias_permute.py:34-75 (m2n3), :100-140 (m3n2) and
    test_gemm_permute.py of the reference."""
    X = Tensor([4 * 256, 256], name="x", is_input=True)
    W = Tensor([4 * 16 * 128, 256], name="w", is_input=True)
    Bv = Tensor([4 * 16 * 128], name="b", is_input=True)
    op = ops.gemm_rcr_bias_permute((256, 4, 16), layout="m2n3")
    y = op(X, W, Bv)
    assert op._attrs["op"] == "gemm_rcr_bias_permute_m2n3" and op._attrs["layout"] == "Permute5D_m2n3"
    assert [d.value() for d in y.shape()] == [4, 4, 16, 256, 128]  # [N0, M0, N1, M1, N2]
    assert [d.value() for d in op._attrs["outputs"][0].shape()] == [1024, 8192]
    assert op._attrs["permute_shape"] == "256_4_16" and op._attrs["epilogue_alignment"] == 8
    clone = ops.gemm_rcr_bias_permute(**op._get_op_attributes())
    assert clone._attrs["op"] == op._attrs["op"] and clone._attrs["shape"] == (256, 4, 16)

    X3 = Tensor([4 * 16 * 32, 256], name="x3", is_input=True)
    W3 = Tensor([8 * 128, 256], name="w3", is_input=True)
    B3 = Tensor([8 * 128], name="b3", is_input=True)
    for layout, name in (("m3n2", "gemm_rcr_bias_permute_m3n2"), ("20314", "gemm_rcr_bias_permute")):
        op3 = ops.gemm_rcr_bias_permute((16, 32, 8), layout=layout)
        y3 = op3(X3, W3, B3)
        assert op3._attrs["op"] == name
        assert [d.value() for d in y3.shape()] == [32, 4, 8, 16, 128]  # [M2, M0, N0, M1, N1]

    op2 = ops.gemm_rcr_permute((256, 4, 16), layout="m2n3")
    y2 = op2(X, W)
    assert op2._attrs["op"] == "gemm_rcr_permute_m2n3"
    assert [d.value() for d in y2.shape()] == [4, 4, 16, 256, 128]
    with pytest.raises(NotImplementedError):
        ops.gemm_rcr_permute((2, 2), layout="0213")  # CUDA-only layout of the reference
    with pytest.raises(NotImplementedError):
        ops.gemm_rcr_bias_permute((1, 2, 3), layout="nope")
    with pytest.raises(RuntimeError, match="does not split"):
        ops.gemm_rcr_bias_permute((100, 4, 16), layout="m2n3")(X, W, Bv)
    # a 3-D A folds its leading dims into M
    y4 = ops.gemm_rcr_permute((64, 3, 2), layout="m2n3")(Tensor([5, 64, 32], name="x4", is_input=True),
                                                        Tensor([96, 32], name="w4", is_input=True))
    assert [d.value() for d in y4.shape()] == [3, 5, 2, 64, 16]
    detect_target()
    for name in ("gemm_rcr_permute_m2n3", "gemm_rcr_bias_permute", "gemm_rcr_bias_permute_m2n3",
                 "gemm_rcr_bias_permute_m3n2"):
        for hook in ("config", "filter", "gen_profiler", "select_algo", "gen_function", "func_decl", "func_call"):
            assert registry.exists(f"rocm.{name}.{hook}")


def test_bmm_rcr_permute_op_attrs():
    op = ops.bmm_rcr_permute(shape=(12,))
    y = op(Tensor([24, 80, 88], name="q", is_input=True), Tensor([24, 64, 88], name="k", is_input=True))
    assert [d.value() for d in y.shape()] == [2, 80, 12, 64]
    assert [d.value() for d in op._attrs["outputs"][0].shape()] == [24, 80, 64]
    assert op._attrs["op"] == "bmm_rcr_permute" and op._attrs["permute_shape"] == "12"
    assert ops.bmm_rcr_permute(**op._get_op_attributes())._attrs["shape"] == (12,)
    with pytest.raises(NotImplementedError):
        ops.bmm_rcr_permute(shape=(2,), layout="0321")(Tensor([4, 8, 8], name="a", is_input=True),
                                                      Tensor([4, 8, 8], name="b", is_input=True))
    with pytest.raises(RuntimeError, match="multiple"):
        ops.bmm_rcr_permute(shape=(5,))(Tensor([24, 8, 8], name="a2", is_input=True),
                                        Tensor([24, 8, 8], name="b2", is_input=True))
    detect_target()
    for hook in ("config", "filter", "gen_profiler", "select_algo", "gen_function", "func_decl", "func_call"):
        assert registry.exists(f"rocm.bmm_rcr_permute.{hook}")


def test_bmm_layout_ops_shapes_keys_and_hooks():
    """Operand shapes of bmm_xxx.py:204-260 and the reference's exec keys (B, M, N, K order)."""
    B, M, N, K = 6, 40, 24, 16
    cases = {"bmm_rrr": ([B, M, K], [B, K, N]), "bmm_ccr": ([B, K, M], [B, N, K]), "bmm_crr": ([B, K, M], [B, K, N])}
    detect_target()
    for name, (a_shape, b_shape) in cases.items():
        op = getattr(ops, name)()
        y = op(Tensor(a_shape, name="a", is_input=True), Tensor(b_shape, name="b", is_input=True))
        assert [d.value() for d in y.shape()] == [B, M, N] and op._attrs["op"] == name
        op._extract_exec_path(DynamicProfileStrategy.MAX)
        assert list(op._attrs["exec_path"]) == [f"B == {B} && M == {M} && N == {N} && K == {K}"]
        for hook in ("config", "filter", "gen_profiler", "select_algo", "gen_function", "func_decl", "func_call"):
            assert registry.exists(f"rocm.{name}.{hook}")
    with pytest.raises(RuntimeError, match="same K"):
        ops.bmm_rrr()(Tensor([2, 8, 16], name="a", is_input=True), Tensor([2, 8, 16], name="b", is_input=True))
    g = ops.gemm_rrr()
    y = g(Tensor([5, 7, 16], name="a3", is_input=True), Tensor([16, 24], name="b2", is_input=True))
    assert [d.value() for d in y.shape()] == [5, 7, 24]
    g._extract_exec_path(DynamicProfileStrategy.MAX)
    assert list(g._attrs["exec_path"]) == ["M == 35 && N == 24 && K == 16"]
    X, W, D = Tensor([B, M, K], name="x", is_input=True), Tensor([B, K, N], name="w", is_input=True), \
        Tensor([B, M, N], name="d", is_input=True)
    fused = ops.bmm_rrr()(X, W) + D
    fused._attrs["is_output"] = True
    graph, _ = _fuse([fused])
    assert _op_names(graph) == ["bmm_rrr_add"]
    with pytest.raises(RuntimeError, match="doesn't match"):
        ops.bmm_ccr_add()(Tensor([B, K, M], name="xa", is_input=True), Tensor([B, N, K], name="wa", is_input=True),
                          Tensor([B, M, N + 8], name="da", is_input=True))
    rp = ops.gemm_rrr_bias_permute((2, 4, 3))
    yr = rp(Tensor([16, 8], name="rx", is_input=True), Tensor([8, 24], name="rw", is_input=True),
            Tensor([24], name="rb", is_input=True))
    assert [d.value() for d in yr.shape()] == [4, 2, 3, 2, 8] and rp._attrs["op"] == "gemm_rrr_bias_permute"
    for name in ("bmm_rrr_add", "bmm_ccr_add", "bmm_crr_add", "gemm_rrr", "gemm_rrr_bias_permute", "bmm_rrr_permute"):
        for hook in ("config", "filter", "gen_profiler", "select_algo", "gen_function", "func_decl", "func_call"):
            assert registry.exists(f"rocm.{name}.{hook}"), f"rocm.{name}.{hook}"
    p = ops.bmm_rrr_permute(shape=(3,))
    yp = p(Tensor([B, M, K], name="pa", is_input=True), Tensor([B, K, N], name="pb", is_input=True))
    assert [d.value() for d in yp.shape()] == [2, M, 3, N] and p._attrs["op"] == "bmm_rrr_permute"
    assert ops.bmm_rrr_permute(**p._get_op_attributes())._attrs["shape"] == (3,)


def test_split_is_a_view_with_byte_offsets():
    x = Tensor([3, 2, 4, 8, 16], name="x", is_input=True)
    q, k, v = ops.split()(x, 1, dim=0)
    assert [d.value() for d in k.shape()] == [1, 2, 4, 8, 16]
    piece = 2 * 4 * 8 * 16 * 2
    assert [t._attrs["view_offset_bytes"] for t in (q, k, v)] == [0, piece, 2 * piece]
    a, b = ops.split()(Tensor([1, 10, 4], name="z", is_input=True), [3, 7], dim=1)
    assert [d.value() for d in b.shape()] == [1, 7, 4] and b._attrs["view_offset_bytes"] == 3 * 4 * 2
    parts = ops.split()(Tensor([10, 4], name="u", is_input=True), 4)  # torch semantics: 4, 4, 2
    assert [p.shape()[0].value() for p in parts] == [4, 4, 2]
    # a split along a middle dim makes strided pieces (the strided-view pass gives each a row copy)
    m0, m1 = ops.split()(Tensor([2, 10, 4], name="w", is_input=True), 5, dim=1)
    assert m1._attrs["strided_view_of"][1:] == (1, 5) and [d.value() for d in m1.shape()] == [2, 5, 4]
    with pytest.raises(RuntimeError, match="does not match"):
        ops.split()(Tensor([10, 4], name="t", is_input=True), [3, 3], dim=0)
    # offsets accumulate through views of views and reach the generated bindings
    from aitemplate_amd.compiler.transform.mark_param_tensor import storage_offset_bytes

    k2 = ops.reshape()(k, [-1, 8, 16])
    assert storage_offset_bytes(k2) == piece


def _strided_view_graph(Ms=(48,), K0=96, K1=64, N=40):
    """Two GEMMs between a last-dim split of the activations and of the residuals, and a concatenate."""
    m = shape_utils.gen_int_var_min_max(list(Ms), name="m")
    X = Tensor([m, IntImm(K0 + K1)], name="x", is_input=True)
    R = Tensor([m, IntImm(2 * N)], name="r", is_input=True)
    W0, B0 = Tensor([N, K0], name="w0", is_input=True), Tensor([N], name="b0", is_input=True)
    W1, B1 = Tensor([N, K1], name="w1", is_input=True), Tensor([N], name="b1", is_input=True)
    xa, xb = ops.split()(X, [K0, K1], dim=-1)
    r0, r1 = ops.split()(R, N, dim=1)
    y0 = ops.gemm_rcr_bias_add()(xa, W0, B0, r0)
    y1 = ops.gemm_rcr_bias_add()(xb, W1, B1, r1)
    Y = ops.concatenate()([y0, y1], dim=-1)
    Y._attrs["name"] = "y"
    Y._attrs["is_output"] = True
    return Y, (xa, xb, r0, r1, y0, y1)


def test_last_dim_split_and_concatenate_become_offsets_and_pitches(tmp_path, monkeypatch):
    """The rewrites of the reference's transform_strided_ops.py:33-64 on the GEMM family: pieces of a last-dim split
    are read, and inputs of a last-dim concatenate are written, through TensorAccessor.update_base_tensor."""
    K0, K1, N = 96, 64, 40
    Y, (xa, xb, r0, r1, y0, y1) = _strided_view_graph(K0=K0, K1=K1, N=N)
    assert xb._attrs["strided_view_of"][1:] == (1, K0) and "view_offset_bytes" not in xb._attrs
    graph = transform.toposort(Y)
    assert {op._attrs["op"] for op in transform.get_sorted_ops(graph)} == {"split", "gemm_rcr_bias_add", "concatenate"}
    graph = transform.fuse_strided_views(graph, [Y])
    sorted_ops = transform.get_sorted_ops(graph)
    assert [op._attrs["op"] for op in sorted_ops] == ["gemm_rcr_bias_add"] * 2
    assert all(t not in graph for t in (xa, xb, r0, r1, y0, y1))
    g0, g1 = sorted_ops
    assert [t._attrs["name"] for t in g1._attrs["inputs"]] == ["x", "w1", "b1", "r"] and g1._attrs["outputs"] == [Y]
    a, _, _, d = g1._attrs["input_accessors"]
    c = g1._attrs["output_accessors"][0]
    assert (a.offset, a.row_pitch(), a.is_contiguous) == (K0, K0 + K1, False)
    assert [x.value() for x in a.original_shapes[1:]] == [K1]
    assert (d.offset, d.row_pitch()) == (N, 2 * N) and (c.offset, c.row_pitch()) == (N, 2 * N)
    assert g0._attrs["input_accessors"][0].offset == 0 and g0._attrs["output_accessors"][0].row_pitch() == 2 * N
    assert list(Y.src_ops()) == [g0, g1]
    # the problem sizes still come from the views' own shapes
    g1._extract_exec_path(DynamicProfileStrategy.MAX)
    assert list(g1._attrs["exec_path"]) == [f"M == 48 && N == {N} && K == {K1}"]

    # through compile_model: generated launch code and the dim members of the vanished views
    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    reset_name_counters()
    Y, _ = _strided_view_graph(Ms=(16, 48), K0=K0, K1=K1, N=N)
    import torch

    if torch.cuda.is_available():
        compile_model(Y, detect_target(), str(tmp_path), "strided").close()
    else:
        with pytest.raises(RuntimeError, match="AITemplateModelContainerCreate"):
            compile_model(Y, detect_target(), str(tmp_path), "strided")
    build = tmp_path / "strided"
    model_src = (build / "model-generated.cpp").read_text()
    entries = re.findall(r'OpEntry\{"(\w+)"', model_src)
    assert len(entries) == 2
    srcs = [(build / f"{e}.cpp").read_text() for e in entries]
    assert f"static_cast<const uint16_t*>(in_ptr) + {K0};" in srcs[1] and f"const int64_t lda = {K0 + K1};" in srcs[1]
    assert f"static_cast<uint16_t*>(out_ptr) + {N};" in srcs[1] and f"const int64_t ldc = {2 * N};" in srcs[1]
    assert f"const uint16_t* d0 = static_cast<const uint16_t*>(d0_ptr) + {N};" in srcs[1]
    assert f"const int64_t ldd = {2 * N};" in srcs[1] and "bias_ptr, d0, nullptr, c, M, N, K" in srcs[1]
    assert "static_cast<const uint16_t*>(in_ptr) + 0;" in srcs[0] and f"const int64_t lda = {K0 + K1};" in srcs[0]
    # both ops are handed x, r and y; the views' static dims are members of the model
    assert model_src.count("(x, w") == 2 and model_src.count(", y, b") == 2
    for e in entries:
        assert re.search(rf"int64_t {e}_input0_dim_1 \{{({K0}|{K1})\}};", model_src), e
        assert f"&m, &{e}_input0_dim_1" in model_src


def _ops_of(graph):
    from aitemplate_amd.compiler.transform.transform_utils import get_sorted_ops

    return [op for op in get_sorted_ops(graph) if not op._attrs.get("is_view_op")]


def test_strided_views_that_no_gemm_can_take_become_row_copies():
    from aitemplate_amd.compiler.ops.common.view_ops import copy_geometry

    N, K = 16, 32
    X = Tensor([8, 2 * K], name="x", is_input=True)
    B = Tensor([N], name="b", is_input=True)
    # a piece read by an op without accessors: a copy of 8 rows of K elements out of rows 2 K apart
    xa, xb = ops.split()(X, K, dim=1)
    out = ops.reshape()(xb, [4, -1])
    out._attrs["is_output"] = True
    g = transform.fuse_strided_views(transform.toposort(out), [out])
    (cp,) = _ops_of(g)
    assert cp._attrs["op"] == "strided_copy" and cp._attrs["copy_kind"] == "slice"
    assert cp._attrs["inputs"] == [X] and cp._attrs["outputs"] == [xb]
    assert xb._attrs["is_view_of"] is None and xb._attrs["strided_view_of"] is None
    assert copy_geometry(cp._attrs)[2:] == (K * 2, 2 * K * 2, K * 2)
    # a piece that is a graph output
    xa, xb = ops.split()(X, K, dim=1)
    xa._attrs["is_output"] = True
    (cp,) = _ops_of(transform.fuse_strided_views(transform.toposort(xa), [xa]))
    assert cp._attrs["op"] == "strided_copy" and cp._attrs["copy_start"] == 0 and cp._attrs["outputs"] == [xa]
    # a bias cannot be a view
    b0, b1 = ops.split()(Tensor([1, 2 * N], name="b2", is_input=True), N, dim=1)
    # (dims of size 1 in front: this is the contiguous kind of split, not a strided view)
    assert "strided_view_of" not in b1._attrs
    # concatenate of a GEMM output and a graph input: the GEMM writes its columns, the input is copied into its
    Z = Tensor([8, N], name="z", is_input=True)
    y = ops.gemm_rcr_bias()(X, Tensor([N, 2 * K], name="w2", is_input=True), B)
    cat = ops.concatenate()([y, Z], dim=1)
    cat._attrs["is_output"] = True
    kinds = sorted(op._attrs["op"] for op in _ops_of(transform.fuse_strided_views(transform.toposort(cat), [cat])))
    assert kinds == ["gemm_rcr_bias", "strided_copy"]
    (cp,) = [op for op in cat.src_ops() if op._attrs["op"] == "strided_copy"]
    assert cp._attrs["copy_kind"] == "place" and cp._attrs["inputs"] == [Z] and cp._attrs["copy_start"] == N
    assert copy_geometry(cp._attrs)[2:] == (N * 2, 2 * N * 2, N * 2)
    # a tensor with a second consumer keeps its own buffer and is copied
    y = ops.gemm_rcr_bias()(X, Tensor([N, 2 * K], name="w3", is_input=True), B)
    y2 = ops.gemm_rcr_bias()(y, Tensor([N, N], name="w4", is_input=True), B)
    cat = ops.concatenate()([y, y2], dim=-1)
    cat._attrs["is_output"] = True
    g = transform.fuse_strided_views(transform.toposort(cat), [cat])
    assert sorted(op._attrs["op"] for op in _ops_of(g)) == ["gemm_rcr_bias", "gemm_rcr_bias", "strided_copy"]
    assert y._attrs["src_ops"] and [op._attrs["op"] for op in y.src_ops()] == ["gemm_rcr_bias"]
    # along another dim every input is copied: rows = 1, the whole tensor one row
    y = ops.gemm_rcr_bias()(X, Tensor([N, 2 * K], name="w5", is_input=True), B)
    cat = ops.concatenate()([y, Z], dim=0)
    cat._attrs["is_output"] = True
    g = transform.fuse_strided_views(transform.toposort(cat), [cat])
    copies = [op for op in _ops_of(g) if op._attrs["op"] == "strided_copy"]
    assert len(copies) == 2 and sorted(c._attrs["copy_start"] for c in copies) == [0, 8]
    assert copy_geometry(copies[0]._attrs)[2:4] == (8 * N * 2, 16 * N * 2)
    with pytest.raises(RuntimeError, match="dim 0 differs"):
        ops.concatenate()([y, Tensor([9, N], name="z2", is_input=True)], dim=1)


def test_two_residuals_are_views_only_when_they_share_one_row_pitch(tmp_path, monkeypatch):
    """The generated launch has one `ldd` for both residuals: a piece of a last-dim split may be read in place as a
    residual only when the op's other residual ends up with the same row pitch; otherwise it is copied, as the
    reference does for every split it cannot fuse."""
    M, N, K = 8, 16, 32

    def graph(d0_of, d1_of):
        X = Tensor([M, K], name="x", is_input=True)
        W = Tensor([N, K], name="w", is_input=True)
        B = Tensor([N], name="b", is_input=True)
        y = ops.gemm_rcr_bias_add_add()(X, W, B, d0_of(), d1_of())
        y._attrs["name"], y._attrs["is_output"] = "y", True
        return y

    def piece_of(name, width, index=1):
        def make():
            return ops.split()(Tensor([M, width], name=name, is_input=True), N, dim=1)[index]
        return make

    def plain(name):
        return lambda: Tensor([M, N], name=name, is_input=True)

    def run(y):
        g = transform.fuse_strided_views(transform.toposort(y), [y])
        kinds = sorted(op._attrs["op"] for op in _ops_of(g))
        (gemm,) = [op for op in _ops_of(g) if op._attrs["op"] == "gemm_rcr_bias_add_add"]
        return kinds, [gemm._attrs["input_accessors"][i].row_pitch() for i in (3, 4)]

    # a piece and a plain tensor: pitches 2N and N, so the piece is copied
    kinds, pitches = run(graph(piece_of("r", 2 * N), plain("p")))
    assert kinds == ["gemm_rcr_bias_add_add", "strided_copy"] and pitches == [N, N]
    kinds, pitches = run(graph(plain("p"), piece_of("r", 2 * N)))
    assert kinds == ["gemm_rcr_bias_add_add", "strided_copy"] and pitches == [N, N]
    # pieces of splits of different widths: both copied
    kinds, pitches = run(graph(piece_of("r", 2 * N), piece_of("q", 3 * N)))
    assert kinds == ["gemm_rcr_bias_add_add", "strided_copy", "strided_copy"] and pitches == [N, N]
    # pieces of splits of the same width (or of one split): both stay views
    kinds, pitches = run(graph(piece_of("r", 2 * N), piece_of("q", 2 * N, index=0)))
    assert kinds == ["gemm_rcr_bias_add_add"] and pitches == [2 * N, 2 * N]
    # the partner has to be copied for a reason of its own (it is a graph output too): then so is the piece
    X = Tensor([M, K], name="x", is_input=True)
    q0, q1 = ops.split()(Tensor([M, 2 * N], name="q", is_input=True), N, dim=1)
    r1 = ops.split()(Tensor([M, 2 * N], name="r", is_input=True), N, dim=1)[1]
    y = ops.gemm_rcr_bias_add_add()(X, Tensor([N, K], name="w", is_input=True), Tensor([N], name="b", is_input=True), r1, q1)
    y._attrs["name"], y._attrs["is_output"] = "y", True
    q1._attrs["is_output"] = True
    g = transform.fuse_strided_views(transform.toposort([y, q1]), [y, q1])
    assert sorted(op._attrs["op"] for op in _ops_of(g)) == ["gemm_rcr_bias_add_add", "strided_copy", "strided_copy"]

    # the mixed case compiles (it raised NotImplementedError in the code generator before)
    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    reset_name_counters()
    y = graph(piece_of("r", 2 * N), plain("p"))
    import torch

    if torch.cuda.is_available():
        compile_model(y, detect_target(), str(tmp_path), "mixed_residuals").close()
    else:
        with pytest.raises(RuntimeError, match="AITemplateModelContainerCreate"):
            compile_model(y, detect_target(), str(tmp_path), "mixed_residuals")
    assert f"const int64_t ldd = N;" in "".join(
        f.read_text() for f in (tmp_path / "mixed_residuals").glob("gemm_rcr_bias_add_add*.cpp"))


def test_row_copy_codegen_for_a_middle_dim_split(tmp_path, monkeypatch):
    """[batch, 10, 4] split along dim 1 into 3 + 7: two generated functions with literal geometry, called with the
    dynamic batch as the number of rows."""
    from aitemplate_amd.backend import codegen
    from aitemplate_amd.compiler.base import IntVar
    from aitemplate_amd.testing import detect_target

    batch = IntVar([1, 8], name="batch")
    X = Tensor([batch, 10, 4], name="x", is_input=True)
    a, b = ops.split()(X, [3, 7], dim=1)
    a._attrs["name"], a._attrs["is_output"] = "out_a", True
    b._attrs["name"], b._attrs["is_output"] = "out_b", True
    with detect_target():
        g = transform.fuse_strided_views(transform.toposort([a, b]), [a, b])
        transform.name_graph(g)
        transform.mark_param_tensor(g, [a, b])
        pairs = codegen.gen_function_src(g, str(tmp_path), "m")
    srcs = sorted(open(src).read() for src, _ in pairs)
    assert len(srcs) == 2
    assert "aitamd_copy_rows(static_cast<const char*>(src) + 0, dst, rows, 24, 80, 24, stream)" in srcs[0]
    assert "aitamd_copy_rows(static_cast<const char*>(src) + 24, dst, rows, 56, 80, 56, stream)" in srcs[1]


def test_multihead_attention_block_compiles_to_three_kernels(tmp_path, monkeypatch):
    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    reset_name_counters()
    B, S, D, H = 2, 64, 128, 4
    x = Tensor([B, S, D], name="x", is_input=True)
    res = Tensor([B * S, D], name="res", is_input=True)  # same shape as the projection, as the reference requires
    mha = nn.MultiheadAttention(D, B, S, H, qkv_bias=True)
    mha.name_parameter_tensor()
    y = mha(x, res)
    y._attrs["is_output"] = True
    y._attrs["name"] = "y"
    assert [d.value() for d in y.shape()] == [B, S, D]
    import torch

    if torch.cuda.is_available():
        compile_model(y, detect_target(), str(tmp_path), "mha").close()
    else:
        with pytest.raises(RuntimeError, match="AITemplateModelContainerCreate"):
            compile_model(y, detect_target(), str(tmp_path), "mha")
    build = tmp_path / "mha"
    model_src = (build / "model-generated.cpp").read_text()
    entries = re.findall(r'OpEntry\{"(\w+)"', model_src)
    assert entries == ["gemm_rcr_bias_permute_m2n3_0", "bmm_softmax_bmm_permute_3", "gemm_rcr_bias_add_6"] or \
        [e.rsplit("_", 1)[0] for e in entries] == ["gemm_rcr_bias_permute_m2n3", "bmm_softmax_bmm_permute",
                                                   "gemm_rcr_bias_add"], entries
    qkv_src = (build / f"{entries[0]}.cpp").read_text()
    assert "const int p_dim0, const int p_dim1, const int p_dim2, hipStream_t stream)" in qkv_src
    assert "aitamd_gemm_permute(0, 1, 0, algo, a, b, bias_ptr, out_ptr, M, N, K, lda, ldb, 1, p_dim0, p_dim1, " \
           "p_dim2, stream)" in qkv_src
    assert f", {S}, 3, {H}, stream);" in model_src
    # K and V are the second and third [B, heads, S, head_dim] pieces of the packed projection
    piece = B * S * D * 2
    assert f"+ ({piece});" in model_src and f"+ ({2 * piece});" in model_src
    with pytest.raises(NotImplementedError):
        nn.MultiheadAttention(D, B, S, H, mask_seq=4)


def test_mem_eff_attention_op_shapes_keys_and_hooks():
    """Operator attributes, output shape and exec keys as python/aitemplate/compiler/ops/attention/
    mem_eff_attention.py:49-263 gives them; variable sequence lengths are refused, not approximated."""
    import aitemplate_amd.backend.rocm  # noqa: F401  registers the hooks

    q = Tensor([2, 8, 64, 40], name="q", is_input=True)
    k = Tensor([2, 8, 77, 40], name="k", is_input=True)
    v = Tensor([2, 8, 77, 48], name="v", is_input=True)
    op = ops.mem_eff_attention(causal=False)
    y = op(q, k, v)
    assert [d.value() for d in y.shape()] == [2, 64, 8, 48]
    assert op._get_op_attributes() == {"causal": False, "variable_seq_length_kv": False,
                                       "variable_seq_length_q": False, "use_grouped_fmha": False}
    assert op._attrs["head_size"] == 48 and op._attrs["workspace"] == 0
    assert list(op._attrs["exec_path"]) == ["batch_size == 2 && num_heads == 8 && seq_len == 64 && head_sizes == 40"]
    op._attrs["name"] = "mem_eff_attention_0"
    for t in (q, k, v):
        for i, d in enumerate(t._attrs["shape"]):
            d._attrs["name"] = f"{t._attrs['name']}_dim_{i}"
    y._attrs["name"] = "y"
    decl = registry.get("rocm.mem_eff_attention.func_decl")(op._attrs)
    assert decl.startswith("void mem_eff_attention_0(void* output, const void* q, const void* k, const void* v, "
                           "const void* lengths_kv, const void* lengths_q, int64_t* batch_size, int64_t* seq_len, "
                           "int64_t* seq_len_kv, int num_heads, ")
    call = registry.get("rocm.mem_eff_attention.func_call")(op._attrs)
    assert call == (f"  mem_eff_attention_0(y, q, k, v, nullptr, nullptr, &q_dim_0, &q_dim_2, &k_dim_2, 8, 40, 48, "
                    f"{40 ** -0.5!r}f, stream);")
    causal_op = ops.mem_eff_attention(causal=True)
    causal_op(q, k, v)
    causal_op._attrs["name"] = "mem_eff_attention_1"
    with detect_target():
        src = op.gen_function()
        causal_src = causal_op.gen_function()
    assert ("aitamd_mem_eff_attention(0, q, k, v, output, *batch_size, num_heads, *seq_len, *seq_len_kv, head_dim,"
            in src)
    assert "head_dim_v, softmax_scale, 0," in src and "head_dim_v, softmax_scale, 1," in causal_src
    # key lengths: a fourth (and, for query lengths, fifth) input of dtype "int"
    var = ops.mem_eff_attention(causal=False, variable_seq_length_kv=True, variable_seq_length_q=True)
    lens_kv = Tensor([2, 1], name="lens_kv", dtype="int", is_input=True)
    lens_q = Tensor([2, 1], name="lens_q", dtype="int", is_input=True)
    y2 = var(q, k, v, lens_kv, lens_q)
    assert [t._attrs["name"] for t in var._attrs["inputs"]] == ["q", "k", "v", "lens_kv", "lens_q"]
    assert lens_kv._attrs["dtype"] == "int32"
    var._attrs["name"] = "mem_eff_attention_2"
    y2._attrs["name"] = "y2"
    assert registry.get("rocm.mem_eff_attention.func_call")(var._attrs).startswith(
        "  mem_eff_attention_2(y2, q, k, v, lens_kv, lens_q, &q_dim_0,")
    only_q = ops.mem_eff_attention(causal=False, variable_seq_length_q=True)
    y3 = only_q(q, k, v, None, lens_q)
    only_q._attrs["name"], y3._attrs["name"] = "mem_eff_attention_3", "y3"
    assert registry.get("rocm.mem_eff_attention.func_call")(only_q._attrs).startswith(
        "  mem_eff_attention_3(y3, q, k, v, nullptr, lens_q, &q_dim_0,")
    copy = ops.mem_eff_attention(**var._get_op_attributes())
    assert copy._attrs["variable_seq_length_kv"] and copy._attrs["variable_seq_length_q"]
    with pytest.raises(AssertionError):
        ops.mem_eff_attention(causal=False, variable_seq_length_kv=True)(q, k, v)
    with pytest.raises(RuntimeError, match="one entry per batch"):
        ops.mem_eff_attention(causal=False, variable_seq_length_kv=True)(
            q, k, v, Tensor([3, 1], name="bad_len", dtype="int", is_input=True))
    with pytest.raises(RuntimeError, match="batch and heads"):
        ops.mem_eff_attention(causal=False)(q, Tensor([2, 4, 77, 40], name="k4", is_input=True), v)
    with pytest.raises(RuntimeError, match="int32"):
        ops.mem_eff_attention(causal=False, variable_seq_length_kv=True)(
            q, k, v, Tensor([2, 1], name="bad", dtype="float16", is_input=True))
    with pytest.raises(RuntimeError, match="head dims"):
        ops.mem_eff_attention(causal=False)(q, Tensor([2, 8, 77, 32], name="k2", is_input=True), v)


def test_cross_attention_block_compiles_to_five_kernels(tmp_path, monkeypatch):
    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    reset_name_counters()
    B, S, Skv, D, H = 2, 64, 77, 128, 4
    q = Tensor([B, S, D], name="q", is_input=True)
    k = Tensor([B, Skv, D], name="k", is_input=True)
    v = Tensor([B, Skv, D], name="v", is_input=True)
    res = Tensor([B * S, D], name="res", is_input=True)
    att = nn.CrossAttention(D, S, Skv, H)
    att.name_parameter_tensor()
    assert [n for n, _ in att.named_parameters()] == ["proj_q.weight", "proj_k.weight", "proj_v.weight",
                                                      "proj.weight", "proj.bias"]
    y = att(q, k, v, res)
    y._attrs["is_output"] = True
    y._attrs["name"] = "y"
    assert [d.value() for d in y.shape()] == [B, S, D]
    import torch

    if torch.cuda.is_available():
        compile_model(y, detect_target(), str(tmp_path), "cross").close()
    else:
        with pytest.raises(RuntimeError, match="AITemplateModelContainerCreate"):
            compile_model(y, detect_target(), str(tmp_path), "cross")
    model_src = (tmp_path / "cross" / "model-generated.cpp").read_text()
    entries = [e.rsplit("_", 1)[0] for e in re.findall(r'OpEntry\{"(\w+)"', model_src)]
    assert sorted(entries) == sorted(["gemm_rcr_permute_m2n3"] * 3 + ["mem_eff_attention", "gemm_rcr_bias_add"]), entries
    assert entries[-2:] == ["mem_eff_attention", "gemm_rcr_bias_add"]
    assert f", {S}, 1, {H}, stream);" in model_src and f", {Skv}, 1, {H}, stream);" in model_src
    assert f", {H}, {D // H}, {D // H}, {(D // H) ** -0.5!r}f, stream);" in model_src


# ---- fuse_mm_elementwise ----------------------------------------------------------------------
def _fuse(outputs):
    outputs = list(outputs)
    graph = transform.fuse_mm_elementwise(transform.toposort(outputs), outputs)
    return graph, outputs


def _op_names(graph):
    return [op._attrs["op"] for op in transform.get_sorted_ops(graph)]


@pytest.mark.parametrize("funcs,fused", [
    (("RELU",), "gemm_rcr_bias_relu"), (("SIGMOID",), "gemm_rcr_bias_sigmoid"), (("TANH",), "gemm_rcr_bias_tanh"),
    (("GELU",), "gemm_rcr_bias_gelu"), (("FASTGELU",), "gemm_rcr_bias_fast_gelu"),
    (("ADD",), "gemm_rcr_bias_add"), (("ADD", "ADD"), "gemm_rcr_bias_add_add"),
    (("ADD", "RELU"), "gemm_rcr_bias_add_relu"), (("ADD", "ADD", "RELU"), "gemm_rcr_bias_add_add_relu"),
    (("MUL",), "gemm_rcr_bias_mul"), (("MUL", "ADD"), "gemm_rcr_bias_mul_add"), (("MUL", "TANH"), "gemm_rcr_bias_mul_tanh"),
    (("SIGMOID", "MUL"), "gemm_rcr_bias_sigmoid_mul"), (("SIGMOID", "MUL", "TANH"), "gemm_rcr_bias_sigmoid_mul_tanh"),
])
def test_fuse_mm_elementwise_patterns(funcs, fused):
    """Every row of the reference's table (fuse_mm_elementwise_patterns.py:66-190) for gemm_rcr_bias."""
    M, N, K = 32, 48, 16
    X, W, Bv = Tensor([M, K], name="x", is_input=True), Tensor([N, K], name="w", is_input=True), \
        Tensor([N], name="b", is_input=True)
    y = ops.gemm_rcr_bias()(X, W, Bv)
    residuals = []
    for i, f in enumerate(funcs):
        if f in ("ADD", "MUL"):
            d = Tensor([M, N], name=f"d{i}", is_input=True)
            residuals.append(d)
            y = ops.elementwise(ops.FuncEnum[f])(y, d) if i % 2 == 0 else ops.elementwise(ops.FuncEnum[f])(d, y)
        else:
            y = ops.elementwise(ops.FuncEnum[f])(y)
    y._attrs["is_output"] = True
    y._attrs["name"] = "out"
    graph, outs = _fuse([y])
    assert _op_names(graph) == [fused]
    out = outs[0]
    assert out._attrs["name"] == "out" and out._attrs["is_output"] and graph[-1] is out
    op = list(out.src_ops())[0]
    assert op._attrs["inputs"][:3] == [X, W, Bv] and op._attrs["inputs"][3:] == residuals
    for t in (X, W, Bv, *residuals):
        assert list(t.dst_ops()) == [op]  # the replaced ops no longer hang off the inputs
    transform.check_leftover_elementwise(graph)


def test_fuse_mm_elementwise_bias_swish_operators_and_limits():
    M, N, K = 32, 48, 16
    X, W, Bv = Tensor([M, K], name="x", is_input=True), Tensor([N, K], name="w", is_input=True), \
        Tensor([N], name="b", is_input=True)
    # gemm_rcr + bias written with the + operator, then swish = x * sigmoid(x)
    x = ops.gemm_rcr()(X, W) + Bv
    y = x * ops.elementwise(ops.FuncEnum.SIGMOID)(x)
    y._attrs["is_output"] = True
    graph, outs = _fuse([y])
    assert _op_names(graph) == ["gemm_rcr_bias_swish"]
    # a tensor that is also a graph output, or has two consumers, ends the chain
    h = ops.gemm_rcr_bias()(X, W, Bv)
    h._attrs["is_output"] = True
    r = ops.elementwise(ops.FuncEnum.RELU)(h)
    r._attrs["is_output"] = True
    graph, outs = _fuse([h, r])
    assert _op_names(graph) == ["gemm_rcr_bias", "elementwise"]
    transform.check_leftover_elementwise(graph)  # the left-over RELU runs as a stand-alone launch
    # a residual of another shape (row broadcast) is not an epilogue of this backend
    h2 = ops.gemm_rcr_bias()(X, W, Bv)
    z = h2 + Tensor([1, N], name="row", is_input=True)
    z._attrs["is_output"] = True
    graph, outs = _fuse([z])
    assert _op_names(graph) == ["gemm_rcr_bias", "elementwise"]
    # the longest row wins and the rest of the chain stays: bias -> relu fused, the following tanh is left
    h3 = ops.elementwise(ops.FuncEnum.TANH)(ops.elementwise(ops.FuncEnum.RELU)(ops.gemm_rcr_bias()(X, W, Bv)))
    h3._attrs["is_output"] = True
    graph, outs = _fuse([h3])
    assert _op_names(graph) == ["gemm_rcr_bias_relu", "elementwise"]
    # scalars are accepted by the op and broadcasting follows numpy
    s = ops.elementwise(ops.FuncEnum.MUL)(Tensor([4, 1, 8], name="a", is_input=True), Tensor([5, 1], name="c", is_input=True))
    assert [d.value() for d in s.shape()] == [4, 5, 8]
    assert (2.0 * X)._attrs["src_ops"] and list((X / 2).src_ops())[0]._attrs["func"] == ops.FuncEnum.DIV
    with pytest.raises(RuntimeError, match="not compatible"):
        ops.elementwise(ops.FuncEnum.ADD)(Tensor([4, 3], name="p", is_input=True), Tensor([4, 2], name="q", is_input=True))


def test_compile_model_runs_the_fusion_pass_and_rejects_leftovers(tmp_path, monkeypatch):
    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    reset_name_counters()
    X = Tensor([64, 32], name="x", is_input=True)
    lin = nn.Linear(32, 48)
    lin.name_parameter_tensor("fc")
    y = ops.elementwise(ops.FuncEnum.RELU)(lin(X))
    y._attrs["is_output"] = True
    y._attrs["name"] = "y"
    import torch

    if torch.cuda.is_available():
        compile_model(y, detect_target(), str(tmp_path), "fused").close()
    else:
        with pytest.raises(RuntimeError, match="AITemplateModelContainerCreate"):
            compile_model(y, detect_target(), str(tmp_path), "fused")
    model_src = (tmp_path / "fused" / "model-generated.cpp").read_text()
    assert re.findall(r'OpEntry\{"(\w+)"', model_src) == ["gemm_rcr_bias_relu_0"]
    # a function without a stand-alone kernel, and a broadcast the stand-alone kernel cannot tile
    z = ops.elementwise(ops.FuncEnum.ELU)(nn.Linear(32, 48)(Tensor([64, 32], name="x2", is_input=True)))
    z._attrs["is_output"] = True
    with pytest.raises(NotImplementedError, match="no stand-alone kernel.*could not be fused"):
        compile_model(z, detect_target(), str(tmp_path), "leftover")
    col = Tensor([64, 1], name="col", is_input=True)
    z = ops.elementwise(ops.FuncEnum.EXP)(nn.Linear(32, 48)(Tensor([64, 32], name="x3", is_input=True))) * col
    z._attrs["is_output"] = True
    with pytest.raises(NotImplementedError, match="does not tile.*could not be fused"):
        compile_model(z, detect_target(), str(tmp_path), "leftover2")


def test_leftover_elementwise_ops_become_standalone_launches(tmp_path, monkeypatch):
    """Counterpart of the reference's fused_elementwise code generation
    (backend/rocm/elementwise/fused_elementwise.py) for ops no GEMM epilogue absorbed: one launch each."""
    from aitemplate_amd import _kernels
    from aitemplate_amd.compiler.ops.common.elementwise import STANDALONE_FUNCS, standalone_plan

    monkeypatch.setenv("CI_FLAG", "CIRCLECI")
    reset_name_counters()
    lib = _kernels.load()
    assert {f.value for f in ops.FuncEnum if lib.aitamd_elementwise_supported(f.value)} == \
        {f.value for f in STANDALONE_FUNCS}
    B = IntVar([1, 8], name="batch")
    X = Tensor([B, 64, 32], name="x", is_input=True)
    row = Tensor([1, 48], name="row", is_input=True)
    lin = nn.Linear(32, 48)
    lin.name_parameter_tensor("fc")
    h = lin(X)
    h._attrs["is_output"] = True  # two consumers: the chain cannot fold into the GEMM
    h._attrs["name"] = "h"
    e = ops.elementwise(ops.FuncEnum.EXP)(h)
    s = 2.0 - e  # constant first: f(b, a)
    r = ops.elementwise(ops.FuncEnum.MAX)(row, s)  # broadcast operand first
    y = r / h  # same shape
    y._attrs["is_output"] = True
    y._attrs["name"] = "y"
    plans = []
    for t in (e, s, r, y):
        a, b, value, swap = standalone_plan(list(t.src_ops())[0]._attrs)
        plans.append((a is h or a is e or a is s or a is r, None if b is None else b._attrs["name"], value, swap))
    assert plans == [(True, None, 0.0, 0), (True, None, 2.0, 1), (True, "row", 0.0, 1), (True, "h", 0.0, 0)]
    import torch

    if torch.cuda.is_available():
        compile_model([h, y], detect_target(), str(tmp_path), "ew").close()
    else:
        with pytest.raises(RuntimeError, match="AITemplateModelContainerCreate"):
            compile_model([h, y], detect_target(), str(tmp_path), "ew")
    model_src = (tmp_path / "ew" / "model-generated.cpp").read_text()
    assert re.findall(r'OpEntry\{"(\w+)"', model_src) == ["gemm_rcr_bias_0", "elementwise_1", "elementwise_2",
                                                          "elementwise_3", "elementwise_4"]
    assert "elementwise_3(" in model_src and "row, batch * " in model_src.replace("\n", " ")
    src = (tmp_path / "ew" / "elementwise_2.cpp").read_text()
    assert "aitamd_elementwise(2 /* SUB */, 0, a, b, out, numel, b_period" in src and "2.0f, 1, stream" in src
    # both operands broadcast, and an operand that broadcasts over an inner dim, are refused with the reason
    with pytest.raises(NotImplementedError, match="both broadcast"):
        list((Tensor([4, 1], name="p", is_input=True) + Tensor([1, 6], name="q", is_input=True)).src_ops())[0] \
            .standalone_plan()
    with pytest.raises(NotImplementedError, match="with 2 operands is not supported"):
        list(ops.elementwise(ops.FuncEnum.RELU)(h, h).src_ops())[0].standalone_plan()


def test_non_finite_constant_operands_are_spelled_as_cmath_macros(tmp_path):
    """A clamp against float('inf') is a legal graph; repr() would give the literal `inff`."""
    import subprocess

    from aitemplate_amd.backend.rocm.elementwise.elementwise import float_literal, gen_function

    assert float_literal(2.0) == "2.0f" and float_literal(-0.5) == "-0.5f" and float_literal(1e-8) == "1e-08f"
    assert float_literal(float("inf")) == "INFINITY" and float_literal(float("-inf")) == "-INFINITY"
    assert float_literal(float("nan")) == "NAN"
    X = Tensor([4, 8], name="x", is_input=True)
    y = ops.elementwise(ops.FuncEnum.MIN)(X, float("inf"))
    attrs = list(y.src_ops())[0]._attrs
    attrs["name"] = "elementwise_inf"
    src = gen_function(attrs)
    assert "INFINITY, 0, stream" in src and "inff" not in src and "#include <cmath>" in src
    # the generated function is valid C++ (syntax only: the kernel library's header is the one it includes)
    f = tmp_path / "ew.cpp"
    f.write_text(src)
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
                        f"-I{os.path.join(ROOT, 'include')}", f"-I{os.path.join(ROOT, 'aitemplate_amd', 'static', 'include')}",
                        str(f)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
