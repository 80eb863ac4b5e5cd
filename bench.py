"""Benchmark of the headline configuration: gemm_rcr_bias_gelu, fp16, M=24576 N=3072 K=768
(BERT-base FFN up-projection), on one MI355X, through the C ABI of the kernel library.

A "step" is one launch of the fused GEMM+bias+GELU over one full-size batch of synthetic
input that is already resident in HBM.  Operand sets rotate through a pool larger than the
256 MiB Infinity Cache so every step reads its inputs from HBM.

Prints ONE JSON line:  value = TFLOP/s over the K timed steps (wall clock between two device
synchronisations);  roofline.achieved = algorithmic FLOPs / average launch duration from HIP
events recorded around the same K launches on the launch stream (events at group boundaries
inside the same region give the median of the per-group averages beside it);
other_configs = the remaining benchmark configurations, each on the instance an untimed
profiling pass picked, each with its own roofline;  cpu_baseline = the reference tests'
PyTorch fp32 expression timed on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch, per (configuration, kernel instance): (bytes, the file under profiles/ that holds the two
# counter runs of this script the figure comes from: FETCH_SIZE, then WRITE_SIZE, each scaled by what the same
# counter read for the 256 MiB copy of --copy-probe in the same run).  A pair that is not listed was never measured
# and reports null with that reason.
MEASURED_TRAFFIC = {
    ("c2a", "gemm_rcr_f16_256x256x32_w2x4_persist4_m16"):
        (309_944_000, "profiles/gemm_rcr_persist_kernel_bias_gelu_M24576_N3072_K768_counters.txt"),
    ("c2b", "gemm_rcr_f16_320x256x32_w2x4_persist4_m16"):
        (307_647_000, "profiles/gemm_rcr_persist_kernel_bias_add_M24576_N768_K3072.txt"),
    ("c3", "gemm_rcr_f16_224x256x32_w2x4_persist4_m16"):
        (253_664_000, "profiles/gemm_rcr_persist_kernel_bias_add_add_M12608_N1024_K4096.txt"),
    ("c1", "gemm_rcr_f16_32x32x128_w2x2_dma4_o2_p0_m16_c0"):
        (6_892_000, "profiles/gemm_rcr_dma_kernel_bias_M256_N1024_K1024.txt"),
}


def measured_traffic(workload, instance):
    """(bytes or None, where the figure comes from or why there is none)."""
    t = MEASURED_TRAFFIC.get((workload, instance))
    if t is None:
        return None, f"no counter run of instance {instance} on configuration {workload} is held under profiles/"
    return t[0], f"{t[1]} (instance {instance})"

SHAPES = {
    # name: (op, M, N, K, residuals)
    "c1": ("gemm_rcr_bias", 256, 1024, 1024, 0),
    "c2a": ("gemm_rcr_bias_gelu", 24576, 3072, 768, 0),
    "c2b": ("gemm_rcr_bias_add", 24576, 768, 3072, 1),
    "c3": ("gemm_rcr_bias_add_add", 12608, 1024, 4096, 2),
}


def _median(values):
    v = sorted(values)
    n = len(v)
    return v[n // 2] if n % 2 else 0.5 * (v[n // 2 - 1] + v[n // 2])


class PowerSampler:
    """Board power from the amdgpu hwmon files of the first card, read every 20 ms by a thread while a timed
    region runs.  Reports nothing (None) where the files are missing or unreadable."""

    def __init__(self):
        import glob
        self.path = self.cap_path = None
        for h in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
            for f in ("power1_average", "power1_input"):
                if os.path.exists(os.path.join(h, f)):
                    self.path = os.path.join(h, f)
                    self.cap_path = os.path.join(h, "power1_cap")
                    break
            if self.path:
                break
        self.samples = []

    def _read(self, path):
        try:
            with open(path) as f:
                return int(f.read()) / 1e6
        except (OSError, ValueError, TypeError):
            return None

    def __enter__(self):
        import threading
        self.samples = []
        self._stop = threading.Event()

        def loop():
            while not self._stop.is_set():
                w = self._read(self.path) if self.path else None
                if w is not None:
                    self.samples.append(w)
                self._stop.wait(0.02)
        self._thread = threading.Thread(target=loop, daemon=True)
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join()

    def report(self):
        if not self.samples:
            return None
        cap = self._read(self.cap_path) if self.cap_path else None
        tail = self.samples[len(self.samples) * 2 // 5:]  # the sensor averages over about a second: drop the ramp
        return {"avg_w": round(sum(tail) / len(tail), 1), "max_w": round(max(tail), 1), "cap_w": cap, "samples": len(tail),
                "source": f"{os.path.basename(self.path)} of the card's hwmon, every 20 ms over the last 60 % of the region"}


# untimed launches in front of every timed region, whatever --warmup says (AITAMD_BENCH_SETTLE overrides: a knob for
# measuring how long the clocks take to settle, not for the metric)
SETTLE_LAUNCHES = int(os.environ.get("AITAMD_BENCH_SETTLE", "400"))
GRAPH_MIN_LAUNCHES = 100   # launches held by the graph a launch-bound configuration is timed with
MIN_GROUP_LAUNCHES = 10    # fewest direct launches between two of the events that cut a timed region into groups


def graph_plan(steps, groups, min_launches=GRAPH_MIN_LAUNCHES):
    """(launches per captured graph, replays in the timed region).  A graph of one 5 us kernel measures the cost of
    launching a graph, not the kernel: the graph always holds at least `min_launches` launches, however few steps
    were asked for, and the timed region replays it once per group."""
    groups = max(1, min(groups, steps))
    return max(min_launches, -(-steps // groups)), groups


def timed_region(torch, step, steps, warmup, groups=20, graph=False, power=None, settle=SETTLE_LAUNCHES):
    """`settle` + W untimed steps, then exactly K steps between two device synchronisations.  The settle launches
    take the region out of the transient after an idle spell (clocks and translation caches need some 30 ms of
    load; the first 200 launches run up to 1.5x slower), so that the figure does not depend on the W the caller
    chose.  Events on the launch stream bracket the region and cut it into up to `groups` groups of consecutive
    launches: the region's average and the median of the group averages both come from the same K launches.  With
    `graph` the launches are captured once (untimed, graph_plan() says how many) and the timed region replays
    them: for kernels of a few microseconds, whose launches the host cannot issue as fast as the GPU retires
    them."""
    for i in range(settle + warmup):
        step(i)
    torch.cuda.synchronize()
    # a group holds at least MIN_GROUP_LAUNCHES launches: an event between two launches keeps the second from
    # starting while the first one's last workgroups finish, 3 to 4 us per launch of the headline kernel (measured:
    # 20 steps in 20 groups 0.1265-0.1305 ms per launch, in the same process 1000 steps in 20 groups 0.1230-0.1241)
    groups = max(1, min(groups, steps // MIN_GROUP_LAUNCHES if not graph else steps))
    cuts = [steps * g // groups for g in range(groups + 1)]
    if graph:
        per, groups = graph_plan(steps, groups)
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()  # default priority
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                for i in range(per):
                    step(i)
        torch.cuda.current_stream().wait_stream(side)
        for _ in range(1 + -(-settle // per)):  # untimed: the first replay uploads the graph
            g.replay()
        torch.cuda.synchronize()
        cuts = [per * k for k in range(groups + 1)]
        steps = per * groups
    events = [torch.cuda.Event(enable_timing=True) for _ in cuts]
    if power is not None:
        power.__enter__()
    t0 = time.perf_counter()
    events[0].record()
    for k in range(groups):
        if graph:
            g.replay()
        else:
            for i in range(cuts[k], cuts[k + 1]):
                step(i)
        events[k + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    if power is not None:
        power.__exit__()
    per_group = [events[k].elapsed_time(events[k + 1]) / (cuts[k + 1] - cuts[k]) for k in range(groups)]
    return {"steps": steps, "wall_ms_per_step": wall_ms / steps,
            "event_ms_per_launch": events[0].elapsed_time(events[-1]) / steps,
            "median_ms_per_launch": _median(per_group), "groups": groups, "settle_launches": settle}


def _make_pool(torch, op, M, N, K, nres, pool_bytes=600 << 20):
    set_bytes = 2 * (M * K + N * K + N + (1 + nres) * M * N)
    sets = max(2, min(16, pool_bytes // set_bytes + 1)) if pool_bytes else 1
    g = torch.Generator(device="cuda").manual_seed(1)
    pool = []
    for _ in range(sets):
        x = torch.randn(M, K, device="cuda", generator=g).half()
        w = (torch.randn(N, K, device="cuda", generator=g) * K ** -0.5).half()
        b = ((torch.rand(N, device="cuda", generator=g) - 0.5) * 0.2).half()
        d = [torch.randn(M, N, device="cuda", generator=g).half() for _ in range(nres)]
        out = torch.empty(M, N, device="cuda", dtype=torch.float16)
        pool.append((x, w, b, d, out))
    return pool


class GemmCase:
    """One GEMM configuration: its operand pool and, for the instances that split K, the scratch memory."""

    def __init__(self, torch, eager, kernels, name):
        self.torch, self.eager, self.kernels, self.name = torch, eager, kernels, name
        self.op, self.M, self.N, self.K, self.nres = SHAPES[name]
        self.epi = kernels.EPILOGUE_OF_OP[self.op]
        self.pool = _make_pool(torch, self.op, self.M, self.N, self.K, self.nres)
        lib = kernels.load()
        self.supported = [a for a in range(lib.aitamd_gemm_num_algos(self.epi, 0))
                          if lib.aitamd_gemm_algo_supported(self.epi, 0, a, self.M, self.N, self.K, self.K, self.K, 16)]
        need = max([eager.gemm_workspace_bytes(self.op, a, self.M, self.N, self.K) for a in self.supported] + [0])
        self.workspace = eager.new_workspace(need) if need > 0 else None
        self.flops = 2 * self.M * self.N * self.K
        self.bytes = 2 * (self.M * self.K + self.N * self.K + self.N + (1 + self.nres) * self.M * self.N)

    def step_fn(self, algo):
        pool, op, nres, ws, gemm = self.pool, self.op, self.nres, self.workspace, self.eager.gemm

        def step(i):
            x, w, b, d, out = pool[i % len(pool)]
            gemm(op, x, w, b, d[0] if nres >= 1 else None, d[1] if nres >= 2 else None, out=out, algo=algo,
                 workspace=ws)
        return step

    @property
    def launch_bound(self):
        """A launch lasts a few microseconds: only a replayed graph lets the GPU, not the host, set the pace."""
        return self.flops < 5e9

    def pick_instance(self, iters=15, regions=3):
        """Untimed selection pass, the same procedure compile_model's profiling step applies
        (python/aitemplate/compiler/ops/gemm_universal/gemm_common.py:743-829 in the reference):
        time every instance that supports the problem and keep the fastest.  Every instance gets `regions`
        regions, visited round-robin so that a slow spell of the box does not fall on one instance, and counts
        with its best one."""
        best_ms = {algo: float("inf") for algo in self.supported}
        settle = SETTLE_LAUNCHES
        for _ in range(regions):
            for algo in self.supported:
                ms = timed_region(self.torch, self.step_fn(algo), iters * (4 if self.launch_bound else 1), 3, groups=1,
                                  graph=self.launch_bound, settle=settle)["event_ms_per_launch"]
                best_ms[algo] = min(best_ms[algo], ms)
                settle = 0  # the pass itself keeps the device loaded from here on
        return min(self.supported, key=lambda a: best_ms[a]) if self.supported else -1

    def instance_name(self, algo):
        return self.kernels.gemm_algo_names(self.epi, 0)[algo]


def _roofline(bound, work, ms_avg, ms_median):
    """work = algorithmic FLOPs (bound "mfma") or bytes (bound "hbm") of one launch."""
    peak, unit, scale = (PEAK_FP16_TFLOPS, "TFLOP/s", 1e9) if bound == "mfma" else (PEAK_HBM_GBS, "GB/s", 1e6)
    achieved = work / ms_avg / scale
    return {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "frac_at_median_launch": round(work / ms_median / scale / peak, 4)}


def other_configs(torch, eager, kernels, steps, warmup, vendor_baseline=True):
    """Configurations 1, 2b, 3 (MFMA-bound GEMMs), 4 (bmm_rcr, HBM-bound) and 5 (fused attention)."""
    out = {}
    for name in ("c1", "c2b", "c3"):
        case = GemmCase(torch, eager, kernels, name)
        algo = case.pick_instance()
        graph = case.launch_bound  # (config 1)
        r = timed_region(torch, case.step_fn(algo), steps, warmup, graph=graph)
        ws = eager.gemm_workspace_bytes(case.op, algo, case.M, case.N, case.K)
        out[name] = {"op": case.op, "M": case.M, "N": case.N, "K": case.K, "instance": case.instance_name(algo),
                     "workspace_bytes": ws,
                     "launches": f"graph replay, {graph_plan(steps, 20)[0]} launches per graph" if graph else "direct",
                     "timed_launches": r["steps"], "settle_launches": r["settle_launches"],
                     "ms": round(r["event_ms_per_launch"], 5), "median_ms": round(r["median_ms_per_launch"], 5),
                     "tflops": round(case.flops / r["event_ms_per_launch"] / 1e9, 2),
                     "roofline": _roofline("mfma", case.flops, r["event_ms_per_launch"], r["median_ms_per_launch"])}
        out[name]["roofline"]["traffic"], out[name]["roofline"]["traffic_source"] = measured_traffic(
            name, out[name]["instance"])
        if vendor_baseline:
            # a baseline, not part of the product: the same result from PyTorch-ROCm's own operators on the same
            # operand sets (its GEMM library with a bias, then one add kernel per residual)
            try:
                pool, nres = case.pool, case.nres

                def torch_ops(i):
                    x, w, b, d, _ = pool[i % len(pool)]
                    y = torch.nn.functional.linear(x, w, b)
                    for t in d[:nres]:
                        y = y + t
                    return y
                rv = timed_region(torch, torch_ops, steps, warmup, graph=graph)
                out[name]["vendor_baseline"] = {"torch_linear_plus_adds_median_ms": round(rv["median_ms_per_launch"], 5),
                                                "kernels_per_step": 1 + nres}
            except Exception as e:
                out[name]["vendor_baseline"] = {"error": f"{type(e).__name__}: {e}"}
        del case
    g = torch.Generator(device="cuda").manual_seed(4)
    sets4 = [(torch.randn(768, 384, 64, device="cuda", generator=g).half() / 8,
              torch.randn(768, 384, 64, device="cuda", generator=g).half() / 8,
              torch.empty(768, 384, 384, device="cuda", dtype=torch.float16)) for _ in range(3)]
    r4 = timed_region(torch, lambda i: eager.bmm_rcr(sets4[i % 3][0], sets4[i % 3][1], out=sets4[i % 3][2]), steps, warmup)
    b4 = 2 * 768 * (2 * 384 * 64 + 384 * 384)
    out["c4"] = {"op": "bmm_rcr", "B": 768, "M": 384, "N": 384, "K": 64, "ms": round(r4["event_ms_per_launch"], 5),
                 "median_ms": round(r4["median_ms_per_launch"], 5),
                 "roofline": _roofline("hbm", b4, r4["event_ms_per_launch"], r4["median_ms_per_launch"])}
    if vendor_baseline:
        try:
            rv = timed_region(torch, lambda i: torch.bmm(sets4[i % 3][0], sets4[i % 3][1].transpose(1, 2), out=sets4[i % 3][2]),
                              steps, warmup)
            out["c4"]["vendor_baseline"] = {"torch_bmm_median_ms": round(rv["median_ms_per_launch"], 5)}
        except Exception as e:
            out["c4"]["vendor_baseline"] = {"error": f"{type(e).__name__}: {e}"}
    del sets4
    sets5 = [tuple(torch.randn(16, 4096, 40, device="cuda", generator=g).half() for _ in range(3)) for _ in range(16)]
    out5 = torch.empty(2, 4096, 8, 40, device="cuda", dtype=torch.float16)
    r5 = timed_region(torch, lambda i: eager.bmm_softmax_bmm_permute(*sets5[i % 16], shape=(8,), scale=40 ** -0.5, out=out5),
                      steps, warmup)
    f5 = 4 * 16 * 4096 * 4096 * 40
    out["c5"] = {"op": "bmm_softmax_bmm_permute", "B": 16, "M": 4096, "N": 4096, "K": 40, "O": 40,
                 "ms": round(r5["event_ms_per_launch"], 5), "median_ms": round(r5["median_ms_per_launch"], 5),
                 "tflops": round(f5 / r5["event_ms_per_launch"] / 1e9, 2),
                 "roofline": _roofline("mfma", f5, r5["event_ms_per_launch"], r5["median_ms_per_launch"])}
    if vendor_baseline:
        # a baseline, not part of the product: PyTorch-ROCm's fused attention on the same operand sets
        try:
            sdpa = torch.nn.functional.scaled_dot_product_attention
            v5 = [tuple(t.view(2, 8, 4096, 40) for t in s) for s in sets5]
            rv = timed_region(torch, lambda i: sdpa(*v5[i % 16]), steps, warmup)
            out["c5"]["vendor_baseline"] = {"torch_scaled_dot_product_attention_median_ms": round(rv["median_ms_per_launch"], 5)}
        except Exception as e:
            out["c5"]["vendor_baseline"] = {"error": f"{type(e).__name__}: {e}"}
    return out


def power_and_vendor_baseline(torch, eager, case, algo, seconds=2.5):
    """Board power under the headline launch, and a baseline that is not part of the product: the bias-only GEMM of
    the headline shape through this library and through torch.nn.functional.linear (the vendor's GEMM library under
    PyTorch-ROCm; it has no fused tanh-GELU epilogue, so the comparison is on gemm_rcr_bias).  Each leg repeats its
    launch for about `seconds`, long enough for the board's power sensor, on the same rotating operand sets, one
    leg after the other in this process."""
    pool, out = case.pool, {}

    def ours_bias(i):
        x, w, b, _, o = pool[i % len(pool)]
        eager.gemm("gemm_rcr_bias", x, w, b, out=o)

    def vendor(i):
        x, w, b, _, o = pool[i % len(pool)]
        torch.nn.functional.linear(x, w, b)
    for name, fn in (("headline_launch", case.step_fn(algo)), ("this_library_gemm_rcr_bias", ours_bias),
                     ("torch_nn_functional_linear", vendor)):
        try:
            ps = PowerSampler()
            r = timed_region(torch, fn, int(seconds / 0.000125), 300, power=ps)
            out[name] = {"median_ms": round(r["median_ms_per_launch"], 5),
                         "tflops": round(case.flops / r["median_ms_per_launch"] / 1e9, 2), "board_power": ps.report()}
        except Exception as e:  # a baseline must never take the bench line down
            out[name] = {"error": f"{type(e).__name__}: {e}"}
    out["note"] = (f"M={case.M} N={case.N} K={case.K} fp16, {int(seconds / 0.000125)} launches per leg after 300 untimed; "
                   "headline_launch is gemm_rcr_bias_gelu, the other two are gemm_rcr_bias")
    return out


def copy_probe(torch, nbytes=256 << 20, reps=5):
    """A plain device copy of known size, for scaling the FETCH_SIZE / WRITE_SIZE counters of a
    counter-collection run of this script (the copy reads nbytes and writes nbytes per launch)."""
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(reps):
        dst.copy_(src)
    torch.cuda.synchronize()


def in_abi(torch, count=100):
    """The same workload through the whole product path: ops.gemm_rcr_bias_gelu -> compile_model
    (instance chosen by the prebuilt profiler program) -> AITemplateModelContainerBenchmark.
    One fixed operand set, as a serving loop would hold it."""
    import tempfile

    from aitemplate_amd.compiler import compile_model, ops
    from aitemplate_amd.compiler.base import Tensor
    from aitemplate_amd.testing import detect_target

    op, M, N, K, _ = SHAPES["c2a"]
    X = Tensor([M, K], name="input_0", is_input=True)
    W = Tensor([N, K], name="input_1", is_input=True)
    B = Tensor([N], name="input_2", is_input=True)
    Y = getattr(ops, op)()(X, W, B)
    Y._attrs["name"], Y._attrs["is_output"] = "output_0", True
    (x, w, b, _, out), = _make_pool(torch, op, M, N, K, 0, pool_bytes=0)[:1]
    with tempfile.TemporaryDirectory(prefix="aitamd_bench_") as tmp:
        with compile_model(Y, detect_target(), tmp, "bench_c2a") as module:
            # the GPU has idled through the build: one untimed batch brings the clocks back up
            module.benchmark_with_tensors([x, w, b], [out], count=count)
            ms = sorted(module.benchmark_with_tensors([x, w, b], [out], count=count)[0] for _ in range(3))[1]
    return {"ms_per_run": round(ms, 5), "tflops": round(2 * M * N * K / (ms * 1e-3) / 1e12, 2),
            "via": f"compile_model + AITemplateModelContainerBenchmark, median of 3 batches of count={count} after "
                   "one untimed batch, one fixed operand set"}


def cpu_baseline(torch, max_seconds=20.0):
    """The oracle expression of the headline config in fp32 on the host cores."""
    from oracle import oracle

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    op, M, N, K, _ = SHAPES["c2a"]
    inp = oracle.config_inputs("c2a")
    x, w, b = inp["x"].float(), inp["w"].float(), inp["bias"].float()
    times = []
    t_start = time.perf_counter()
    for i in range(2 + 5):
        t0 = time.perf_counter()
        oracle.torch_gemm(op, x, w, b)
        dt = time.perf_counter() - t0
        if i >= 2:
            times.append(dt)
        if time.perf_counter() - t_start > max_seconds and len(times) >= 1:
            break
    times.sort()
    med = times[len(times) // 2]
    return {"value": 2 * M * N * K / med / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"full c2a workload (M={M} N={N} K={K}), fp32 torch F.gelu(F.linear) on CPU, "
                      f"median of {len(times)} runs after 2 warm-ups, {med * 1e3:.1f} ms each"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults: the first 200 or so launches after an idle spell run up to 1.5x slower (clocks and translation
    # caches settle over some 30 ms); 500 untimed launches put the timed region into the steady state a loaded
    # server is in
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--algo", default="-1",
                    help="kernel instance, by index or by name (default: see --select)")
    ap.add_argument("--select", choices=("profile", "heuristic"), default="profile",
                    help="how the kernel instance is chosen when --algo is not given: an untimed profiling "
                         "pass over all instances (what compile_model does) or the library's heuristic")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch a 256 MiB device copy 5 times (counter calibration for profiler runs)")
    ap.add_argument("--workload", choices=tuple(SHAPES), default="c2a",
                    help="diagnostic, for profiler runs of one kernel: time this configuration in the headline "
                         "region instead of configs[1] (the line then says so in `data` and is not the metric)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--constant-operands", action="store_true",
                    help="diagnostic: time the headline kernel on x = 1, w = 1/K instead of the random operands")
    ap.add_argument("--no-constant-data", action="store_true",
                    help="skip the diagnostic launch of the same kernel on constant operands")
    ap.add_argument("--no-in-abi", action="store_true", help="skip the compile_model + container Benchmark leg")
    ap.add_argument("--no-vendor-baseline", action="store_true",
                    help="skip the board-power legs (headline launch, bias-only GEMM through this library and through "
                         "torch.nn.functional.linear)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="time the headline configuration only (for profiler runs of one kernel)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no exchange step and every GPU box here has one "
              "GPU; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from aitemplate_amd import _kernels, eager

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    _kernels.load()

    case = GemmCase(torch, eager, _kernels, args.workload)
    M, N, K = case.M, case.N, case.K
    diagnostic = args.workload != "c2a"
    if diagnostic:  # one kernel under a profiler: none of the legs that belong to the metric's line
        args.no_vendor_baseline = args.no_other_configs = args.no_in_abi = args.no_cpu_baseline = True
    if args.algo.lstrip("-").isdigit():
        algo = int(args.algo)
    else:
        algo = _kernels.load().aitamd_gemm_find_algo(case.epi, 0, args.algo.encode())
        if algo < 0:
            sys.exit(f"bench.py: no kernel instance named {args.algo}")
    algo_given = algo >= 0
    if algo < 0 and args.select == "profile":
        algo = case.pick_instance()
    if algo < 0:
        algo = _kernels.load().aitamd_gemm_heuristic_algo(case.epi, 0, 1, M, N, K, K, K, 16)
    if args.copy_probe:
        copy_probe(torch)
    if args.constant_operands:
        # diagnostic run (engine clock on idle multiplier inputs, for the counter profiles): not the metric
        case.pool = [(torch.ones_like(x), torch.full_like(w, 1.0 / K), torch.zeros_like(b), d, out)
                     for (x, w, b, d, out) in case.pool]
    r = timed_region(torch, case.step_fn(algo), args.steps, args.warmup, graph=diagnostic and case.launch_bound)
    tflops = case.flops / (r["wall_ms_per_step"] * 1e-3) / 1e12
    instance = case.instance_name(algo)
    roofline = _roofline("mfma", case.flops, r["event_ms_per_launch"], r["median_ms_per_launch"])
    roofline["avg_launch_ms"] = round(r["event_ms_per_launch"], 5)
    roofline["median_launch_ms"] = round(r["median_ms_per_launch"], 5)
    roofline["median_of"] = f"{r['groups']} groups of consecutive launches inside the timed region"
    roofline["settle_launches"] = r["settle_launches"]
    roofline["traffic"], roofline["traffic_source"] = measured_traffic(args.workload, instance)
    # The device is power-limited on this kernel and its engine clock follows the operands: the same launch on
    # constant data (no toggling in the multipliers) is a diagnostic for how much of the distance to the peak is
    # clock, not schedule.  Never the reported value.
    const_ms = None
    if not args.no_constant_data:
        import types
        const_pool = [(torch.ones_like(x), torch.full_like(w, 1.0 / K), torch.zeros_like(b), d, out)
                      for (x, w, b, d, out) in case.pool[:2]]
        shadow = types.SimpleNamespace(pool=const_pool, op=case.op, nres=case.nres, workspace=case.workspace, eager=eager)
        rc = timed_region(torch, GemmCase.step_fn(shadow, algo), max(20, args.steps // 4), max(20, args.warmup // 4))
        const_ms = rc["median_ms_per_launch"]
        del const_pool, shadow
    roofline["same_launch_on_constant_operands"] = None if const_ms is None else {
        "median_launch_ms": round(const_ms, 5), "frac": round(case.flops / const_ms / 1e9 / PEAK_FP16_TFLOPS, 4),
        "note": "x = 1, w = 1/K, bias = 0: same instructions, idle multiplier inputs; the difference to the "
                "measured launch is the engine clock under the board's power limit"}
    line = {
        "metric": "TFLOP/s + % fp16 MFMA peak, gemm_rcr_bias_gelu M=24576 K=768 N=3072",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(r["wall_ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": ("constant operands (diagnostic run, not the metric)" if args.constant_operands else
                 f"synthetic; DIAGNOSTIC run of configuration {args.workload} ({case.op} M={M} N={N} K={K}), not the metric"
                 if diagnostic else "synthetic"),
        "pct_of_fp16_mfma_peak": round(100.0 * tflops / PEAK_FP16_TFLOPS, 2),
        "config": {"workload": "configs[1]: gemm_rcr_bias_gelu fp16 X[24576,768] W[3072,768] bias[3072], "
                               "fp32 accumulate, tanh-GELU fused, inputs resident in HBM, rotating operand sets",
                   "instance": instance, "instance_index": algo,
                   "instance_selected_by": "--algo" if algo_given else args.select},
        "roofline": roofline,
    }
    # The headline is measured; the legs below add to the line and must not be able to take it away.
    def leg(key, fn):
        try:
            line[key] = fn()
        except Exception as e:
            line[key] = {"error": f"{type(e).__name__}: {e}"}
    if not args.no_vendor_baseline:
        leg("power_and_vendor_baseline", lambda: power_and_vendor_baseline(torch, eager, case, algo))
    del case
    if not args.no_other_configs:
        leg("other_configs", lambda: other_configs(torch, eager, _kernels, max(20, min(200, args.steps // 2)),
                                                   max(5, min(50, args.warmup // 2)),
                                                   vendor_baseline=not args.no_vendor_baseline))
    if not args.no_in_abi:
        leg("in_abi", lambda: in_abi(torch))
    if not args.no_cpu_baseline:
        leg("cpu_baseline", lambda: cpu_baseline(torch))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
