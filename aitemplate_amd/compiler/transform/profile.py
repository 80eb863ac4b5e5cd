"""Profile every op that has a profiler and record the winning kernel instances.

Counterpart of python/aitemplate/compiler/transform/profile.py:52-128 together with
backend/codegen.gen_profiler (codegen.py:69-88): generate / place profilers, run them on the
given devices (one at a time per device), then let the delegate pick the fastest instance per
workload.  Without a GPU, or with CI_FLAG=CIRCLECI, instances are chosen by heuristic."""
import logging
import os
from typing import List, Optional

from ...backend.builder import Builder
from ...backend.profiler_runner import ProfilerRunner
from ...backend.target import Target
from ..base import DynamicProfileStrategy, Tensor
from ..ops.gemm_universal.gemm_common import GemmProfilerPostprocessingDelegate
from .transform_utils import get_sorted_ops

_LOGGER = logging.getLogger(__name__)


def _gpu_available() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return os.path.exists("/dev/kfd")


def profile(sorted_graph: List[Tensor], workdir: str = "./tmp", devices: Optional[List[int]] = None,
            dynamic_profiling_strategy=DynamicProfileStrategy.MAX, timeout: int = 500) -> None:
    target = Target.current()
    if devices is None:
        env = os.environ.get(target.dev_select_flag())
        devices = [d for d in env.split(",") if d != ""] if env else ["0"]
    profile_dir = workdir
    ops = [op for op in get_sorted_ops(sorted_graph) if op._attrs.get("has_profiler")]
    generated = []
    done = set()
    for op in ops:
        res = op.gen_profiler(profile_dir, dynamic_profiling_strategy)
        if res:
            generated.extend(res)
    Builder().make_profilers(generated, profile_dir)
    use_gpu = _gpu_available() and not target.use_dummy_profiling_results()
    runner = None
    if use_gpu:
        runner = ProfilerRunner([str(d) for d in devices], GemmProfilerPostprocessingDelegate(), timeout=timeout)
    cache = {}
    for op in ops:
        # identical workloads of identical ops are timed once
        sig = (op._attrs["op"], tuple(op._attrs["exec_path"].keys()), tuple(op._attrs["op_instance"].keys()),
               op._attrs.get("scale"), str(op._attrs.get("shape")))
        if sig in cache:
            done.add(id(op))
            continue
        cache[sig] = op
        op.profile(runner, profile_dir)
    if runner is not None:
        runner.join()
    for op in ops:
        if id(op) in done:
            sig = (op._attrs["op"], tuple(op._attrs["exec_path"].keys()), tuple(op._attrs["op_instance"].keys()),
                   op._attrs.get("scale"), str(op._attrs.get("shape")))
            first = cache[sig]
            for key, item in op._attrs["exec_path"].items():
                item.algo = first._attrs["exec_path"][key].algo
            op._attrs["workspace"] = first._attrs["workspace"]
    for op in ops:
        for key, item in op._attrs["exec_path"].items():
            if not item.algo:
                raise RuntimeError(f"profiling left {op._attrs['name']} {key} without a kernel instance")
