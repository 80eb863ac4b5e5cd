"""Base class of the GEMM-family ops: dim bookkeeping, exec keys, profiling, registry dispatch.

Counterpart of python/aitemplate/compiler/ops/gemm_universal/gemm_common.py:198-838.
The protocol towards the backend is the current frontend one:
  "<target>.<op>.config"(attrs, dtype)                      -> fills attrs["op_instance"]
  "<target>.<op>.filter"(instance_name, attrs, ab_alignment) -> bool
  "<target>.<op>.gen_profiler"(attrs, workdir, profiler_filename, dim_info_dict) -> [(src, exe)]
  "<target>.<op>.gen_function"(attrs, exec_cond_template, dim_info_dict) -> str
  "<target>.<op>.func_decl"(attrs) / "<target>.<op>.func_call"(attrs, indent)  (used by codegen)
One profiler executable is run per op and workload; it prints one
"OP:<instance>,TIME:<ms>,WS:<bytes>" line per instance and the fastest wins.
"""
from __future__ import annotations

import logging
import math
import os
import re
from collections import OrderedDict
from dataclasses import dataclass
from enum import Enum
from hashlib import sha1
from typing import Any, Dict, List, Optional, Union

from ....backend import registry
from ....backend.target import Target
from ....utils import alignment
from ...base import DynamicProfileStrategy, ExecItem, IntImm, IntVar, Operator, Tensor
from ...dtype import is_same_dtype
from ...tensor_accessor import TensorAccessor

_LOGGER = logging.getLogger(__name__)

# C++ condition wrapped around the launch of one profiled workload
EXEC_COND_TEMPLATE = """{indent}if ({cond}) {{
{indent}  {program}
{indent}  return;
{indent}}}
"""


class Source(Enum):
    INPUT = 1
    OUTPUT = 2


@dataclass
class DimInfo:
    """Where one problem dim (M, N, K, B, O) lives: which tensor, which of its dims.
    `placeholder` marks a batch dim of 1 that broadcasts and must not define B."""

    source: Source
    tensor_idx: int
    dim_idx: Union[int, List[int]]
    placeholder: bool = False

    def __post_init__(self):
        if isinstance(self.dim_idx, int):
            self.dim_idx = [self.dim_idx]


def extract_shape_from_accessor(attrs: Dict[str, Any], source: Source, idx: int):
    key = "input_accessors" if source == Source.INPUT else "output_accessors"
    if key in attrs:
        return attrs[key][idx].original_shapes
    tensors = attrs["inputs"] if source == Source.INPUT else attrs["outputs"]
    return tensors[idx]._attrs["shape"]


def create_input_batch_diminfo(input_shapes, batch_dims, output_batch) -> List[DimInfo]:
    out = []
    for idx, shape in enumerate(input_shapes):
        if len(shape) > 2:
            out.append(DimInfo(Source.INPUT, tensor_idx=idx, dim_idx=batch_dims[idx],
                               placeholder=shape[batch_dims[idx]] != output_batch))
    return out


def gemm_inverse_key_func(key: str) -> List[int]:
    """Recover the integers of an exec key positionally ("M == 256 && N == 1024 && K == 1024" -> [256, 1024, 1024])."""
    return [int(x) for x in re.findall(r"(\d+)", key)]


def default_align_ab(a: int, b: int, dtype: str) -> int:
    return alignment.find_max_alignment(math.gcd(a, b), dtype)


def profile_cache_args(func_attrs: Dict[str, Any], exec_key: str) -> Optional[Dict[str, Any]]:
    """Key of one workload in the profiling-result cache (reference: the GemmQueryEntry built at
    gemm_common.py:436-458), or None when no target is active."""
    from ....backend import target as target_mod
    from ....backend.profiler_cache import exec_entry_sha1

    if target_mod.CURRENT_TARGET is None or "inputs" not in func_attrs or not func_attrs.get("op_instance"):
        return None
    names = sorted(func_attrs["op_instance"].keys())
    shape = func_attrs.get("shape")
    entry = exec_key if shape is None else f"{exec_key} | shape={tuple(shape)} | causal={func_attrs.get('causal')}"
    return {
        "op_type": func_attrs["op"],
        "dtype": func_attrs["inputs"][0]._attrs["dtype"],
        "device": target_mod.CURRENT_TARGET.device_name(),
        "instances_sha1": sha1(";".join(names).encode("utf-8")).hexdigest(),
        "exec_entry": entry,
        "exec_entry_sha1": exec_entry_sha1(entry),
    }


class GemmProfilerPostprocessingDelegate:
    """Collects the profiler runs of all GEMM ops and, once they have finished, writes the
    fastest instance of each workload into the op's exec_path
    (reference: gemm_common.py:853-935)."""

    def __init__(self):
        self._instances = []

    def add_instance(self, result, func_attrs, profiler_filename, exec_key, split_k, exec_entry_sha1=None):
        self._instances.append((result, func_attrs, profiler_filename, exec_key, split_k))

    def postprocess_results(self):
        by_workload = OrderedDict()
        for result, attrs, fname, exec_key, split_k in self._instances:
            by_workload.setdefault((id(attrs), exec_key), []).append((result, attrs, split_k))
        for (_, exec_key), entries in by_workload.items():
            # each entry's result is a list of (instance name, ProfileResult); min time wins
            best = None
            for results, attrs, split_k in entries:
                for name, res in results:
                    if best is None or res.duration < best[1].duration:
                        best = (name, res, attrs, split_k)
            if best is None:
                raise RuntimeError(f"Profile workload: {exec_key} failed. Results: {entries}.")
            name, res, attrs, split_k = best
            attrs["exec_path"][exec_key].algo = name
            attrs["workspace"] = max(attrs["workspace"], res.workspace)
            attrs["split_k"] = split_k
            _LOGGER.info("Profiler (%s %s) selected %s: %.4f ms", attrs["op"], exec_key, name, res.duration)
            args = profile_cache_args(attrs, exec_key)
            if args is not None:
                args.update(algo=name, workspace=res.workspace, split_k=split_k, duration=res.duration)
                Target.current().insert_profile_cache("gemm", args)


class gemm(Operator):
    """Base gemm operator."""

    def __init__(self):
        super().__init__()
        self._attrs["op"] = "gemm"
        self._attrs["has_profiler"] = True
        self._attrs["f_ab_alignment"] = None
        self._attrs["epilogue_alignment"] = 1
        self._attrs["epilogue"] = "LinearCombination"
        self._attrs["workspace"] = 0
        self._attrs["split_k"] = 1
        self._attrs["num_sources"] = 0
        self._attrs["alpha"] = 1.0
        self._attrs["permute_shape"] = ""
        self.exec_cond_template = EXEC_COND_TEMPLATE

    # ---- shapes -------------------------------------------------------------
    def _extract_epilogue_alignment(self, output_shape: List[Any], dynamic_profiling_strategy=None) -> None:
        last = output_shape[-1]
        if isinstance(last, int):
            n = last
        elif isinstance(last, IntImm):
            n = last.value()
        elif dynamic_profiling_strategy is None:
            return
        elif dynamic_profiling_strategy == DynamicProfileStrategy.MAX:
            n = last.upper_bound()
        elif dynamic_profiling_strategy == DynamicProfileStrategy.MIN:
            n = last.lower_bound()
        else:
            raise RuntimeError(f"Unsupported dynamic profiling strategy: {dynamic_profiling_strategy}")
        self._attrs["epilogue_alignment"] = alignment.find_max_alignment(n, self._attrs["inputs"][0].dtype())

    def _infer_shapes(self, a: Tensor, b: Tensor):
        raise NotImplementedError("_infer_shapes() is not implemented!")

    def _extract_dims(self, for_profiling: bool = False) -> Dict[str, List[DimInfo]]:
        raise NotImplementedError("extract_dims() is not implemented!")

    @staticmethod
    def _gen_exec_key(name_value_mapping: Dict[str, List[int]]) -> str:
        parts = []
        for name, values in name_value_mapping.items():
            if len(values) == 1:
                parts.append(f"{name} == {values[0]}")
            elif len(values) > 1:
                parts.append(f"{name} >= {values[0]} && {name} <= {values[-1]}")
            else:
                raise RuntimeError(f"Gemm input has empty dim values: {values}")
        return " && ".join(parts)

    def _dim_value_ranges(self) -> "OrderedDict[str, List[int]]":
        """{dim name: sorted unique [min, max]} over the op's current shapes."""
        out = OrderedDict()
        for name, infos in self._extract_dims().items():
            chosen = None
            for d in infos:
                if d.placeholder:
                    continue
                if chosen is None or d.source == Source.INPUT:
                    chosen = d
            assert chosen is not None, f"Couldn't find valid dim info for dim {name}"
            shape = extract_shape_from_accessor(self._attrs, chosen.source, chosen.tensor_idx)
            dims = [shape[i] for i in chosen.dim_idx]
            lo = math.prod(d.lower_bound() for d in dims)
            hi = math.prod(d.upper_bound() for d in dims)
            out[name] = sorted({lo, hi})
        return out

    def _extract_exec_path(self, dynamic_profiling_strategy) -> None:
        """Fill attrs["exec_path"]: {profiling key: ExecItem(key, run-time condition, algo="")}."""
        ranges = self._dim_value_ranges()
        if dynamic_profiling_strategy == DynamicProfileStrategy.MAX:
            point = {n: [max(v)] for n, v in ranges.items()}
        elif dynamic_profiling_strategy == DynamicProfileStrategy.MIN:
            point = {n: [min(v)] for n, v in ranges.items()}
        else:
            raise NotImplementedError(
                f"Gemm only supports MIN or MAX dynamic profiling! Current dynamic_profiling_strategy: "
                f"{dynamic_profiling_strategy}"
            )
        item = ExecItem(profiling_key=self._gen_exec_key(point), exec_cond=self._gen_exec_key(ranges), algo="")
        self._attrs["exec_path"] = OrderedDict([(item.profiling_key, item)])

    # ---- profiling -----------------------------------------------------------
    def _registry_key(self, hook: str) -> str:
        return f"{Target.current().name()}.{self._attrs['op']}.{hook}"

    def _get_profiler_filename(self) -> str:
        names = list(self._attrs["op_instance"].keys())
        digest = sha1(";".join(names).encode("utf-8")).hexdigest()
        target = Target.current()
        if target.use_dummy_profiling_results():
            return f"{self._attrs['op']}_{digest}"
        return f"{self._attrs['op']}_{digest}_{target.get_profile_cache_version('gemm')}"

    def _invert_exec_key(self, key: str) -> List[int]:
        return gemm_inverse_key_func(key)

    def _get_ab_alignment(self, exec_key: str) -> int:
        m, n, k = self._invert_exec_key(exec_key)[-3:]
        ab = self._attrs["f_ab_alignment"](m, n, k)
        if not alignment.valid_alignment(ab, self._attrs["inputs"][0].dtype()):
            raise RuntimeError(f"A / B ab_alignment={ab} is not valid! m: {m}, n: {n}, k: {k}.")
        return ab

    def gen_profiler(self, workdir: str = None, dynamic_profiling_strategy=DynamicProfileStrategy.MAX):
        """Prepare profiling: list the kernel instances, derive the workloads, drop instances that
        cannot run them and let the backend provide the profiler executable.
        Returns [(sources, executable)] as the backend reports them."""
        func = registry.get(self._registry_key("config"))
        func(self._attrs, dtype=self._attrs["inputs"][0]._attrs["dtype"])
        self._extract_exec_path(dynamic_profiling_strategy)
        filter_func = registry.get(self._registry_key("filter"))
        kept = OrderedDict()
        for key in self._attrs["exec_path"]:
            ab = self._get_ab_alignment(key)
            for name, inst in self._attrs["op_instance"].items():
                if filter_func(name, self._attrs, ab):
                    kept[name] = inst
        if not kept:
            raise RuntimeError(f"No kernel instance supports {self._attrs['op']} {list(self._attrs['exec_path'])}")
        self._attrs["op_instance"] = kept
        return registry.get(self._registry_key("gen_profiler"))(
            self._attrs, workdir, self._get_profiler_filename(), self._extract_dims(for_profiling=True)
        )

    def _profile_cmd_dims(self, exec_key: str) -> List[int]:
        """Integers appended to the profiler command line for one workload (gemm: M N K)."""
        return self._invert_exec_key(exec_key)

    def _gen_profile_cmd(self, profiler_prefix: str, profiler_filename: str, exec_key: str) -> List[str]:
        exe = os.path.join(profiler_prefix, profiler_filename)
        if not os.access(exe, os.X_OK):
            raise RuntimeError("Profiler %s is not executable" % exe)
        cmd = [exe] + list(self._attrs["profiler_args"]) + [str(x) for x in self._profile_cmd_dims(exec_key)]
        if self._attrs.get("shape") is not None:
            cmd += [str(x) for x in self._attrs["shape"]]
        return cmd

    def _split_k_search_space(self, M, N, K):
        return {1}  # no split-K on this backend: the launchers take no workspace

    def profile(self, profiler_runner, workdir: str = "./") -> None:
        """Time every workload without a chosen instance, or pick by heuristic when profiling is off."""
        target = Target.current()
        prefix = os.path.join(workdir, "profiler", self._attrs["op"])
        filename = self._get_profiler_filename()
        for key, item in self._attrs["exec_path"].items():
            if item.algo != "" and not target.force_profile():
                continue
            if target.use_dummy_profiling_results() or profiler_runner is None:
                item.algo = registry.get(self._registry_key("select_algo"))(self._attrs, key)
                self._attrs["workspace"] = 0
                continue
            # a workload that was timed before (same op, type, device and instance list) is not timed again
            args = profile_cache_args(self._attrs, key)
            cached = None if args is None or target.force_profile() else target.query_profile_cache("gemm", args)
            if cached is not None and cached[0] in self._attrs["op_instance"]:
                _LOGGER.info("Load profiling result for %s %s from cache: %s", self._attrs["op"], key, cached)
                item.algo = cached[0]
                self._attrs["workspace"] = max(self._attrs["workspace"], cached[1])
                self._attrs["split_k"] = cached[2]
                continue
            cmd = self._gen_profile_cmd(prefix, filename, key)
            profiler_runner.push(cmd, process_result_callback=None, func_attrs=self._attrs,
                                 profiler_filename=filename, exec_key=key, split_k=1)

    # ---- code generation --------------------------------------------------------
    def gen_function(self) -> str:
        return registry.get(self._registry_key("gen_function"))(
            self._attrs, self.exec_cond_template, self._extract_dims()
        )

    def _signature(self) -> str:
        return sha1((self._attrs["op"] + "split_" + str(self._attrs["split_k"])).encode("utf-8")).hexdigest()

    # ---- construction --------------------------------------------------------
    def _align_ab(self, a: Tensor, b: Tensor):
        return a, b

    def _sanity_check(self, a: Tensor, b: Tensor):
        a_shapes = a._attrs["shape"]
        if len(a_shapes) < 2:
            raise RuntimeError(f"gemm operand A should have >= 2 dimensions! Current shape: {a_shapes}.")
        b_shapes = b._attrs["shape"]
        if len(b_shapes) != 2:
            raise RuntimeError(f"gemm operand B should have 2 dimensions! Current shape: {b_shapes}.")
        if not is_same_dtype(a.dtype(), b.dtype()):
            raise RuntimeError(
                f"gemm operand A and B should have the same data type! Current A: {a.dtype()}, B: {b.dtype()}."
            )

    def _finish_call(self, inputs: List[Tensor], output_shape) -> Tensor:
        self._extract_epilogue_alignment(output_shape)
        output = Tensor(output_shape, src_ops={self}, dtype=inputs[0].dtype())
        self._attrs["outputs"] = [output]
        self._attrs["output_accessors"] = [TensorAccessor(output)]
        return output

    def __call__(self, a: Tensor, b: Tensor) -> Tensor:
        a, b = self._align_ab(a, b)
        self._attrs["inputs"] = [a, b]
        self._attrs["input_accessors"] = [TensorAccessor(a), TensorAccessor(b)]
        self._set_depth()
        self._sanity_check(a, b)
        return self._finish_call([a, b], self._infer_shapes(a, b))
