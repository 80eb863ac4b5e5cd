"""compile_model(): graph -> profiled kernel choices -> generated sources -> shared library -> Model.

Counterpart of python/aitemplate/compiler/compiler.py:147-354.  The signature is the
reference's; the pass pipeline is reduced to what a GEMM-family graph needs (the fused ops are
called directly, as the reference's unit tests do): toposort, naming, parameter / alias
marking, profiling, function de-duplication, memory planning, code generation, build."""
from __future__ import annotations

import logging
import os
from typing import Dict, List, Optional, Union

from ..backend import builder as builder_mod
from ..backend import codegen
from ..backend.target import Target
from ..utils import environ
from . import transform
from .base import ConstantTensorData, DynamicProfileStrategy, Tensor
from .model import Model, TorchTensor
from .transform.name_graph import reset_name_counters

_LOGGER = logging.getLogger(__name__)


def _bind_constants(graph: List[Tensor], constants: Optional[Dict[str, "TorchTensor"]]) -> None:
    if not constants:
        return
    by_name = {t._attrs["name"]: t for t in graph if t._attrs["name"] is not None}
    for name, value in constants.items():
        if name not in by_name:
            raise ValueError(f"constant {name} is not a tensor of the graph")
        t = by_name[name]
        if t._attrs["is_input"] or t.src_ops():
            raise ValueError(f"{name} is not a constant tensor")
        data = value if isinstance(value, ConstantTensorData) else ConstantTensorData.from_torch(value)
        t._bind_data(data)


def compile_model(
    tensor: Union[Tensor, List[Tensor]],
    target: Target,
    workdir: str,
    test_name: str,
    profile_devs: List[int] = None,
    dynamic_profiling_strategy: DynamicProfileStrategy = DynamicProfileStrategy.MAX,
    dll_name: str = "test.so",
    num_runtimes: int = 1,
    profile_dir: str = None,
    constants: Optional[Dict[str, TorchTensor]] = None,
    allocator_kind=None,
    debug_settings=None,
    do_optimize_graph: bool = True,
    profile_timeout: int = 500,
) -> Model:
    """Compile the graph ending in `tensor` and return a loaded Model.

    The library is written to <workdir>/<test_name>/<dll_name>.  With AIT_RECOMPILE=0 nothing
    is regenerated and the existing library is loaded."""
    from ..backend import rocm as _rocm_backend  # noqa: F401  (registers the rocm.* hooks)

    output_tensors = [tensor] if isinstance(tensor, Tensor) else list(tensor)
    for t in output_tensors:
        if not t._attrs["is_output"]:
            raise ValueError(f"tensor {t._attrs['name']} passed to compile_model is not marked is_output")
    test_name = test_name.replace(",", "_")
    test_dir = os.path.join(workdir, test_name)
    lib_path = os.path.join(test_dir, dll_name)
    if profile_dir is None:
        profile_dir = workdir
    if environ.recompile():
        os.makedirs(test_dir, exist_ok=True)
        with target:
            reset_name_counters()
            graph = transform.toposort(output_tensors)
            _bind_constants(graph, constants)
            if do_optimize_graph:
                graph = transform.fuse_mm_elementwise(graph, output_tensors)
            transform.check_leftover_elementwise(graph)
            # last-dim split / concatenate become offsets and row pitches of the GEMM ops around them
            graph = transform.fuse_strided_views(graph, output_tensors)
            transform.name_graph(graph)
            transform.mark_param_tensor(graph, output_tensors)
            transform.profile(graph, profile_dir, profile_devs, dynamic_profiling_strategy, profile_timeout)
            transform.refine_graph(graph)
            blob, workspace = transform.memory_planning(graph)
            file_pairs = codegen.gen_function_src(graph, workdir, test_name)
            file_pairs += codegen.gen_library_src(graph, blob, workspace, workdir, output_tensors, test_name)
            builder_mod.Builder().make(file_pairs, dll_name, workdir, test_name, debug_settings)
    elif not os.path.exists(lib_path):
        raise RuntimeError(f"AIT_RECOMPILE=0 but {lib_path} does not exist")
    module = Model(lib_path, num_runtimes, allocator_kind)
    return module
