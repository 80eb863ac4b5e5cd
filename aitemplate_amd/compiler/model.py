"""ctypes wrapper of a compiled model library (the AITemplateModelContainer* C ABI).

Counterpart of python/aitemplate/compiler/model.py:55-1118: same class name, constructor
and method names / argument meaning, so code written against the reference's `Model` works.
Every C call is checked; a non-zero return raises RuntimeError("Error in function: ...").
torch is optional: the *_with_tensors helpers import it lazily, everything else works with
raw pointers (AITData) and the library's own device-memory helpers.
"""
from __future__ import annotations

import ctypes
import enum
import logging
import math
from typing import Any, Callable, Dict, Iterable, List, NamedTuple, Optional, Tuple, TypeVar, Union

import numpy as np

from .dtype import dtype_str_to_enum, get_dtype_size

TorchTensor = TypeVar("TorchTensor")
_LOGGER = logging.getLogger(__name__)


class AITemplateMemcpyKind(enum.Enum):
    HostToDevice = 0
    DeviceToHost = 1
    DeviceToDevice = 2


class AITemplateAllocatorKind(enum.Enum):
    DEFAULT = 0
    TRACKING = 1


class AITData(NamedTuple):
    """A tensor handed to Model.run: device pointer, shape, dtype name."""

    data_ptr: int
    shape: List[int]
    dtype: str


class _AITemplateShape(ctypes.Structure):
    _fields_ = [("shape_data", ctypes.POINTER(ctypes.c_longlong)), ("size", ctypes.c_size_t)]


class _CFormatAITData(ctypes.Structure):
    _fields_ = [("pointer", ctypes.c_void_p), ("shape", _AITemplateShape), ("dtype", ctypes.c_int)]


_ENUM_TO_DTYPE = {1: "float16", 2: "float32", 3: "int32", 4: "int64", 5: "bool", 6: "bfloat16"}


def _dlclose(dll: ctypes.CDLL) -> None:
    try:
        libc = ctypes.CDLL(None)
        libc.dlclose.argtypes = [ctypes.c_void_p]
        libc.dlclose(dll._handle)
    except Exception:  # pragma: no cover
        _LOGGER.warning("dlclose was not found, the model library stays mapped")


def _check_tensors(tensor_list, is_error_fn: Callable[[Any], bool], list_name: str, condition: str) -> None:
    if isinstance(tensor_list, dict):
        tensor_list = tensor_list.values()
    for i, t in enumerate(tensor_list):
        if is_error_fn(t):
            raise ValueError(f"{list_name}[{i}] failed check: {condition}")


def _check_tensors_contiguous_and_on_gpu(tensors, name: str) -> None:
    _check_tensors(tensors, lambda t: not t.is_contiguous() or not t.is_cuda, name, "contiguous and on GPU")


def _check_tensors_contiguous_and_on_host(tensors, name: str) -> None:
    _check_tensors(tensors, lambda t: not t.is_contiguous() or t.is_cuda, name, "contiguous and on host")


def torch_dtype_to_string(dtype) -> str:
    import torch

    return {torch.float16: "float16", torch.bfloat16: "bfloat16", torch.float32: "float32",
            torch.int32: "int32", torch.int64: "int64", torch.bool: "bool"}[dtype]


def torch_to_ait_data(tensor) -> AITData:
    return AITData(tensor.data_ptr(), list(tensor.size()), torch_dtype_to_string(tensor.dtype))


def _convert_tensor_args(params):
    if isinstance(params, dict):
        return {name: torch_to_ait_data(t) for name, t in params.items()}
    return [torch_to_ait_data(t) for t in params]


def _reshape_tensor(tensor, shape: List[int]):
    """View the leading prod(shape) elements of an over-allocated output as `shape`."""
    assert tensor.ndim == len(shape), f"Expected output tensor's ndim to match the length of Run()'s return value: {tensor.ndim} != {len(shape)}"
    numel = math.prod(shape)
    return tensor.flatten()[:numel].reshape(shape)


class Model:
    class _DLLWrapper:
        """The loaded model library.  Looking up an exported function returns a callable that raises when the
        function reports a non-zero AITemplateError; once closed, every lookup raises."""

        def __init__(self, lib_path: str):
            self.lib_path = lib_path
            self.DLL = ctypes.cdll.LoadLibrary(lib_path)
            self.is_open = True
            self._checked = {}

        def close(self):
            if not self.is_open:
                return
            self.is_open = False
            self._checked.clear()
            _dlclose(self.DLL)

        def _make_checked(self, name: str):
            c_func = getattr(self.DLL, name)

            def call(*args):
                if c_func(*args) != 0:
                    raise RuntimeError(f"Error in function: {name}")

            call.__name__ = name
            return call

        def __getattr__(self, name):
            # only reached for names that are not instance attributes, i.e. the library's symbols
            if name.startswith("__") or not self.__dict__.get("is_open", False):
                if name.startswith("__"):
                    raise AttributeError(name)
                raise RuntimeError(f"Cannot use closed AIT library: {self.__dict__.get('lib_path')}")
            fn = self._checked.get(name)
            if fn is None:
                fn = self._checked[name] = self._make_checked(name)
            return fn

    def __init__(self, lib_path: str, num_runtimes: int = 1,
                 allocator_kind: Optional[AITemplateAllocatorKind] = None):
        """Load <lib_path> and create a container with `num_runtimes` concurrent runtimes."""
        self.lib_path = lib_path
        self.DLL = self._DLLWrapper(lib_path)
        self.handle = ctypes.c_void_p()
        self.allocator_handle = ctypes.c_void_p()
        # tensors bound as constants are referenced here until replaced, so that their memory outlives
        # the caller's variables (reference: compiler/model.py:246,874-910)
        self.torch_constant_tensors = {}
        if num_runtimes <= 0:
            raise ValueError(f"num_runtimes must be positive, but got {num_runtimes}")
        if allocator_kind is not None:
            self.DLL.AITemplateAllocatorCreate(ctypes.byref(self.allocator_handle), ctypes.c_int(allocator_kind.value))
        self.DLL.AITemplateModelContainerCreate(ctypes.pointer(self.handle), ctypes.c_size_t(num_runtimes),
                                                self.allocator_handle)
        self._input_name_to_index = self._construct_input_name_to_index_map()
        self._output_name_to_index = self._construct_output_name_to_index_map()
        self._output_ndims = [len(self.get_output_maximum_shape(i)) for i in range(len(self._output_name_to_index))]

    def __enter__(self):
        return self

    def __exit__(self, *args):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def close(self):
        """Delete the container (and its allocator) and unmap the library; further use raises."""
        if getattr(self, "DLL", None) is not None and self.DLL.is_open:
            if self.handle:
                self.DLL.AITemplateModelContainerDelete(self.handle)
                self.handle = ctypes.c_void_p()
            if self.allocator_handle:
                self.DLL.AITemplateAllocatorDelete(self.allocator_handle)
                self.allocator_handle = ctypes.c_void_p()
            self.DLL.close()

    def __getstate__(self):
        return {"lib_path": self.lib_path}

    def __setstate__(self, d):
        if "lib_path" not in d:
            raise RuntimeError(f"Didn't find 'lib_path' property in {d}")
        self.__init__(d["lib_path"])

    # ---- marshalling ---------------------------------------------------------------
    def _convert_single_param_to_c_format(self, param: AITData) -> _CFormatAITData:
        pointer, shape, dtype = param
        c_pointer = ctypes.c_void_p(pointer)
        c_shape_data = (ctypes.c_longlong * len(shape))(*[int(s) for s in shape])
        c_shape = _AITemplateShape(c_shape_data, ctypes.c_size_t(len(shape)))
        return _CFormatAITData(c_pointer, c_shape, dtype_str_to_enum(dtype))

    def _convert_params_to_c_format(self, params: List[AITData]):
        return (_CFormatAITData * len(params))(*[self._convert_single_param_to_c_format(p) for p in params])

    def _prepare_run(self, inputs, outputs, stream_ptr):
        c_inputs = self._convert_params_to_c_format(inputs)
        c_outputs = self._convert_params_to_c_format(outputs)
        c_stream = ctypes.c_void_p() if stream_ptr is None else ctypes.c_void_p(stream_ptr)
        num_outputs = len(self._output_ndims)
        c_output_shapes_out = (ctypes.POINTER(ctypes.c_int64) * num_outputs)()
        for i in range(num_outputs):
            c_output_shapes_out[i] = ctypes.cast((ctypes.c_int64 * self._output_ndims[i])(), ctypes.POINTER(ctypes.c_int64))
        return c_inputs, c_outputs, c_stream, c_output_shapes_out

    def _dict_to_ordered_list(self, params, is_inputs):
        mapping = self._input_name_to_index if is_inputs else self._output_name_to_index
        if len(params) != len(mapping):
            raise ValueError(f"Did not get correct number of {'inputs' if is_inputs else 'outputs'} expected "
                             f"{len(mapping)}, got {len(params)}")
        result = [None] * len(mapping)
        for name, tensor in params.items():
            if name not in mapping:
                raise ValueError(f"Got unexpected {'input' if is_inputs else 'output'}: {name}")
            result[mapping[name]] = tensor
        return result

    def _make_ait_outputs(self, outputs: List[AITData], c_output_shapes) -> Dict[str, AITData]:
        out = {}
        for name, idx in self._output_name_to_index.items():
            shape = [int(c_output_shapes[idx][j]) for j in range(self._output_ndims[idx])]
            out[name] = AITData(outputs[idx].data_ptr, shape, outputs[idx].dtype)
        return out

    # ---- run ------------------------------------------------------------------------
    def _run_impl(self, inputs, outputs, stream_ptr=None, sync=True, graph_mode=False, outputs_on_host=False):
        if isinstance(inputs, dict):
            inputs = self._dict_to_ordered_list(inputs, is_inputs=True)
        if isinstance(outputs, dict):
            outputs = self._dict_to_ordered_list(outputs, is_inputs=False)
        c_inputs, c_outputs, c_stream, c_shapes = self._prepare_run(inputs, outputs, stream_ptr)
        if not outputs_on_host:
            self.DLL.AITemplateModelContainerRun(self.handle, c_inputs, ctypes.c_size_t(len(inputs)), c_outputs,
                                                 ctypes.c_size_t(len(outputs)), c_stream, ctypes.c_bool(sync),
                                                 ctypes.c_bool(graph_mode), c_shapes)
        else:
            self.DLL.AITemplateModelContainerRunWithOutputsOnHost(
                self.handle, c_inputs, ctypes.c_size_t(len(inputs)), c_outputs, ctypes.c_size_t(len(outputs)),
                c_stream, ctypes.c_bool(graph_mode), c_shapes)
        return self._make_ait_outputs(outputs, c_shapes)

    def run(self, inputs, outputs, stream_ptr: Optional[int] = None, sync: bool = True,
            graph_mode: bool = False) -> Dict[str, AITData]:
        """Run the model on AITData inputs / outputs (lists in index order, or dicts by name).
        Outputs must hold their maximum size; the returned AITData carry the actual shapes."""
        return self._run_impl(inputs, outputs, stream_ptr, sync, graph_mode, outputs_on_host=False)

    def _interpret_tensors_as_shapes(self, outputs, outputs_ait: Dict[str, AITData]):
        if isinstance(outputs, dict):
            return {name: _reshape_tensor(t, outputs_ait[name].shape) for name, t in outputs.items()}
        return {name: _reshape_tensor(outputs[idx], outputs_ait[name].shape)
                for name, idx in self._output_name_to_index.items()}

    def run_with_tensors(self, inputs, outputs, stream_ptr: Optional[int] = None, sync: bool = True,
                         graph_mode: bool = False):
        """Run with torch tensors (contiguous, on the GPU).  When no stream is given the current
        torch stream is used so that the call is ordered with surrounding torch work."""
        _check_tensors_contiguous_and_on_gpu(inputs, name="inputs")
        _check_tensors_contiguous_and_on_gpu(outputs, name="outputs")
        if stream_ptr is None:
            stream_ptr = self._current_torch_stream()
        outputs_ait = self.run(_convert_tensor_args(inputs), _convert_tensor_args(outputs), stream_ptr=stream_ptr,
                               sync=sync, graph_mode=graph_mode)
        return self._interpret_tensors_as_shapes(outputs, outputs_ait)

    @staticmethod
    def _current_torch_stream() -> Optional[int]:
        try:
            import torch

            return torch.cuda.current_stream().cuda_stream or None
        except Exception:
            return None

    def _run_with_outputs_on_host(self, inputs, outputs, stream_ptr=None, graph_mode=False):
        return self._run_impl(inputs, outputs, stream_ptr, graph_mode=graph_mode, outputs_on_host=True)

    def _run_with_tensors_outputs_on_host(self, inputs, outputs, stream_ptr=None, graph_mode=False):
        _check_tensors_contiguous_and_on_gpu(inputs, name="inputs")
        _check_tensors_contiguous_and_on_host(outputs, name="outputs")
        output_shapes = self._run_with_outputs_on_host(_convert_tensor_args(inputs), _convert_tensor_args(outputs),
                                                       stream_ptr=stream_ptr, graph_mode=graph_mode)
        return self._interpret_tensors_as_shapes(outputs, output_shapes)

    def profile(self, inputs, outputs, num_iters: int, filename: str, stream_ptr: Optional[int] = None) -> None:
        """Time every op `num_iters` times and write a JSON report to `filename`."""
        if isinstance(inputs, dict):
            inputs = self._dict_to_ordered_list(inputs, is_inputs=True)
        if isinstance(outputs, dict):
            outputs = self._dict_to_ordered_list(outputs, is_inputs=False)
        c_inputs, c_outputs, c_stream, _ = self._prepare_run(inputs, outputs, stream_ptr)
        self.DLL.AITemplateModelContainerProfile(self.handle, c_inputs, ctypes.c_size_t(len(inputs)), c_outputs,
                                                 ctypes.c_size_t(len(outputs)), c_stream, ctypes.c_size_t(num_iters),
                                                 ctypes.c_char_p(filename.encode("utf-8")))

    def profile_with_tensors(self, inputs, outputs, num_iters: int, filename: str,
                             stream_ptr: Optional[int] = None) -> None:
        _check_tensors_contiguous_and_on_gpu(inputs, name="inputs")
        _check_tensors_contiguous_and_on_gpu(outputs, name="outputs")
        self.profile(_convert_tensor_args(inputs), _convert_tensor_args(outputs), num_iters, filename, stream_ptr)

    def benchmark(self, inputs, outputs, stream_ptr: Optional[int] = None, graph_mode: bool = False,
                  count: int = 10, repeat: int = 1, num_threads: int = 1,
                  use_unique_stream_per_thread: bool = False) -> Tuple[float, float, Dict[str, AITData]]:
        """(mean ms, std ms, outputs) over `repeat` measurements of `count` runs each."""
        if isinstance(inputs, dict):
            inputs = self._dict_to_ordered_list(inputs, is_inputs=True)
        if isinstance(outputs, dict):
            outputs = self._dict_to_ordered_list(outputs, is_inputs=False)
        c_inputs, c_outputs, c_stream, c_shapes = self._prepare_run(inputs, outputs, stream_ptr)
        times = []
        runtime_ms = ctypes.c_float()
        for _ in range(repeat):
            self.DLL.AITemplateModelContainerBenchmark(
                self.handle, c_inputs, ctypes.c_size_t(len(inputs)), c_outputs, ctypes.c_size_t(len(outputs)),
                c_stream, ctypes.c_bool(graph_mode), ctypes.c_size_t(count), ctypes.c_size_t(num_threads),
                ctypes.c_bool(use_unique_stream_per_thread), ctypes.byref(runtime_ms), c_shapes)
            times.append(runtime_ms.value)
        return float(np.mean(times)), float(np.std(times)), self._make_ait_outputs(outputs, c_shapes)

    def benchmark_with_tensors(self, inputs, outputs, stream_ptr: Optional[int] = None, graph_mode: bool = False,
                               count: int = 10, repeat: int = 1, num_threads: int = 1,
                               use_unique_stream_per_thread: bool = False):
        _check_tensors_contiguous_and_on_gpu(inputs, name="inputs")
        _check_tensors_contiguous_and_on_gpu(outputs, name="outputs")
        mean, std, ait_outputs = self.benchmark(_convert_tensor_args(inputs), _convert_tensor_args(outputs),
                                                stream_ptr, graph_mode, count, repeat, num_threads,
                                                use_unique_stream_per_thread)
        return mean, std, self._interpret_tensors_as_shapes(outputs, ait_outputs)

    # ---- metadata -------------------------------------------------------------------
    def _get_map_helper(self, n: int, get_name_func) -> Dict[str, int]:
        result = {}
        for i in range(n):
            c_name = ctypes.c_char_p()
            get_name_func(ctypes.c_size_t(i), ctypes.byref(c_name))
            result[c_name.value.decode("utf-8")] = i
        return result

    def _construct_input_name_to_index_map(self) -> Dict[str, int]:
        num = ctypes.c_size_t()
        self.DLL.AITemplateModelContainerGetNumInputs(self.handle, ctypes.byref(num))
        return self._get_map_helper(num.value, lambda i, out: self.DLL.AITemplateModelContainerGetInputName(self.handle, i, out))

    def get_input_name_to_index_map(self) -> Dict[str, int]:
        return self._input_name_to_index.copy()

    def _construct_output_name_to_index_map(self) -> Dict[str, int]:
        num = ctypes.c_size_t()
        self.DLL.AITemplateModelContainerGetNumOutputs(self.handle, ctypes.byref(num))
        return self._get_map_helper(num.value, lambda i, out: self.DLL.AITemplateModelContainerGetOutputName(self.handle, i, out))

    def get_output_name_to_index_map(self) -> Dict[str, int]:
        return self._output_name_to_index.copy()

    def get_output_maximum_shape(self, output_idx_or_name: Union[int, str]) -> List[int]:
        if isinstance(output_idx_or_name, int):
            idx = output_idx_or_name
        elif isinstance(output_idx_or_name, str):
            if output_idx_or_name not in self._output_name_to_index:
                raise ValueError(f"Name {output_idx_or_name} not in OutputNameToIndexMap! Available names: "
                                 f"{list(self._output_name_to_index.keys())}")
            idx = self._output_name_to_index[output_idx_or_name]
        else:
            raise TypeError(f"output_idx_or_name must be str or int, but got {type(output_idx_or_name)}")
        shape = _AITemplateShape()
        self.DLL.AITemplateModelContainerGetMaximumOutputShape(self.handle, ctypes.c_size_t(idx), ctypes.byref(shape))
        return [int(shape.shape_data[i]) for i in range(shape.size)]

    def get_input_maximum_shape(self, idx: int) -> List[int]:
        shape = _AITemplateShape()
        self.DLL.AITemplateModelContainerGetMaximumInputShape(self.handle, ctypes.c_size_t(idx), ctypes.byref(shape))
        return [int(shape.shape_data[i]) for i in range(shape.size)]

    def get_output_dtype(self, index: int) -> int:
        out = ctypes.c_int()
        self.DLL.AITemplateModelContainerGetOutputDtype(self.handle, ctypes.c_size_t(index), ctypes.byref(out))
        return out.value

    def get_input_dtype(self, index: int) -> int:
        out = ctypes.c_int()
        self.DLL.AITemplateModelContainerGetInputDtype(self.handle, ctypes.c_size_t(index), ctypes.byref(out))
        return out.value

    def get_num_runtimes(self) -> int:
        out = ctypes.c_size_t()
        self.DLL.AITemplateModelContainerGetNumRuntimes(self.handle, ctypes.byref(out))
        return out.value

    # ---- constants --------------------------------------------------------------------
    def set_constant(self, name: str, tensor: AITData) -> None:
        b_name = name.encode("utf-8")
        c_tensor = self._convert_single_param_to_c_format(tensor)
        self.DLL.AITemplateModelContainerSetConstant(self.handle, ctypes.c_char_p(b_name), ctypes.byref(c_tensor))

    def set_many_constants(self, tensors: Dict[str, AITData]) -> None:
        c_names = (ctypes.c_char_p * len(tensors))(*[n.encode("utf-8") for n in tensors])
        c_tensors = self._convert_params_to_c_format(list(tensors.values()))
        self.DLL.AITemplateModelContainerSetManyConstants(self.handle, c_names, c_tensors, ctypes.c_size_t(len(tensors)))

    def set_double_buffer_constant(self, name: str, tensor: AITData, stream_ptr: Optional[int] = None) -> None:
        b_name = name.encode("utf-8")
        c_tensor = self._convert_single_param_to_c_format(tensor)
        self.DLL.AITemplateModelContainerSetDoubleBufferConstant(
            self.handle, ctypes.c_void_p(stream_ptr), ctypes.c_char_p(b_name), ctypes.byref(c_tensor))

    def set_many_double_buffer_constants(self, tensors: Dict[str, AITData], stream_ptr: Optional[int] = None) -> None:
        c_names = (ctypes.c_char_p * len(tensors))(*[n.encode("utf-8") for n in tensors])
        c_tensors = self._convert_params_to_c_format(list(tensors.values()))
        self.DLL.AITemplateModelContainerSetManyDoubleBufferConstants(
            self.handle, ctypes.c_void_p(stream_ptr), c_names, c_tensors, ctypes.c_size_t(len(tensors)))

    def set_constant_with_tensor(self, name: str, tensor) -> None:
        """Bind a torch tensor to a constant; the model keeps using that memory and holds a reference to
        the tensor in `torch_constant_tensors` until it is replaced."""
        _check_tensors_contiguous_and_on_gpu([tensor], name="constant")
        self.set_constant(name, torch_to_ait_data(tensor))
        self.torch_constant_tensors[name] = tensor

    def set_many_constants_with_tensors(self, tensors: Dict[str, Any]) -> None:
        _check_tensors_contiguous_and_on_gpu(tensors, name="constants")
        self.set_many_constants({n: torch_to_ait_data(t) for n, t in tensors.items()})
        self.torch_constant_tensors.update(tensors)

    def set_double_buffer_constant_with_tensor(self, name: str, tensor, stream_ptr: Optional[int] = None) -> None:
        _check_tensors_contiguous_and_on_gpu([tensor], name="constant")
        self.set_double_buffer_constant(name, torch_to_ait_data(tensor), stream_ptr)
        self.torch_constant_tensors[name] = tensor

    def set_many_double_buffer_constants_with_tensors(self, tensors: Dict[str, Any],
                                                      stream_ptr: Optional[int] = None) -> None:
        _check_tensors_contiguous_and_on_gpu(tensors, name="constants")
        self.set_many_double_buffer_constants({n: torch_to_ait_data(t) for n, t in tensors.items()}, stream_ptr)
        self.torch_constant_tensors.update(tensors)

    def fold_constants(self, stream_ptr: Optional[int] = None, sync: bool = True, double_buffer: bool = False) -> None:
        fn = (self.DLL.AITemplateModelContainerFoldConstantsInDoubleBuffer if double_buffer
              else self.DLL.AITemplateModelContainerFoldConstants)
        fn(self.handle, ctypes.c_void_p(stream_ptr), ctypes.c_bool(sync))

    def swap_constants(self) -> None:
        self.DLL.AITemplateModelContainerSwapConstants(self.handle)

    def _get_constant_names_impl(self, unbound_constants_only: bool, constant_folding_only: bool) -> Iterable[str]:
        num = ctypes.c_size_t()
        self.DLL.AITemplateModelContainerGetNumConstants(self.handle, ctypes.c_bool(unbound_constants_only),
                                                         ctypes.c_bool(constant_folding_only), ctypes.byref(num))
        names = (ctypes.c_char_p * num.value)()
        self.DLL.AITemplateModelContainerGetConstantNames(self.handle, ctypes.c_bool(unbound_constants_only),
                                                          ctypes.c_bool(constant_folding_only), names)
        return [n.decode("utf-8") for n in names]

    def get_constant_names(self, unbound_constants_only: bool = True, constant_folding_only: bool = False):
        return self._get_constant_names_impl(unbound_constants_only, constant_folding_only)

    def get_constant_folding_input_names(self, unbound_constants_only: bool = True):
        return self._get_constant_names_impl(unbound_constants_only, True)

    # ---- device memory helpers (no torch needed) ---------------------------------------
    def allocate_gpu_memory(self, nbytes: int, stream_ptr: Optional[int] = None, sync: bool = True) -> int:
        ptr = ctypes.c_void_p()
        self.DLL.AITemplateDeviceMalloc(ctypes.byref(ptr), ctypes.c_size_t(nbytes), ctypes.c_void_p(stream_ptr),
                                        ctypes.c_bool(sync))
        return ptr.value

    def free_gpu_memory(self, ptr: int, stream_ptr: Optional[int] = None, sync: bool = True) -> None:
        self.DLL.AITemplateDeviceFree(ctypes.c_void_p(ptr), ctypes.c_void_p(stream_ptr), ctypes.c_bool(sync))

    def memcpy(self, dst: int, src: int, count: int, kind: AITemplateMemcpyKind, stream_ptr: Optional[int] = None,
               sync: bool = True) -> None:
        self.DLL.AITemplateMemcpy(ctypes.c_void_p(dst), ctypes.c_void_p(src), ctypes.c_size_t(count),
                                  ctypes.c_int(kind.value), ctypes.c_void_p(stream_ptr), ctypes.c_bool(sync))

    def numpy_to_ait_data(self, arr: np.ndarray, stream_ptr: Optional[int] = None, sync: bool = True) -> AITData:
        """Copy a numpy array to freshly allocated device memory (free it with free_gpu_memory)."""
        dtype = str(arr.dtype)
        arr = np.ascontiguousarray(arr)
        nbytes = arr.size * get_dtype_size(dtype)
        gpu = self.allocate_gpu_memory(max(nbytes, 1), stream_ptr, sync)
        if nbytes:
            self.memcpy(gpu, arr.ctypes.data, nbytes, AITemplateMemcpyKind.HostToDevice, stream_ptr, sync)
        return AITData(gpu, list(arr.shape), dtype)

    def ait_data_to_numpy(self, ait_data: AITData, stream_ptr: Optional[int] = None, sync: bool = True) -> np.ndarray:
        arr = np.empty(ait_data.shape, dtype=ait_data.dtype)
        nbytes = arr.size * get_dtype_size(ait_data.dtype)
        if nbytes:
            self.memcpy(arr.ctypes.data, ait_data.data_ptr, nbytes, AITemplateMemcpyKind.DeviceToHost, stream_ptr, sync)
        return arr
