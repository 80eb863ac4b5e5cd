// The extern "C" surface: converts every C++ exception into AITemplateFailure + a log line.
#include "model_interface.h"

#include <stdio.h>

#include "model_container.h"

namespace {

ait::DefaultAllocator g_default_allocator;

struct Handle {
  ait::ModelContainer* container;
};

template <class F>
AITemplateError guarded(const char* where, F&& body) {
  try {
    body();
    return AITemplateError::AITemplateSuccess;
  } catch (const std::exception& e) {
    fprintf(stderr, "[aitemplate_amd] Error in %s: %s\n", where, e.what());
  } catch (...) {
    fprintf(stderr, "[aitemplate_amd] Unknown exception in %s\n", where);
  }
  return AITemplateError::AITemplateFailure;
}

ait::ModelContainer& container_of(AITemplateModelHandle handle) {
  if (handle == nullptr) throw std::runtime_error("model handle cannot be null");
  return *reinterpret_cast<ait::ModelContainer*>(handle);
}

template <class T>
T* non_null(T* p, const char* what) {
  if (p == nullptr) throw std::runtime_error(std::string(what) + " cannot be null");
  return p;
}

ait::StreamType as_stream(AITemplateStreamHandle s) { return reinterpret_cast<ait::StreamType>(s); }

}  // namespace

#define GUARDED(body) return guarded(__func__, [&] { body })

extern "C" {

AITemplateError AITemplateModelContainerCreate(AITemplateModelHandle* ret, size_t num_runtimes,
                                               AITemplateAllocator* allocator) {
  GUARDED(
    non_null(ret, "ret");
    AITemplateAllocator& alloc = allocator != nullptr ? *allocator : g_default_allocator;
    *ret = reinterpret_cast<AITemplateModelHandle>(new ait::ModelContainer(num_runtimes, alloc));
  );
}

AITemplateError AITemplateModelContainerDelete(AITemplateModelHandle handle) {
  GUARDED(
    if (handle != nullptr) delete reinterpret_cast<ait::ModelContainer*>(handle);
  );
}

AITemplateError AITemplateModelContainerSetConstant(AITemplateModelHandle handle, const char* name,
                                                    const AITData* tensor) {
  GUARDED(container_of(handle).SetConstant(name, *non_null(tensor, "tensor"), false, nullptr););
}

AITemplateError AITemplateModelContainerSetManyConstants(AITemplateModelHandle handle, const char** names,
                                                         const AITData* tensors, size_t num_tensors) {
  GUARDED(
    auto& c = container_of(handle);
    if (num_tensors > 0) {
      non_null(names, "names");
      non_null(tensors, "tensors");
    }
    for (size_t i = 0; i < num_tensors; ++i) c.SetConstant(names[i], tensors[i], false, nullptr);
  );
}

AITemplateError AITemplateModelContainerSetDoubleBufferConstant(AITemplateModelHandle handle,
                                                                AITemplateStreamHandle stream_handle,
                                                                const char* name, const AITData* tensor) {
  GUARDED(container_of(handle).SetConstant(name, *non_null(tensor, "tensor"), true, as_stream(stream_handle)););
}

AITemplateError AITemplateModelContainerSetManyDoubleBufferConstants(AITemplateModelHandle handle,
                                                                     AITemplateStreamHandle stream_handle,
                                                                     const char** names, const AITData* tensors,
                                                                     size_t num_tensors) {
  GUARDED(
    auto& c = container_of(handle);
    if (num_tensors > 0) {
      non_null(names, "names");
      non_null(tensors, "tensors");
    }
    for (size_t i = 0; i < num_tensors; ++i) c.SetConstant(names[i], tensors[i], true, as_stream(stream_handle));
  );
}

AITemplateError AITemplateModelContainerGetNumConstants(AITemplateModelHandle handle, bool unbound_constants_only,
                                                        bool constant_folding_inputs_only,
                                                        size_t* num_constants_out) {
  GUARDED(*non_null(num_constants_out, "num_constants_out") =
              container_of(handle).GetNumConstants(unbound_constants_only, constant_folding_inputs_only););
}

AITemplateError AITemplateModelContainerGetConstantNames(AITemplateModelHandle handle, bool unbound_constants_only,
                                                         bool constant_folding_inputs_only,
                                                         const char** constant_names_out) {
  GUARDED(
    auto& c = container_of(handle);
    if (c.GetNumConstants(unbound_constants_only, constant_folding_inputs_only) > 0)
      non_null(constant_names_out, "constant_names_out");
    c.WriteAllConstantNamesTo(constant_names_out, unbound_constants_only, constant_folding_inputs_only);
  );
}

AITemplateError AITemplateModelContainerGetConstantDtype(AITemplateModelHandle handle, const char* name,
                                                         AITemplateDtype* dtype) {
  GUARDED(*non_null(dtype, "dtype") = container_of(handle).ConstantDtype(name););
}

AITemplateError AITemplateModelContainerGetConstantOriginalName(AITemplateModelHandle handle, const char* name,
                                                                const char** original_name_out) {
  GUARDED(*non_null(original_name_out, "original_name_out") = container_of(handle).ConstantOriginalName(name););
}

AITemplateError AITemplateModelContainerRun(AITemplateModelHandle handle, const AITData* inputs, size_t num_inputs,
                                            AITData* outputs, size_t num_outputs,
                                            AITemplateStreamHandle stream_handle, bool sync, bool graph_mode,
                                            int64_t** output_shapes_out) {
  GUARDED(container_of(handle).Run(inputs, num_inputs, outputs, num_outputs, as_stream(stream_handle), sync,
                                   graph_mode, output_shapes_out););
}

AITemplateError AITemplateModelContainerRunWithOutputsOnHost(AITemplateModelHandle handle, const AITData* inputs,
                                                             size_t num_inputs, AITData* outputs,
                                                             size_t num_outputs,
                                                             AITemplateStreamHandle stream_handle, bool graph_mode,
                                                             int64_t** output_shapes_out) {
  GUARDED(container_of(handle).RunWithOutputsOnHost(inputs, num_inputs, outputs, num_outputs,
                                                    as_stream(stream_handle), graph_mode, output_shapes_out););
}

AITemplateError AITemplateModelContainerProfile(AITemplateModelHandle handle, const AITData* inputs,
                                                size_t num_inputs, AITData* outputs, size_t num_outputs,
                                                AITemplateStreamHandle stream_handle, size_t num_iters,
                                                const char* filename) {
  GUARDED(container_of(handle).Profile(inputs, num_inputs, outputs, num_outputs, as_stream(stream_handle), num_iters,
                                       filename););
}

AITemplateError AITemplateModelContainerBenchmark(AITemplateModelHandle handle, const AITData* inputs,
                                                  size_t num_inputs, AITData* outputs, size_t num_outputs,
                                                  AITemplateStreamHandle stream_handle, bool graph_mode,
                                                  size_t count, size_t num_threads,
                                                  bool use_unique_stream_per_thread, float* runtime_ms,
                                                  int64_t** output_shapes_out) {
  GUARDED(*non_null(runtime_ms, "runtime_ms") = container_of(handle).Benchmark(
              inputs, num_inputs, outputs, num_outputs, as_stream(stream_handle), graph_mode, count, num_threads,
              use_unique_stream_per_thread, output_shapes_out););
}

AITemplateError AITemplateModelContainerGetNumInputs(AITemplateModelHandle handle, size_t* num_inputs_out) {
  GUARDED(*non_null(num_inputs_out, "num_inputs_out") = container_of(handle).NumInputs(););
}
AITemplateError AITemplateModelContainerGetInputName(AITemplateModelHandle handle, size_t input_idx,
                                                     const char** input_name_out) {
  GUARDED(*non_null(input_name_out, "input_name_out") = container_of(handle).InputName(input_idx););
}
AITemplateError AITemplateModelContainerGetMaximumInputShape(AITemplateModelHandle handle, size_t input_idx,
                                                             AITemplateParamShape* shape) {
  GUARDED(*non_null(shape, "shape") = container_of(handle).MaxInputShape(input_idx););
}
AITemplateError AITemplateModelContainerGetInputDtype(AITemplateModelHandle handle, size_t input_idx,
                                                      AITemplateDtype* input_dtype) {
  GUARDED(*non_null(input_dtype, "input_dtype") = container_of(handle).InputDtype(input_idx););
}
AITemplateError AITemplateModelContainerGetNumOutputs(AITemplateModelHandle handle, size_t* num_outputs_out) {
  GUARDED(*non_null(num_outputs_out, "num_outputs_out") = container_of(handle).NumOutputs(););
}
AITemplateError AITemplateModelContainerGetOutputName(AITemplateModelHandle handle, size_t output_idx,
                                                      const char** output_name_out) {
  GUARDED(*non_null(output_name_out, "output_name_out") = container_of(handle).OutputName(output_idx););
}
AITemplateError AITemplateModelContainerGetMaximumOutputShape(AITemplateModelHandle handle, size_t output_idx,
                                                              AITemplateParamShape* shape_out) {
  GUARDED(*non_null(shape_out, "shape_out") = container_of(handle).MaxOutputShape(output_idx););
}
AITemplateError AITemplateModelContainerGetOutputDtype(AITemplateModelHandle handle, size_t output_idx,
                                                       AITemplateDtype* out) {
  GUARDED(*non_null(out, "out") = container_of(handle).OutputDtype(output_idx););
}
AITemplateError AITemplateModelContainerGetNumRuntimes(AITemplateModelHandle handle, size_t* num_runtimes_out) {
  GUARDED(*non_null(num_runtimes_out, "num_runtimes_out") = container_of(handle).GetNumRuntimes(););
}

AITemplateError AITemplateModelContainerFoldConstants(AITemplateModelHandle handle,
                                                      AITemplateStreamHandle stream_handle, bool sync) {
  GUARDED(container_of(handle).FoldConstants(as_stream(stream_handle), sync, false););
}
AITemplateError AITemplateModelContainerFoldConstantsInDoubleBuffer(AITemplateModelHandle handle,
                                                                    AITemplateStreamHandle stream_handle,
                                                                    bool sync) {
  GUARDED(container_of(handle).FoldConstants(as_stream(stream_handle), sync, true););
}
AITemplateError AITemplateModelContainerSwapConstants(AITemplateModelHandle handle) {
  GUARDED(container_of(handle).SwapConstants(););
}

AITemplateError AITemplateAllocatorCreate(AITemplateAllocator** allocator_out,
                                          AITemplateAllocatorType allocator_type) {
  GUARDED(
    non_null(allocator_out, "allocator_out");
    switch (allocator_type) {
      case AITemplateAllocatorType::kDefault:
        *allocator_out = new ait::DefaultAllocator();
        break;
      case AITemplateAllocatorType::kTracking:
        *allocator_out = new ait::TrackingAllocator();
        break;
      default:
        throw std::runtime_error("Unrecognized allocator type");
    }
  );
}
AITemplateError AITemplateAllocatorDelete(AITemplateAllocator* allocator) {
  GUARDED(delete allocator;);
}
AITemplateError AITemplateTrackingAllocatorGetNumBytes(AITemplateAllocator* allocator, size_t* num_bytes_out) {
  GUARDED(
    non_null(allocator, "allocator");
    auto* t = dynamic_cast<ait::TrackingAllocator*>(allocator);
    if (t == nullptr) throw std::runtime_error("Allocator was not a tracking allocator!");
    *non_null(num_bytes_out, "num_bytes_out") = t->NumBytesAllocated();
  );
}

AITemplateError AITemplateDeviceMalloc(void** ptr_out, size_t size, AITemplateStreamHandle stream_handle, bool sync) {
  GUARDED(
    non_null(ptr_out, "ptr_out");
    AIT_DEVICE_CHECK(hipMallocAsync(ptr_out, size, as_stream(stream_handle)));
    if (sync) AIT_DEVICE_CHECK(hipStreamSynchronize(as_stream(stream_handle)));
  );
}
AITemplateError AITemplateDeviceFree(void* ptr, AITemplateStreamHandle stream_handle, bool sync) {
  GUARDED(
    AIT_DEVICE_CHECK(hipFreeAsync(ptr, as_stream(stream_handle)));
    if (sync) AIT_DEVICE_CHECK(hipStreamSynchronize(as_stream(stream_handle)));
  );
}
AITemplateError AITemplateMemcpy(void* dst, const void* src, size_t count, AITemplateMemcpyKind kind,
                                 AITemplateStreamHandle stream_handle, bool sync) {
  GUARDED(
    hipMemcpyKind k = hipMemcpyDeviceToDevice;
    switch (kind) {
      case AITemplateMemcpyKind::HostToDevice: k = hipMemcpyHostToDevice; break;
      case AITemplateMemcpyKind::DeviceToHost: k = hipMemcpyDeviceToHost; break;
      case AITemplateMemcpyKind::DeviceToDevice: k = hipMemcpyDeviceToDevice; break;
      default: throw std::runtime_error("Unrecognized memcpy kind");
    }
    AIT_DEVICE_CHECK(hipMemcpyAsync(dst, src, count, k, as_stream(stream_handle)));
    if (sync) AIT_DEVICE_CHECK(hipStreamSynchronize(as_stream(stream_handle)));
  );
}

}  // extern "C"
