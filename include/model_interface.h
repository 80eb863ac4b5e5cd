/*
 * C ABI of a compiled model library (the <workdir>/<test_name>/test.so that
 * compile_model() produces).  It is kept call-compatible with the reference's
 * static/include/model_interface.h:38-311 so that everything that binds to it
 * (the ctypes `Model` wrapper, python/aitemplate/compiler/model.py:172-1118;
 * fx2ait's AITModelImpl; user C++ code) works unchanged: same function names,
 * same argument lists, same enums and struct layouts, same ownership and
 * error conventions.
 *
 *  - every function returns AITemplateError (0 = success, 1 = failure); no
 *    exception crosses the boundary (reference: static/csrc/model_interface.cpp:25-41);
 *    the failure text is logged to stderr;
 *  - the caller owns input / output / stream memory; the container owns constants,
 *    per-runtime activation memory and workspaces, all allocated at creation
 *    through the allocator, which must outlive the container;
 *  - returned `const char*` names stay valid as long as the container lives;
 *  - Run is thread-safe up to `num_runtimes` concurrent inferences and blocks when
 *    every runtime is busy; constant updates are excluded against running inferences.
 */
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <functional>
#include <numeric>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#define AIT_EXPORT __attribute__((__visibility__("default")))

struct AITemplateModelOpaque {};
using AITemplateModelHandle = AITemplateModelOpaque*;

/* reference: model_interface.h:41-44 */
enum class AITemplateError : int {
  AITemplateSuccess = 0,
  AITemplateFailure = 1,
};

#define AIT_ERROR_CHECK(call)                                                                     \
  if ((call) != AITemplateError::AITemplateSuccess) {                                             \
    throw std::runtime_error(std::string(#call " API call failed at ") + __FILE__ + ", line" +    \
                             std::to_string(__LINE__));                                           \
  }

/* reference: model_interface.h:53-65 — a borrowed view of a shape */
struct AITemplateParamShape {
  AITemplateParamShape() : shape_data(nullptr), size(0) {}
  AITemplateParamShape(const int64_t* shape_data_in, size_t size_in) : shape_data(shape_data_in), size(size_in) {}

  const int64_t* shape_data;
  size_t size;

  size_t Numel() const {
    return std::accumulate(shape_data, shape_data + size, (int64_t)1, std::multiplies<int64_t>());
  }
};

/* reference: model_interface.h:67-75 */
enum class AITemplateDtype {
  kUnset = 0,
  kHalf,
  kFloat,
  kInt,
  kLong,
  kBool,
  kBFloat16,
};

/* reference: model_interface.h:77-89 — one tensor handed across the boundary */
struct AITData {
  AITData() : ptr(nullptr), dtype(AITemplateDtype::kUnset) {}
  AITData(void* ptr_in, const AITemplateParamShape& shape_in, AITemplateDtype dtype_in)
      : ptr(ptr_in), shape(shape_in), dtype(dtype_in) {}

  void* ptr;
  AITemplateParamShape shape;
  AITemplateDtype dtype;
};

inline size_t AITemplateDtypeSizeBytes(AITemplateDtype dtype) {
  switch (dtype) {
    case AITemplateDtype::kHalf:
    case AITemplateDtype::kBFloat16:
      return 2;
    case AITemplateDtype::kFloat:
    case AITemplateDtype::kInt:
      return 4;
    case AITemplateDtype::kLong:
      return 8;
    case AITemplateDtype::kBool:
      return 1;
    case AITemplateDtype::kUnset:
      throw std::runtime_error("Unset dtype has no size!");
  }
  throw std::runtime_error("dtype handling is not implemented!");
}

struct AITemplateStreamOpaque {};
using AITemplateStreamHandle = AITemplateStreamOpaque*; /* a hipStream_t */

/* reference: model_interface.h:115-121 — device memory source for the container */
class AITemplateAllocator {
 public:
  virtual void* Allocate(size_t nbytes) = 0;
  virtual void Free(void* ptr) = 0;
  virtual ~AITemplateAllocator() = default;
};

/* reference: model_interface.h:125-131 */
enum class AITemplateAllocatorType {
  kDefault = 0, /* hipMalloc / hipFree */
  kTracking,    /* same, and counts the bytes handed out */
};

extern "C" {

/* reference: model_interface.h:140-146.  allocator == nullptr -> default allocator. */
AIT_EXPORT AITemplateError AITemplateModelContainerCreate(AITemplateModelHandle* ret, size_t num_runtimes,
                                                          AITemplateAllocator* allocator = nullptr);
AIT_EXPORT AITemplateError AITemplateModelContainerDelete(AITemplateModelHandle handle);

/* reference: model_interface.h:148-170 — bind device memory to an unbound constant */
AIT_EXPORT AITemplateError AITemplateModelContainerSetConstant(AITemplateModelHandle handle, const char* name,
                                                               const AITData* tensor);
AIT_EXPORT AITemplateError AITemplateModelContainerSetManyConstants(AITemplateModelHandle handle,
                                                                    const char** names, const AITData* tensors,
                                                                    size_t num_tensors);
AIT_EXPORT AITemplateError AITemplateModelContainerSetDoubleBufferConstant(AITemplateModelHandle handle,
                                                                           AITemplateStreamHandle stream_handle,
                                                                           const char* name, const AITData* tensor);
AIT_EXPORT AITemplateError AITemplateModelContainerSetManyDoubleBufferConstants(
    AITemplateModelHandle handle, AITemplateStreamHandle stream_handle, const char** names, const AITData* tensors,
    size_t num_tensors);

/* reference: model_interface.h:172-192 */
AIT_EXPORT AITemplateError AITemplateModelContainerGetNumConstants(AITemplateModelHandle handle,
                                                                   bool unbound_constants_only,
                                                                   bool constant_folding_inputs_only,
                                                                   size_t* num_constants_out);
AIT_EXPORT AITemplateError AITemplateModelContainerGetConstantNames(AITemplateModelHandle handle,
                                                                    bool unbound_constants_only,
                                                                    bool constant_folding_inputs_only,
                                                                    const char** constant_names_out);
AIT_EXPORT AITemplateError AITemplateModelContainerGetConstantDtype(AITemplateModelHandle handle, const char* name,
                                                                    AITemplateDtype* dtype);
AIT_EXPORT AITemplateError AITemplateModelContainerGetConstantOriginalName(AITemplateModelHandle handle,
                                                                           const char* name,
                                                                           const char** original_name_out);

/* reference: model_interface.h:194-217.  output_shapes_out[i] is caller-allocated with the
 * rank of output i; may be nullptr. */
AIT_EXPORT AITemplateError AITemplateModelContainerRun(AITemplateModelHandle handle, const AITData* inputs,
                                                       size_t num_inputs, AITData* outputs, size_t num_outputs,
                                                       AITemplateStreamHandle stream_handle, bool sync,
                                                       bool graph_mode, int64_t** output_shapes_out);
AIT_EXPORT AITemplateError AITemplateModelContainerRunWithOutputsOnHost(
    AITemplateModelHandle handle, const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs,
    AITemplateStreamHandle stream_handle, bool graph_mode, int64_t** output_shapes_out);

/* reference: model_interface.h:219-242 */
AIT_EXPORT AITemplateError AITemplateModelContainerProfile(AITemplateModelHandle handle, const AITData* inputs,
                                                           size_t num_inputs, AITData* outputs, size_t num_outputs,
                                                           AITemplateStreamHandle stream_handle, size_t num_iters,
                                                           const char* filename);
AIT_EXPORT AITemplateError AITemplateModelContainerBenchmark(
    AITemplateModelHandle handle, const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs,
    AITemplateStreamHandle stream_handle, bool graph_mode, size_t count, size_t num_threads,
    bool use_unique_stream_per_thread, float* runtime_ms, int64_t** output_shapes_out);

/* reference: model_interface.h:244-284 */
AIT_EXPORT AITemplateError AITemplateModelContainerGetNumInputs(AITemplateModelHandle handle, size_t* num_inputs_out);
AIT_EXPORT AITemplateError AITemplateModelContainerGetInputName(AITemplateModelHandle handle, size_t input_idx,
                                                                const char** input_name_out);
AIT_EXPORT AITemplateError AITemplateModelContainerGetMaximumInputShape(AITemplateModelHandle handle,
                                                                        size_t input_idx,
                                                                        AITemplateParamShape* shape);
AIT_EXPORT AITemplateError AITemplateModelContainerGetInputDtype(AITemplateModelHandle handle, size_t input_idx,
                                                                 AITemplateDtype* input_dtype);
AIT_EXPORT AITemplateError AITemplateModelContainerGetNumOutputs(AITemplateModelHandle handle,
                                                                 size_t* num_outputs_out);
AIT_EXPORT AITemplateError AITemplateModelContainerGetOutputName(AITemplateModelHandle handle, size_t output_idx,
                                                                 const char** output_name_out);
AIT_EXPORT AITemplateError AITemplateModelContainerGetMaximumOutputShape(AITemplateModelHandle handle,
                                                                         size_t output_idx,
                                                                         AITemplateParamShape* shape_out);
AIT_EXPORT AITemplateError AITemplateModelContainerGetOutputDtype(AITemplateModelHandle handle, size_t output_idx,
                                                                  AITemplateDtype* out);
AIT_EXPORT AITemplateError AITemplateModelContainerGetNumRuntimes(AITemplateModelHandle handle,
                                                                  size_t* num_runtimes_out);

/* reference: model_interface.h:286-297 */
AIT_EXPORT AITemplateError AITemplateModelContainerFoldConstants(AITemplateModelHandle handle,
                                                                 AITemplateStreamHandle stream_handle, bool sync);
AIT_EXPORT AITemplateError AITemplateModelContainerFoldConstantsInDoubleBuffer(AITemplateModelHandle handle,
                                                                               AITemplateStreamHandle stream_handle,
                                                                               bool sync);
AIT_EXPORT AITemplateError AITemplateModelContainerSwapConstants(AITemplateModelHandle handle);

/* reference: model_interface.h:299-309 */
AIT_EXPORT AITemplateError AITemplateAllocatorCreate(AITemplateAllocator** allocator_out,
                                                     AITemplateAllocatorType allocator_type);
AIT_EXPORT AITemplateError AITemplateAllocatorDelete(AITemplateAllocator* allocator_out);
AIT_EXPORT AITemplateError AITemplateTrackingAllocatorGetNumBytes(AITemplateAllocator* allocator,
                                                                  size_t* num_bytes_out);

/* reference: static/include/utility.h:31-53, static/csrc/utility.cpp:24-69 — device memory helpers
 * used by Model.allocate_gpu_memory / free_gpu_memory / memcpy so a harness needs no torch. */
enum class AITemplateMemcpyKind { HostToDevice = 0, DeviceToHost, DeviceToDevice };
AIT_EXPORT AITemplateError AITemplateDeviceMalloc(void** ptr_out, size_t size,
                                                  AITemplateStreamHandle stream_handle = nullptr, bool sync = true);
AIT_EXPORT AITemplateError AITemplateDeviceFree(void* ptr, AITemplateStreamHandle stream_handle = nullptr,
                                                bool sync = true);
AIT_EXPORT AITemplateError AITemplateMemcpy(void* dst, const void* src, size_t count, AITemplateMemcpyKind kind,
                                            AITemplateStreamHandle stream_handle = nullptr, bool sync = true);

} /* extern "C" */
