// Runtime side of one compiled model instance ("runtime").
//
// The generated model source derives `Model` from ModelBase, fills the parameter
// table with pointers to its own dim members, and appends one OpEntry per graph
// op whose body calls the per-op launch function.  Everything else - input /
// output binding with shape-range checks, activation and workspace memory,
// constant binding, stream-ordered completion tracking, optional hipGraph
// replay, per-op profiling - lives here, prebuilt in libaitemplate_amd_runtime.a,
// so building a model compiles only a few lines of host C++.
//
// Role in the reference: static/include/model.h:48-323 (ModelBase<T>, CRTP and
// compiled per model) plus the generated class of backend/main_templates.py:21-335.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <functional>
#include <string>
#include <unordered_map>
#include <vector>

#include "model_interface.h"

namespace ait {

using StreamType = hipStream_t;

// throws std::runtime_error carrying the HIP error text and the call site
void DeviceCheck(hipError_t err, const char* what, const char* file, int line);
#define AIT_DEVICE_CHECK(call) ::ait::DeviceCheck((call), #call, __FILE__, __LINE__)
// after a kernel launch
void DeviceCheckLastError(const char* file, int line);

// One dimension of a parameter: its legal inclusive range and where the current
// value is stored (a member of the generated Model that the op launchers read).
struct ParamDim {
  ParamDim(int64_t lower, int64_t upper, int64_t* value) : lower_bound(lower), upper_bound(upper), value(value) {}
  int64_t lower_bound;
  int64_t upper_bound;
  int64_t* value;
};

struct ParamInfo {
  void* ptr = nullptr;
  const char* name = "";
  std::vector<ParamDim> shape_ptrs;
};

struct OpEntry {
  std::string name;
  std::function<void(StreamType)> launch;
};

// Static description of the compiled graph, defined by the generated source.
struct TensorMeta {
  std::string name;
  AITemplateDtype dtype;
  std::vector<int64_t> max_shape;
};
struct ConstantMeta {
  std::string name;
  std::string original_name;
  AITemplateDtype dtype;
  std::vector<int64_t> shape;
  bool bound;        // bytes live in the library's constant blob
  size_t offset;     // into the constant blob (bound constants)
  size_t num_bytes;
};
struct ModelMeta {
  std::vector<TensorMeta> inputs;
  std::vector<TensorMeta> outputs;
  std::vector<ConstantMeta> constants;
  size_t blob_size = 0;          // activation memory per runtime
  size_t workspace_size = 0;     // shared op workspace per runtime
  size_t constants_size = 0;     // bytes of the bound-constant blob
  const uint8_t* constants_begin = nullptr;  // host image of the blob embedded in the library
  const uint8_t* constants_end = nullptr;
};

class ModelBase {
 public:
  ModelBase(size_t blob_size, size_t workspace_size, size_t num_inputs, size_t num_outputs,
            size_t num_unbound_constants, uint8_t* constants, AITemplateAllocator& allocator);
  virtual ~ModelBase();
  ModelBase(const ModelBase&) = delete;
  ModelBase& operator=(const ModelBase&) = delete;

  // `mark_finished` = false leaves out the completion event (callers that run a batch and mark its end once)
  void Run(StreamType stream, bool graph_mode, bool mark_finished = true);
  void MarkFinished(StreamType stream);
  void Profile(StreamType stream, size_t iters, const std::string& filename);
  bool IsPending();
  void WaitForCompletion();

  size_t NumInputs() const { return num_inputs_; }
  size_t NumOutputs() const { return num_outputs_; }

  void SetInput(const void* src, const AITemplateParamShape& shape, size_t idx);
  void SetOutput(void* src, size_t idx);
  // writes the current shape of output idx; output must have max-rank entries
  void GetOutputShape(size_t idx, int64_t* output_shape_out);
  void SetConstant(const char* name, const void* src);
  uint8_t* GetConstantsBlob() const { return constants_; }
  void SetConstantsBlob(uint8_t* base);

 protected:
  // generated
  virtual void SetUpInputsOutputs() = 0;
  virtual void BindBoundConstants(uint8_t* base) = 0;
  virtual void DeviceToDeviceCopies(StreamType) {}

  void RunImpl(StreamType stream);
  void SetParam(const void* src, size_t param_idx);

  std::vector<ParamInfo> params_;  // inputs, then outputs, then unbound constants
  std::unordered_map<std::string, const void**> constant_name_to_ptr_;
  std::vector<OpEntry> ops_;
  uint8_t* blob_ = nullptr;
  uint8_t* workspace_ = nullptr;
  int64_t workspace_size_ = 0;
  uint8_t* constants_ = nullptr;
  size_t num_inputs_;
  size_t num_outputs_;

 private:
  AITemplateAllocator& allocator_;
  hipEvent_t run_finished_ = nullptr;
  int device_idx_ = 0;
  // hipGraph replay state (graph_mode); re-captured when any bound pointer or dim changes
  hipGraphExec_t graph_exec_ = nullptr;
  StreamType graph_capture_stream_ = nullptr;
  std::vector<uint64_t> graph_signature_;
  std::vector<uint64_t> CurrentSignature() const;
};

}  // namespace ait

// Defined by the generated model source; resolved inside the model library.
extern "C" {
const ait::ModelMeta* aitamd_model_meta();
ait::ModelBase* aitamd_model_create(uint8_t* constants, AITemplateAllocator* allocator);
}
