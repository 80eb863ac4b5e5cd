// ModelBase: binding, range checks, run / graph replay / per-op profile.
#include "model_base.h"

#include <stdio.h>

#include <fstream>
#include <sstream>
#include <stdexcept>

namespace ait {

void DeviceCheck(hipError_t err, const char* what, const char* file, int line) {
  if (err != hipSuccess) {
    std::ostringstream os;
    os << what << " failed: " << hipGetErrorName(err) << " (" << hipGetErrorString(err) << ") at " << file << ":"
       << line;
    throw std::runtime_error(os.str());
  }
}

void DeviceCheckLastError(const char* file, int line) {
  DeviceCheck(hipGetLastError(), "kernel launch", file, line);
}

ModelBase::ModelBase(size_t blob_size, size_t workspace_size, size_t num_inputs, size_t num_outputs,
                     size_t num_unbound_constants, uint8_t* constants, AITemplateAllocator& allocator)
    : params_(num_inputs + num_outputs + num_unbound_constants),
      constants_(constants),
      num_inputs_(num_inputs),
      num_outputs_(num_outputs),
      allocator_(allocator) {
  AIT_DEVICE_CHECK(hipGetDevice(&device_idx_));
  AIT_DEVICE_CHECK(hipEventCreateWithFlags(&run_finished_, hipEventDisableTiming));
  if (blob_size > 0) blob_ = static_cast<uint8_t*>(allocator_.Allocate(blob_size));
  if (workspace_size > 0) {
    // Scratch memory shared by the ops that need some (split-K GEMM instances).  Their arrival counters must be
    // zero before the first launch and every launch leaves them zero, so the buffer is cleared once, here.
    workspace_ = static_cast<uint8_t*>(allocator_.Allocate(workspace_size));
    workspace_size_ = static_cast<int64_t>(workspace_size);
    AIT_DEVICE_CHECK(hipMemset(workspace_, 0, workspace_size));
  }
}

ModelBase::~ModelBase() {
  if (graph_exec_ != nullptr) hipGraphExecDestroy(graph_exec_);
  if (graph_capture_stream_ != nullptr) hipStreamDestroy(graph_capture_stream_);
  if (run_finished_ != nullptr) hipEventDestroy(run_finished_);
  if (blob_ != nullptr) allocator_.Free(blob_);
  if (workspace_ != nullptr) allocator_.Free(workspace_);
}

void ModelBase::RunImpl(StreamType stream) {
  for (auto& op : ops_) {
    op.launch(stream);
    DeviceCheckLastError(__FILE__, __LINE__);
  }
}

std::vector<uint64_t> ModelBase::CurrentSignature() const {
  std::vector<uint64_t> sig;
  for (const auto& p : params_) {
    sig.push_back(reinterpret_cast<uint64_t>(p.ptr));
    for (const auto& d : p.shape_ptrs) sig.push_back(static_cast<uint64_t>(*d.value));
  }
  // Unbound constants are bound through members of the generated class, not through params_, and the bound
  // ones through the blob base: a captured graph holds their addresses, so both belong to the signature.
  // (The map is not modified after construction, so its iteration order is the same on every call.)
  for (const auto& kv : constant_name_to_ptr_) sig.push_back(reinterpret_cast<uint64_t>(*kv.second));
  sig.push_back(reinterpret_cast<uint64_t>(constants_));
  return sig;
}

void ModelBase::MarkFinished(StreamType stream) { AIT_DEVICE_CHECK(hipEventRecord(run_finished_, stream)); }

void ModelBase::Run(StreamType stream, bool graph_mode, bool mark_finished) {
  SetUpInputsOutputs();
  if (!graph_mode) {
    RunImpl(stream);
  } else {
    // Replay a captured graph while pointers and shapes are unchanged; otherwise capture again.
    // The op launchers enqueue kernels only (no memsets), so the capture is replay-safe.
    const std::vector<uint64_t> sig = CurrentSignature();
    if (graph_exec_ == nullptr || sig != graph_signature_) {
      if (graph_exec_ != nullptr) {
        hipGraphExecDestroy(graph_exec_);
        graph_exec_ = nullptr;
      }
      if (graph_capture_stream_ == nullptr)
        AIT_DEVICE_CHECK(hipStreamCreateWithFlags(&graph_capture_stream_, hipStreamNonBlocking));
      hipGraph_t graph = nullptr;
      AIT_DEVICE_CHECK(hipStreamBeginCapture(graph_capture_stream_, hipStreamCaptureModeThreadLocal));
      try {
        RunImpl(graph_capture_stream_);
      } catch (...) {
        hipStreamEndCapture(graph_capture_stream_, &graph);
        if (graph != nullptr) hipGraphDestroy(graph);
        throw;
      }
      AIT_DEVICE_CHECK(hipStreamEndCapture(graph_capture_stream_, &graph));
      AIT_DEVICE_CHECK(hipGraphInstantiate(&graph_exec_, graph, nullptr, nullptr, 0));
      AIT_DEVICE_CHECK(hipGraphDestroy(graph));
      graph_signature_ = sig;
    }
    AIT_DEVICE_CHECK(hipGraphLaunch(graph_exec_, stream));
  }
  DeviceToDeviceCopies(stream);
  if (mark_finished) MarkFinished(stream);
}

void ModelBase::Profile(StreamType stream, size_t iters, const std::string& filename) {
  SetUpInputsOutputs();
  hipEvent_t e0, e1;
  AIT_DEVICE_CHECK(hipEventCreate(&e0));
  AIT_DEVICE_CHECK(hipEventCreate(&e1));
  std::ofstream out(filename);
  if (!out.is_open()) throw std::runtime_error("Could not open profile report file " + filename);
  out << "{\n";
  for (size_t i = 0; i < ops_.size(); ++i) {
    ops_[i].launch(stream);  // warm-up
    DeviceCheckLastError(__FILE__, __LINE__);
    AIT_DEVICE_CHECK(hipEventRecord(e0, stream));
    for (size_t it = 0; it < iters; ++it) ops_[i].launch(stream);
    AIT_DEVICE_CHECK(hipEventRecord(e1, stream));
    AIT_DEVICE_CHECK(hipEventSynchronize(e1));
    DeviceCheckLastError(__FILE__, __LINE__);
    float ms = 0.f;
    AIT_DEVICE_CHECK(hipEventElapsedTime(&ms, e0, e1));
    out << "  \"" << ops_[i].name << "\": { \"ms_per_iter\": " << (iters ? ms / iters : 0.f)
        << ", \"qps\": " << (ms > 0.f ? 1000.0f * iters / ms : 0.f) << " }" << (i + 1 < ops_.size() ? ",\n" : "\n");
  }
  out << "}\n";
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  AIT_DEVICE_CHECK(hipEventRecord(run_finished_, stream));
}

bool ModelBase::IsPending() {
  const hipError_t q = hipEventQuery(run_finished_);
  if (q == hipErrorNotReady) return true;
  if (q != hipSuccess) {
    (void)hipGetLastError();
    throw std::runtime_error(std::string("hipEventQuery failed: ") + hipGetErrorString(q));
  }
  return false;
}

void ModelBase::WaitForCompletion() { AIT_DEVICE_CHECK(hipEventSynchronize(run_finished_)); }

void ModelBase::SetParam(const void* src, size_t param_idx) { params_[param_idx].ptr = const_cast<void*>(src); }

void ModelBase::SetInput(const void* src, const AITemplateParamShape& shape, size_t idx) {
  if (idx >= num_inputs_) throw std::out_of_range("input index out of range");
  ParamInfo& p = params_[idx];
  if (shape.size != p.shape_ptrs.size()) {
    std::ostringstream os;
    os << "Shape of input " << p.name << " has rank " << shape.size << ", expected " << p.shape_ptrs.size();
    throw std::runtime_error(os.str());
  }
  for (size_t i = 0; i < shape.size; ++i) {
    const int64_t v = shape.shape_data[i];
    const ParamDim& d = p.shape_ptrs[i];
    if (v < d.lower_bound || v > d.upper_bound) {
      std::ostringstream os;
      os << "Shape of input " << p.name << " is invalid: dim " << i << " = " << v << " is outside ["
         << d.lower_bound << ", " << d.upper_bound << "]";
      throw std::out_of_range(os.str());
    }
    *d.value = v;
  }
  SetParam(src, idx);
}

void ModelBase::SetOutput(void* src, size_t idx) {
  if (idx >= num_outputs_) throw std::out_of_range("output index out of range");
  SetParam(src, idx + num_inputs_);
}

void ModelBase::GetOutputShape(size_t idx, int64_t* output_shape_out) {
  if (idx >= num_outputs_) throw std::out_of_range("output index out of range");
  const auto& dims = params_[idx + num_inputs_].shape_ptrs;
  for (size_t i = 0; i < dims.size(); ++i) output_shape_out[i] = *dims[i].value;
}

void ModelBase::SetConstant(const char* name, const void* src) {
  auto it = constant_name_to_ptr_.find(name);
  if (it == constant_name_to_ptr_.end()) throw std::out_of_range(std::string("Could not find constant ") + name);
  *it->second = src;
}

void ModelBase::SetConstantsBlob(uint8_t* base) {
  constants_ = base;
  BindBoundConstants(base);
}

}  // namespace ait
