#include "model_container.h"

#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <numeric>
#include <sstream>
#include <stdexcept>
#include <thread>

namespace ait {

void* DefaultAllocator::Allocate(size_t nbytes) {
  void* p = nullptr;
  AIT_DEVICE_CHECK(hipMalloc(&p, nbytes));
  return p;
}
void DefaultAllocator::Free(void* ptr) { AIT_DEVICE_CHECK(hipFree(ptr)); }
void* TrackingAllocator::Allocate(size_t nbytes) {
  void* p = DefaultAllocator::Allocate(nbytes);
  num_bytes_ += nbytes;
  return p;
}

ModelContainer::ModelContainer(size_t num_runtimes, AITemplateAllocator& allocator)
    : meta_(aitamd_model_meta()), allocator_(allocator) {
  if (num_runtimes == 0) throw std::runtime_error("Number of runtimes must be positive");
  if (meta_->constants_size > 0) {
    constants_blob_ = static_cast<uint8_t*>(allocator_.Allocate(meta_->constants_size));
    const size_t image = static_cast<size_t>(meta_->constants_end - meta_->constants_begin);
    if (image < meta_->constants_size) throw std::runtime_error("embedded constant image is smaller than the layout");
    AIT_DEVICE_CHECK(hipMemcpy(constants_blob_, meta_->constants_begin, meta_->constants_size, hipMemcpyHostToDevice));
  }
  models_.reserve(num_runtimes);
  for (size_t i = 0; i < num_runtimes; ++i) {
    models_.emplace_back(aitamd_model_create(constants_blob_, &allocator_));
    available_.push_back(models_.back().get());
  }
}

ModelContainer::~ModelContainer() {
  {
    std::unique_lock<std::mutex> lk(pool_mutex_);
    for (ModelBase* m : pending_) {
      try {
        m->WaitForCompletion();
      } catch (const std::exception& e) {
        fprintf(stderr, "[aitemplate_amd] error while draining a runtime: %s\n", e.what());
      }
    }
    pending_.clear();
  }
  models_.clear();
  for (uint8_t* blob : {constants_blob_, staged_blob_}) {
    if (blob == nullptr) continue;
    try {
      allocator_.Free(blob);
    } catch (...) {
    }
  }
}

// ---- pool ------------------------------------------------------------------
void ModelContainer::ReclaimFinishedModels(std::unique_lock<std::mutex>&) {
  auto it = pending_.begin();
  while (it != pending_.end()) {
    bool done = false;
    try {
      done = !(*it)->IsPending();
    } catch (const std::exception& e) {
      fprintf(stderr, "[aitemplate_amd] a pending runtime failed: %s\n", e.what());
      done = true;  // reclaim it anyway
    }
    if (done) {
      available_.push_back(*it);
      it = pending_.erase(it);
    } else {
      ++it;
    }
  }
}

ModelBase* ModelContainer::GetAvailableModel() {
  std::unique_lock<std::mutex> lk(pool_mutex_);
  for (;;) {
    if (available_.empty()) ReclaimFinishedModels(lk);
    if (!available_.empty()) {
      ModelBase* m = available_.back();
      available_.pop_back();
      return m;
    }
    if (!pending_.empty()) {
      // every runtime is in flight on the GPU: wait for the oldest one
      ModelBase* oldest = pending_.front();
      pending_.erase(pending_.begin());
      lk.unlock();
      try {
        oldest->WaitForCompletion();
      } catch (const std::exception& e) {
        fprintf(stderr, "[aitemplate_amd] a pending runtime failed: %s\n", e.what());
      }
      return oldest;
    }
    // all runtimes are held by other host threads
    pool_cv_.wait(lk);
  }
}

void ModelContainer::ReturnModel(ModelBase* m, bool failed) {
  {
    std::lock_guard<std::mutex> lk(pool_mutex_);
    if (failed)
      available_.push_back(m);
    else
      pending_.push_back(m);
  }
  pool_cv_.notify_one();
}

// ---- run ------------------------------------------------------------------
void ModelContainer::PrepareForRun(ModelBase* m, const AITData* inputs, size_t num_inputs, AITData* outputs,
                                   size_t num_outputs) {
  if (num_inputs != NumInputs()) {
    std::ostringstream os;
    os << "Got wrong number of inputs; expected " << NumInputs() << ", got " << num_inputs;
    throw std::runtime_error(os.str());
  }
  if (num_outputs != NumOutputs()) {
    std::ostringstream os;
    os << "Got wrong number of outputs; expected " << NumOutputs() << ", got " << num_outputs;
    throw std::runtime_error(os.str());
  }
  if (num_inputs > 0 && inputs == nullptr) throw std::runtime_error("inputs cannot be null");
  if (num_outputs > 0 && outputs == nullptr) throw std::runtime_error("outputs cannot be null");
  for (size_t i = 0; i < num_inputs; ++i) {
    const AITData& in = inputs[i];
    if (in.dtype != meta_->inputs[i].dtype)
      throw std::runtime_error("Got wrong dtype for input " + meta_->inputs[i].name);
    size_t numel = 1;
    for (size_t d = 0; d < in.shape.size; ++d) numel *= static_cast<size_t>(in.shape.shape_data[d]);
    if (in.ptr == nullptr && numel != 0)
      throw std::runtime_error("Input " + meta_->inputs[i].name + " has a null data pointer");
    m->SetInput(in.ptr, in.shape, i);
  }
  for (size_t i = 0; i < num_outputs; ++i) {
    if (outputs[i].dtype != meta_->outputs[i].dtype)
      throw std::runtime_error("Got wrong dtype for output " + meta_->outputs[i].name);
    if (outputs[i].ptr == nullptr) {
      // a null output is accepted only when the output can be empty
      const auto& ms = meta_->outputs[i].max_shape;
      const bool may_be_empty = std::any_of(ms.begin(), ms.end(), [](int64_t v) { return v == 0; });
      if (!may_be_empty) throw std::runtime_error("Output " + meta_->outputs[i].name + " has a null data pointer");
    }
    m->SetOutput(outputs[i].ptr, i);
  }
  for (const auto& kv : unbound_ptrs_[0]) m->SetConstant(kv.first.c_str(), kv.second);
}

void ModelContainer::Run(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs,
                         StreamType stream, bool sync, bool graph_mode, int64_t** output_shapes_out) {
  std::shared_lock<std::shared_mutex> constants_lk(constants_mutex_);
  ModelBase* m = GetAvailableModel();
  try {
    PrepareForRun(m, inputs, num_inputs, outputs, num_outputs);
    m->Run(stream, graph_mode);
  } catch (...) {
    ReturnModel(m, /*failed=*/true);
    throw;
  }
  if (output_shapes_out != nullptr) {
    for (size_t i = 0; i < num_outputs; ++i)
      if (output_shapes_out[i] != nullptr) m->GetOutputShape(i, output_shapes_out[i]);
  }
  ReturnModel(m, /*failed=*/false);
  if (sync) AIT_DEVICE_CHECK(hipStreamSynchronize(stream));
}

void ModelContainer::RunWithOutputsOnHost(const AITData* inputs, size_t num_inputs, AITData* outputs,
                                          size_t num_outputs, StreamType stream, bool graph_mode,
                                          int64_t** output_shapes_out) {
  if (num_outputs != NumOutputs()) throw std::runtime_error("Got wrong number of outputs");
  std::vector<void*> device_bufs(num_outputs, nullptr);
  std::vector<AITData> device_outputs(outputs, outputs + num_outputs);
  std::vector<std::vector<int64_t>> shapes(num_outputs);
  std::vector<int64_t*> shape_ptrs(num_outputs);
  auto release = [&] {
    for (void* p : device_bufs)
      if (p != nullptr) hipFree(p);
  };
  try {
    for (size_t i = 0; i < num_outputs; ++i) {
      const auto& ms = meta_->outputs[i].max_shape;
      size_t bytes = AITemplateDtypeSizeBytes(meta_->outputs[i].dtype);
      for (int64_t v : ms) bytes *= static_cast<size_t>(v);
      if (bytes > 0) AIT_DEVICE_CHECK(hipMalloc(&device_bufs[i], bytes));
      device_outputs[i].ptr = device_bufs[i];
      shapes[i].resize(ms.size());
      shape_ptrs[i] = shapes[i].data();
    }
    Run(inputs, num_inputs, device_outputs.data(), num_outputs, stream, /*sync=*/true, graph_mode, shape_ptrs.data());
    for (size_t i = 0; i < num_outputs; ++i) {
      size_t bytes = AITemplateDtypeSizeBytes(meta_->outputs[i].dtype);
      for (int64_t v : shapes[i]) bytes *= static_cast<size_t>(v);
      if (bytes > 0) AIT_DEVICE_CHECK(hipMemcpy(outputs[i].ptr, device_bufs[i], bytes, hipMemcpyDeviceToHost));
      if (output_shapes_out != nullptr && output_shapes_out[i] != nullptr)
        std::copy(shapes[i].begin(), shapes[i].end(), output_shapes_out[i]);
    }
  } catch (...) {
    release();
    throw;
  }
  release();
}

void ModelContainer::Profile(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs,
                             StreamType stream, size_t num_iters, const char* filename) {
  if (filename == nullptr) throw std::runtime_error("profile report filename cannot be null");
  std::shared_lock<std::shared_mutex> constants_lk(constants_mutex_);
  ModelBase* m = GetAvailableModel();
  try {
    PrepareForRun(m, inputs, num_inputs, outputs, num_outputs);
    m->Profile(stream, num_iters, filename);
  } catch (...) {
    ReturnModel(m, true);
    throw;
  }
  ReturnModel(m, false);
}

// One runtime, prepared once, run `count` times back to back between two events - no per-run wait, as in
// the reference (static/csrc/model_container.cpp:856-900).
float ModelContainer::BenchmarkImpl(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs,
                                    StreamType stream, bool graph_mode, size_t count, int64_t** output_shapes_out) {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  AIT_DEVICE_CHECK(hipEventCreate(&e0));
  AIT_DEVICE_CHECK(hipEventCreate(&e1));
  float ms = 0.f;
  std::shared_lock<std::shared_mutex> constants_lk(constants_mutex_);
  ModelBase* m = GetAvailableModel();
  try {
    PrepareForRun(m, inputs, num_inputs, outputs, num_outputs);
    m->Run(stream, graph_mode);  // one untimed run warms code and caches
    AIT_DEVICE_CHECK(hipEventRecord(e0, stream));
    // the timed runs are queued without a completion marker in between; the runtime is marked once
    for (size_t i = 0; i < count; ++i) m->Run(stream, graph_mode, /*mark_finished=*/false);
    AIT_DEVICE_CHECK(hipEventRecord(e1, stream));
    m->MarkFinished(stream);
    if (output_shapes_out != nullptr) {
      for (size_t i = 0; i < num_outputs; ++i)
        if (output_shapes_out[i] != nullptr) m->GetOutputShape(i, output_shapes_out[i]);
    }
    AIT_DEVICE_CHECK(hipEventSynchronize(e1));
    AIT_DEVICE_CHECK(hipEventElapsedTime(&ms, e0, e1));
  } catch (...) {
    ReturnModel(m, /*failed=*/true);
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    throw;
  }
  ReturnModel(m, /*failed=*/false);
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  return count ? ms / count : 0.f;
}

float ModelContainer::Benchmark(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs,
                                StreamType stream, bool graph_mode, size_t count, size_t num_threads,
                                bool use_unique_stream_per_thread, int64_t** output_shapes_out) {
  if (num_threads == 0) num_threads = std::thread::hardware_concurrency();
  if (num_threads <= 1)
    return BenchmarkImpl(inputs, num_inputs, outputs, num_outputs, stream, graph_mode, count, output_shapes_out);
  // Several host threads hammer the pool at once; every thread but the first writes to
  // scratch outputs of its own so that results do not race.
  std::vector<std::vector<void*>> scratch(num_threads);
  std::vector<std::vector<AITData>> outs(num_threads, std::vector<AITData>(outputs, outputs + num_outputs));
  std::vector<StreamType> streams(num_threads, stream);
  std::vector<float> times(num_threads, 0.f);
  std::vector<std::string> errors(num_threads);
  auto cleanup = [&] {
    for (auto& v : scratch)
      for (void* p : v)
        if (p != nullptr) hipFree(p);
    if (use_unique_stream_per_thread)
      for (size_t t = 0; t < num_threads; ++t)
        if (streams[t] != stream && streams[t] != nullptr) hipStreamDestroy(streams[t]);
  };
  try {
    for (size_t t = 0; t < num_threads; ++t) {
      if (use_unique_stream_per_thread) AIT_DEVICE_CHECK(hipStreamCreateWithFlags(&streams[t], hipStreamNonBlocking));
      if (t == 0) continue;
      scratch[t].assign(num_outputs, nullptr);
      for (size_t i = 0; i < num_outputs; ++i) {
        size_t bytes = AITemplateDtypeSizeBytes(meta_->outputs[i].dtype);
        for (int64_t v : meta_->outputs[i].max_shape) bytes *= static_cast<size_t>(v);
        if (bytes > 0) AIT_DEVICE_CHECK(hipMalloc(&scratch[t][i], bytes));
        outs[t][i].ptr = scratch[t][i];
      }
    }
    int dev = 0;
    AIT_DEVICE_CHECK(hipGetDevice(&dev));
    std::vector<std::thread> threads;
    for (size_t t = 0; t < num_threads; ++t) {
      threads.emplace_back([&, t] {
        try {
          AIT_DEVICE_CHECK(hipSetDevice(dev));
          times[t] = BenchmarkImpl(inputs, num_inputs, outs[t].data(), num_outputs, streams[t], graph_mode, count,
                                   t == 0 ? output_shapes_out : nullptr);
        } catch (const std::exception& e) {
          errors[t] = e.what();
        }
      });
    }
    for (auto& th : threads) th.join();
    for (const auto& e : errors)
      if (!e.empty()) throw std::runtime_error("benchmark thread failed: " + e);
  } catch (...) {
    cleanup();
    throw;
  }
  cleanup();
  // per-inference latency seen by one thread, averaged over threads, scaled to throughput time
  const float mean = std::accumulate(times.begin(), times.end(), 0.f) / num_threads;
  return mean / num_threads;
}

// ---- constants --------------------------------------------------------------
const ConstantMeta& ModelContainer::FindConstant(const char* name) const {
  if (name == nullptr) throw std::runtime_error("constant name cannot be null");
  for (const auto& c : meta_->constants)
    if (c.name == name) return c;
  throw std::out_of_range(std::string("Could not find constant ") + name);
}

void ModelContainer::SetConstant(const char* name, const AITData& tensor, bool use_inactive_set, StreamType stream) {
  const ConstantMeta& c = FindConstant(name);
  if (tensor.dtype != c.dtype) throw std::runtime_error(std::string("Got wrong dtype for constant ") + name);
  if (tensor.shape.size != c.shape.size()) throw std::runtime_error(std::string("Got wrong rank for constant ") + name);
  for (size_t i = 0; i < c.shape.size(); ++i)
    if (tensor.shape.shape_data[i] != c.shape[i])
      throw std::runtime_error(std::string("Got wrong shape for constant ") + name);
  if (tensor.ptr == nullptr && c.num_bytes != 0) throw std::runtime_error(std::string("Null data for constant ") + name);
  std::unique_lock<std::shared_mutex> lk(constants_mutex_);
  if (c.bound) {
    if (c.num_bytes == 0) return;
    // Run() gives up the shared lock once its kernels are queued, so a runtime may still be reading the
    // blob on another stream: drain every runtime before bytes change (reference:
    // static/csrc/model_container.cpp:452-455, WaitForAllModels before any SetConstant).
    WaitForAllModels();
    uint8_t* dst = constants_blob_;
    if (use_inactive_set) {
      // double buffering: the bytes go to a second blob that SwapConstants() makes the active one
      // (reference: static/csrc/model_container.cpp:661-680).  The first staged write after a swap starts
      // from a copy of the active blob, so constants that are not staged keep their current values.
      if (staged_blob_ == nullptr) staged_blob_ = static_cast<uint8_t*>(allocator_.Allocate(meta_->constants_size));
      if (!staged_blob_in_use_) {
        AIT_DEVICE_CHECK(hipMemcpyAsync(staged_blob_, constants_blob_, meta_->constants_size, hipMemcpyDeviceToDevice, stream));
        staged_blob_in_use_ = true;
      }
      dst = staged_blob_;
    }
    AIT_DEVICE_CHECK(hipMemcpyAsync(dst + c.offset, tensor.ptr, c.num_bytes, hipMemcpyDeviceToDevice, stream));
    AIT_DEVICE_CHECK(hipStreamSynchronize(stream));
    return;
  }
  unbound_ptrs_[use_inactive_set ? 1 : 0][c.name] = tensor.ptr;
}

// Caller holds constants_mutex_ exclusively, so no Run() can start meanwhile.
void ModelContainer::WaitForAllModels() {
  std::unique_lock<std::mutex> lk(pool_mutex_);
  for (ModelBase* m : pending_) {
    m->WaitForCompletion();
    available_.push_back(m);
  }
  pending_.clear();
}

size_t ModelContainer::GetNumConstants(bool unbound_only, bool folding_inputs_only) const {
  if (folding_inputs_only) return 0;  // nothing is folded at run time: graphs here have no constant sub-graphs
  size_t n = 0;
  for (const auto& c : meta_->constants)
    if (!unbound_only || !c.bound) ++n;
  return n;
}

void ModelContainer::WriteAllConstantNamesTo(const char** out, bool unbound_only, bool folding_inputs_only) const {
  if (folding_inputs_only) return;
  size_t n = 0;
  for (const auto& c : meta_->constants)
    if (!unbound_only || !c.bound) out[n++] = c.name.c_str();
}

AITemplateDtype ModelContainer::ConstantDtype(const char* name) const { return FindConstant(name).dtype; }
const char* ModelContainer::ConstantOriginalName(const char* name) const {
  return FindConstant(name).original_name.c_str();
}

void ModelContainer::FoldConstants(StreamType stream, bool sync, bool) {
  // No op of a GEMM-family graph is evaluated ahead of time, so there is nothing to fold;
  // the call only orders itself on the stream like the original does.
  if (sync) AIT_DEVICE_CHECK(hipStreamSynchronize(stream));
}

void ModelContainer::SwapConstants() {
  std::unique_lock<std::shared_mutex> lk(constants_mutex_);
  // entries staged in the inactive set replace the active ones; unstaged names keep their binding
  for (auto& kv : unbound_ptrs_[1]) std::swap(unbound_ptrs_[0][kv.first], kv.second);
  if (staged_blob_in_use_) {
    // the staged blob becomes the one every runtime reads; the old one is the next staging area
    WaitForAllModels();
    std::swap(constants_blob_, staged_blob_);
    staged_blob_in_use_ = false;
    for (auto& m : models_) m->SetConstantsBlob(constants_blob_);
  }
}

// ---- metadata ---------------------------------------------------------------
const char* ModelContainer::InputName(size_t idx) const { return meta_->inputs.at(idx).name.c_str(); }
const char* ModelContainer::OutputName(size_t idx) const { return meta_->outputs.at(idx).name.c_str(); }
AITemplateParamShape ModelContainer::MaxInputShape(size_t idx) const {
  const auto& s = meta_->inputs.at(idx).max_shape;
  return AITemplateParamShape(s.data(), s.size());
}
AITemplateParamShape ModelContainer::MaxOutputShape(size_t idx) const {
  const auto& s = meta_->outputs.at(idx).max_shape;
  return AITemplateParamShape(s.data(), s.size());
}
AITemplateDtype ModelContainer::InputDtype(size_t idx) const { return meta_->inputs.at(idx).dtype; }
AITemplateDtype ModelContainer::OutputDtype(size_t idx) const { return meta_->outputs.at(idx).dtype; }

}  // namespace ait
