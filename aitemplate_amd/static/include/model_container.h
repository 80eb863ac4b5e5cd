// A pool of `num_runtimes` model instances behind the C ABI: concurrent Run calls each
// take a free instance (blocking when none is free), constants are shared, and constant
// updates exclude running inferences.
//
// Role in the reference: static/include/model_container.h:43-324 and
// static/csrc/model_container.cpp:43-901.
#pragma once

#include <condition_variable>
#include <memory>
#include <mutex>
#include <shared_mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "model_base.h"

namespace ait {

class DefaultAllocator : public AITemplateAllocator {
 public:
  void* Allocate(size_t nbytes) override;
  void Free(void* ptr) override;
};

class TrackingAllocator : public DefaultAllocator {
 public:
  void* Allocate(size_t nbytes) override;
  size_t NumBytesAllocated() const { return num_bytes_; }

 private:
  size_t num_bytes_ = 0;
};

class ModelContainer {
 public:
  ModelContainer(size_t num_runtimes, AITemplateAllocator& allocator);
  ~ModelContainer();

  void Run(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs, StreamType stream,
           bool sync, bool graph_mode, int64_t** output_shapes_out);
  void RunWithOutputsOnHost(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs,
                            StreamType stream, bool graph_mode, int64_t** output_shapes_out);
  void Profile(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs, StreamType stream,
               size_t num_iters, const char* filename);
  float Benchmark(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs, StreamType stream,
                  bool graph_mode, size_t count, size_t num_threads, bool use_unique_stream_per_thread,
                  int64_t** output_shapes_out);

  void SetConstant(const char* name, const AITData& tensor, bool use_inactive_set, StreamType stream);
  size_t GetNumConstants(bool unbound_only, bool folding_inputs_only) const;
  void WriteAllConstantNamesTo(const char** out, bool unbound_only, bool folding_inputs_only) const;
  AITemplateDtype ConstantDtype(const char* name) const;
  const char* ConstantOriginalName(const char* name) const;
  void FoldConstants(StreamType stream, bool sync, bool double_buffer);
  void SwapConstants();

  size_t NumInputs() const { return meta_->inputs.size(); }
  size_t NumOutputs() const { return meta_->outputs.size(); }
  const char* InputName(size_t idx) const;
  const char* OutputName(size_t idx) const;
  AITemplateParamShape MaxInputShape(size_t idx) const;
  AITemplateParamShape MaxOutputShape(size_t idx) const;
  AITemplateDtype InputDtype(size_t idx) const;
  AITemplateDtype OutputDtype(size_t idx) const;
  size_t GetNumRuntimes() const { return models_.size(); }

 private:
  ModelBase* GetAvailableModel();
  void ReclaimFinishedModels(std::unique_lock<std::mutex>& lk);
  void ReturnModel(ModelBase* m, bool failed);
  void PrepareForRun(ModelBase* m, const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs);
  const ConstantMeta& FindConstant(const char* name) const;
  void WaitForAllModels();
  float BenchmarkImpl(const AITData* inputs, size_t num_inputs, AITData* outputs, size_t num_outputs,
                      StreamType stream, bool graph_mode, size_t count, int64_t** output_shapes_out);

  const ModelMeta* meta_;
  AITemplateAllocator& allocator_;
  uint8_t* constants_blob_ = nullptr;  // device image of the bound constants (the one the runtimes read)
  uint8_t* staged_blob_ = nullptr;     // second image: takes double-buffered updates until SwapConstants()
  bool staged_blob_in_use_ = false;    // staged_blob_ holds updates that have not been swapped in yet
  std::vector<std::unique_ptr<ModelBase>> models_;
  std::vector<ModelBase*> available_;
  std::vector<ModelBase*> pending_;
  std::mutex pool_mutex_;
  std::condition_variable pool_cv_;
  // Run holds this shared; constant updates hold it exclusively
  std::shared_mutex constants_mutex_;
  // unbound constants: [0] is the active set, [1] the set SwapConstants() activates
  std::unordered_map<std::string, const void*> unbound_ptrs_[2];
};

}  // namespace ait
