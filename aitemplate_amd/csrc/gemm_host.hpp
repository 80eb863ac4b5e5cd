// Host-side description of one compiled GEMM kernel instance ("algo") and the
// per-(epilogue, dtype) tables the C ABI dispatches through.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_kernel.hpp"

namespace aitamd {

enum DType : int { kF16 = 0, kBF16 = 1, kNumDTypes = 2 };

struct GemmAlgo {
  const char* name;  // e.g. "gemm_rcr_f16_256x256x64_w2x2_v8"
  int bm, bn, bk;
  int threads;
  int kvec;
  int lds_bytes;
  int wgs_per_cu;  // workgroups of this instance one CU holds at once
  int direct_lds;  // 0: register-staged loads, 1: direct-to-LDS ring, 2: persistent direct-to-LDS ring, 4: 1 + split-K
  int layouts;     // bit L set: a kernel for operand layout L exists (0 rcr, 1 rrr, 2 ccr, 3 crr)
  hipError_t (*launch)(const GemmParams& p, hipStream_t stream);
  // bytes of scratch memory (GemmParams::ws) a launch on this problem needs; null for instances that need none
  int64_t (*workspace_bytes)(const GemmParams& p);
};

struct GemmAlgoTable {
  const GemmAlgo* algos;
  int count;
};

// Defined once per (epilogue, dtype) translation unit; nullptr table when that
// combination is not compiled in.
GemmAlgoTable gemm_table(int epilogue, int dtype);

}  // namespace aitamd
