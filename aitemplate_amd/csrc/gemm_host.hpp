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

// Workgroups per tile of a split-K launch (the launcher and the instance choice share the rule): as many as bring
// the grid up to about one workgroup per CU, each with at least two K-slabs, at most 16; 1 (no splitting, nothing
// written to the scratch memory) for grids that fill the device anyway.  Measured against two and four workgroups
// per CU and against longer minimum shares (256x1024x1024, 512x768x3072, 1x6912x8314, 64x256x8192): never slower.
inline int split_k_rule(int64_t tiles, int64_t k_tiles, int cus) {
  if (tiles <= 0) return 1;
  int64_t s = cus / tiles;
  if (s > k_tiles / 2) s = k_tiles / 2;
  if (s > 16) s = 16;
  return (int)(s < 1 ? 1 : s);
}

// Compute units of a device, looked up once per device (256 where the device cannot be asked).  The launcher's grid
// and split-K factor and the instance choice all use this one figure.
inline int device_cus(int dev) {
  constexpr int kSlots = 64;
  static int cus[kSlots] = {};
  if (dev < 0) dev = 0;
  int v = cus[dev % kSlots];
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cus[dev % kSlots] = v;
  }
  return v;
}
inline int current_device_cus() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();  // no device: the instance choice still answers, priced for a 256-CU part
    return 256;
  }
  return device_cus(dev);
}

// Defined once per (epilogue, dtype) translation unit; nullptr table when that
// combination is not compiled in.
GemmAlgoTable gemm_table(int epilogue, int dtype);

}  // namespace aitamd
