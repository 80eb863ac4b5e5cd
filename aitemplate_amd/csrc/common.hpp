// Shared device-side vocabulary for the gfx950 GEMM-family kernels: vector
// types, buffer-resource helpers, fp16/bf16 conversion and the XCD-aware
// workgroup -> output-tile mapping.  gfx950 (MI355X, CDNA4) only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace aitamd {

using f16 = _Float16;
using bf16 = __bf16;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define AITAMD_DEVICE __device__ __forceinline__

constexpr int kWaveSize = 64;
constexpr int kNumXcd = 8;  // MI355X: 8 accelerator dies, one L2 each

// ---------------------------------------------------------------------------
// Element-type traits: 8-wide operand vector and the 32x32x16 / 16x16x32 MFMA.
// ---------------------------------------------------------------------------
template <class T>
struct ElemTraits;

template <>
struct ElemTraits<f16> {
  using vec8 = f16x8;
  using vec4 = f16x4;
  static AITAMD_DEVICE f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static AITAMD_DEVICE f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static AITAMD_DEVICE float to_float(f16 v) { return (float)v; }
  static AITAMD_DEVICE f16 from_float(float v) { return (f16)v; }
  // float(v) + c in one instruction: with `one` = 1.0 in a register the compiler cannot see through, the fused
  // multiply-add of a widened half maps to v_fma_mix_f32 (conversion and add together; same single rounding)
  static AITAMD_DEVICE float to_float_plus(f16 v, float one, float c) { return __builtin_fmaf((float)v, one, c); }
};

template <>
struct ElemTraits<bf16> {
  using vec8 = bf16x8;
  using vec4 = bf16x4;
  static AITAMD_DEVICE f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static AITAMD_DEVICE f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static AITAMD_DEVICE float to_float(bf16 v) { return (float)v; }
  static AITAMD_DEVICE bf16 from_float(float v) { return (bf16)v; }
  static AITAMD_DEVICE float to_float_plus(bf16 v, float one, float c) { (void)one; return (float)v + c; }
};

// LDS transpose read: 4 x 16-bit per lane, gathered across the 16 lanes of a block
AITAMD_DEVICE f16x4 tr_read16(const f16* p) {
  typedef __fp16 raw4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
  const raw4 r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((__attribute__((address_space(3))) raw4*)p);
  return __builtin_bit_cast(f16x4, r);
}
AITAMD_DEVICE bf16x4 tr_read16(const bf16* p) {
  typedef __bf16 raw4 __attribute__((__vector_size__(4 * sizeof(__bf16))));
  const raw4 r = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) raw4*)p);
  return __builtin_bit_cast(bf16x4, r);
}
template <class T>
AITAMD_DEVICE typename ElemTraits<T>::vec8 join_halves(typename ElemTraits<T>::vec4 lo, typename ElemTraits<T>::vec4 hi) {
  typename ElemTraits<T>::vec8 v;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    v[j] = lo[j];
    v[4 + j] = hi[j];
  }
  return v;
}

// ---------------------------------------------------------------------------
// Raw buffer resources.  Loads whose byte offset is >= num_records return 0,
// which is how every M/N/K tail is zero-filled without branches.
// ---------------------------------------------------------------------------
// f(integral_constant<int, I>) for I in [I0, I1): a loop whose index is a constant expression in the body
// (immediate operands of builtins)
template <int I0, int I1, class F>
AITAMD_DEVICE void static_for(F&& f) {
  if constexpr (I0 < I1) {
    f(std::integral_constant<int, I0>{});
    static_for<I0 + 1, I1>(f);
  }
}

constexpr uint32_t kOobOffset = 0x80000000u;  // >= any num_records we build

// Every descriptor in these kernels is the same for all lanes of a wave (one per tile, batch entry or wave
// part), but the compiler cannot prove that for values computed from the wave index or loaded tile coordinates,
// and a buffer access through a descriptor it takes for lane-varying is wrapped in a loop over the wave's
// distinct descriptors (four v_readfirstlane, two 64-bit compares and a branch per access).  Reading base and
// size from the first lane states the uniformity; where they already are scalar registers this folds away.
AITAMD_DEVICE __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t num_bytes) {
  const uint64_t v = reinterpret_cast<uint64_t>(base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uint64_t)hi << 32) | lo), 0,
                                           __builtin_amdgcn_readfirstlane(num_bytes), 0x00020000);
}

AITAMD_DEVICE u32x4 buffer_load_16B(__amdgpu_buffer_rsrc_t r, uint32_t voffset) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, voffset, 0, 0);
}
AITAMD_DEVICE u32x2 buffer_load_8B(__amdgpu_buffer_rsrc_t r, uint32_t voffset) {
  return __builtin_amdgcn_raw_buffer_load_b64(r, voffset, 0, 0);
}
AITAMD_DEVICE uint32_t buffer_load_4B(__amdgpu_buffer_rsrc_t r, uint32_t voffset) {
  return __builtin_amdgcn_raw_buffer_load_b32(r, voffset, 0, 0);
}
AITAMD_DEVICE uint16_t buffer_load_2B(__amdgpu_buffer_rsrc_t r, uint32_t voffset) {
  return __builtin_amdgcn_raw_buffer_load_b16(r, voffset, 0, 0);
}

// Clamp a 64-bit byte count into the 32-bit num_records field.
AITAMD_DEVICE uint32_t clamp_records(int64_t bytes) {
  return bytes <= 0 ? 0u : (bytes >= 0x7fffffffll ? 0x7fffffffu : (uint32_t)bytes);
}

// ---------------------------------------------------------------------------
// Workgroup -> tile mapping.  The hardware deals consecutive workgroup ids
// round-robin over the 8 XCDs; tiles that share an A row-panel or a B
// column-panel should land on the same XCD so the panel is fetched into one
// L2 only.  Step 1 gives every XCD a contiguous range of logical (batch, tile) ids,
// step 2 walks the tiles of a batch in groups of kGroupM tile-rows, column by column.
// ---------------------------------------------------------------------------
AITAMD_DEVICE void map_tile_grouped(int wg, int tiles_m, int tiles_n, int batch, int kGroupM, int& b, int& tm, int& tn);
template <int kGroupM>
AITAMD_DEVICE void map_tile(int wg, int tiles_m, int tiles_n, int batch, int& b, int& tm, int& tn) {
  map_tile_grouped(wg, tiles_m, tiles_n, batch, kGroupM, b, tm, tn);
}
// (the group height as a value: the persistent kernels take it from the launcher)
AITAMD_DEVICE void map_tile_grouped(int wg, int tiles_m, int tiles_n, int batch, int kGroupM, int& b, int& tm, int& tn) {
  // wg runs over batch * tiles_m * tiles_n workgroups; logical ids are batch-major, so an XCD's
  // contiguous id range is a run of whole batches (plus at most two partial ones at its ends):
  // the tiles of one batch share its operands through one L2 and fill its output rows together.
  const int per_batch = tiles_m * tiles_n;
  const int total = per_batch * batch;
  const int xcd = wg % kNumXcd;
  const int local = wg / kNumXcd;
  const int q = total / kNumXcd;
  const int r = total % kNumXcd;
  const int flat = xcd * q + (xcd < r ? xcd : r) + local;
  b = flat / per_batch;
  const int id = flat - b * per_batch;
  const int group_sz = kGroupM * tiles_n;
  const int g = id / group_sz;
  const int first_m = g * kGroupM;
  const int gm = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
  const int in_group = id - g * group_sz;
  tm = first_m + in_group % gm;
  tn = in_group / gm;
}

// Block form of the mapping for one batch whose tile grid divides over the XCDs as xcd_cols column blocks times
// 8 / xcd_cols row blocks: XCD x works through its own block row by row, so the B panels of the block's few
// columns are fetched into its L2 once and stay there for every row (the tiles that need an A panel are adjacent
// in the walk and run at the same time).  Same workgroup -> XCD deal as above: wg % 8 is the XCD.
AITAMD_DEVICE void map_tile_block(int wg, int tiles_m, int tiles_n, int xcd_cols, int& tm, int& tn) {
  const int xcd = wg % kNumXcd;
  const int local = wg / kNumXcd;
  const int cols = tiles_n / xcd_cols;
  const int rows = tiles_m / (kNumXcd / xcd_cols);
  const int cb = xcd % xcd_cols, rb = xcd / xcd_cols;
  const int r = local / cols;
  tm = rb * rows + r;
  tn = cb * cols + (local - r * cols);
}

}  // namespace aitamd
