// Stand-alone element-wise kernel for the element-wise ops of a graph that no GEMM epilogue absorbed.
//
// Takes the place of the reference's fused_elementwise kernels for the single-op case
// (python/aitemplate/backend/common/elementwise_common.py builds them; the function table is
// python/aitemplate/backend/backend_spec.py:100-330, the ROCm device functions
// python/aitemplate/backend/rocm/elementwise/custom_math.h).  out[i] = f(a[i], b[i % b_period]) over the
// flattened output: b_period = numel for a same-shape operand, the product of b's dims for an operand that
// broadcasts over leading dims (a bias row, a scalar tensor), and a constant number when b is null.
// Bound: HBM (2 or 3 streams of 2-byte elements); 16 bytes per lane and access where alignment allows,
// all arithmetic in fp32 with one rounding to the element type, like the GEMM epilogues.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/aitemplate_amd_kernels.h"
#include "epilogue.hpp"
#include "errors.hpp"

namespace aitamd {
namespace {

// ids = the reference's FuncEnum values (compiler/ops/common/epilogue.py:34-70)
enum ElementwiseFunc : int {
  kAdd = 1, kSub = 2, kMul = 3, kDiv = 4, kTanh = 5, kCos = 6, kSin = 7, kSign = 8, kAbs = 9, kLog = 10, kExp = 11,
  kSqrt = 12, kMax = 13, kMin = 14, kSigmoid = 15, kLeakyRelu = 16, kRelu = 18, kSilu = 21, kPow = 22, kGelu = 23,
  kFastGelu = 24, kSoftsign = 27, kFloor = 30, kLog1p = 31, kReciprocal = 32,
};

constexpr bool is_binary(int f) {
  return f == kAdd || f == kSub || f == kMul || f == kDiv || f == kMax || f == kMin || f == kLeakyRelu || f == kPow;
}
constexpr bool is_unary(int f) {
  return f == kTanh || f == kCos || f == kSin || f == kSign || f == kAbs || f == kLog || f == kExp || f == kSqrt ||
      f == kSigmoid || f == kRelu || f == kSilu || f == kGelu || f == kFastGelu || f == kSoftsign || f == kFloor ||
      f == kLog1p || f == kReciprocal;
}

template <int F>
AITAMD_DEVICE float apply(float x, float y) {
  if constexpr (F == kAdd) return x + y;
  if constexpr (F == kSub) return x - y;
  if constexpr (F == kMul) return x * y;
  if constexpr (F == kDiv) return x / y;
  // a NaN in either operand gives NaN (the reference's fmaxf_nan / fminf_nan, custom_math.h:282-310)
  if constexpr (F == kMax) return (x != x || y != y) ? __builtin_nanf("") : fmaxf(x, y);
  if constexpr (F == kMin) return (x != x || y != y) ? __builtin_nanf("") : fminf(x, y);
  if constexpr (F == kLeakyRelu) return x > 0.0f ? x : x * y;  // y: the negative slope
  if constexpr (F == kPow) return powf(x, y);
  if constexpr (F == kCos) return cosf(x);
  if constexpr (F == kSin) return sinf(x);
  if constexpr (F == kSign) return (float)(x > 0.0f) - (float)(x < 0.0f);
  if constexpr (F == kLog) return logf(x);
  if constexpr (F == kLog1p) return log1pf(x);
  if constexpr (F == kSoftsign) return x / (1.0f + fabsf(x));
  if constexpr (F == kFloor) return floorf(x);
  if constexpr (F == kReciprocal) return 1.0f / x;
  if constexpr (F == kTanh) return tanh_f(x);
  if constexpr (F == kAbs) return fabsf(x);
  if constexpr (F == kExp) return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
  if constexpr (F == kSqrt) return sqrtf(x);
  if constexpr (F == kSigmoid) return sigmoid_f(x);
  if constexpr (F == kRelu) return x > 0.0f ? x : 0.0f;  // NaN -> 0, like the reference's relu (custom_math.h:117)
  if constexpr (F == kSilu) return x * sigmoid_f(x);
  if constexpr (F == kGelu) return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
  if constexpr (F == kFastGelu) return gelu_tanh(x);
  return x;
}

struct ElementwiseParams {
  const void* a;
  const void* b;  // null: b_value
  void* out;
  int64_t numel;
  int64_t b_period;
  float b_value;
  int swap;  // f(b, a) instead of f(a, b)
};

// VEC: 8 elements per lane and step (numel, b_period multiples of 8 or b a single value; 16-byte aligned pointers)
template <class T, int F, bool VEC>
__global__ void __launch_bounds__(256) elementwise_kernel(const ElementwiseParams p) {
  using Tr = ElemTraits<T>;
  using vec8 = typename Tr::vec8;
  const T* a = reinterpret_cast<const T*>(p.a);
  const T* b = reinterpret_cast<const T*>(p.b);
  T* out = reinterpret_cast<T*>(p.out);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const bool b_single = b == nullptr || p.b_period == 1;
  const bool b_full = p.b_period == p.numel;       // same shape: no wrap
  const bool narrow = p.numel < (1ll << 31);       // 32-bit remainder instead of the 64-bit one
  auto wrap = [&](int64_t i) -> int64_t {
    if (b_full) return i;
    return narrow ? (int64_t)((uint32_t)i % (uint32_t)p.b_period) : i % p.b_period;
  };
  const float b_one = b == nullptr ? p.b_value : (is_binary(F) ? Tr::to_float(b[0]) : 0.0f);
  if constexpr (VEC) {
    for (int64_t i = tid; i < p.numel / 8; i += stride) {
      const vec8 av = *reinterpret_cast<const vec8*>(a + i * 8);
      vec8 bv = {};
      if (is_binary(F) && !b_single) bv = *reinterpret_cast<const vec8*>(b + wrap(i * 8));
      vec8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = Tr::to_float(av[j]);
        const float y = b_single ? b_one : Tr::to_float(bv[j]);
        o[j] = Tr::from_float(p.swap ? apply<F>(y, x) : apply<F>(x, y));
      }
      *reinterpret_cast<vec8*>(out + i * 8) = o;
    }
  } else {
    for (int64_t i = tid; i < p.numel; i += stride) {
      const float x = Tr::to_float(a[i]);
      const float y = b_single ? b_one : Tr::to_float(b[wrap(i)]);
      out[i] = Tr::from_float(p.swap ? apply<F>(y, x) : apply<F>(x, y));
    }
  }
}

template <class T, int F>
hipError_t launch(const ElementwiseParams& p, hipStream_t stream) {
  const bool aligned = ((reinterpret_cast<uintptr_t>(p.a) | reinterpret_cast<uintptr_t>(p.out) |
                         reinterpret_cast<uintptr_t>(p.b)) & 15) == 0;
  const bool b_ok = p.b == nullptr || p.b_period == 1 || p.b_period % 8 == 0;
  const bool vec = aligned && b_ok && p.numel % 8 == 0;
  const int64_t items = vec ? p.numel / 8 : p.numel;
  int64_t blocks = (items + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;  // grid-stride beyond 32 workgroups per CU
  if (blocks < 1) blocks = 1;
  if (vec)
    hipLaunchKernelGGL((elementwise_kernel<T, F, true>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((elementwise_kernel<T, F, false>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
  return hipGetLastError();
}

template <class T>
hipError_t dispatch(int func, const ElementwiseParams& p, hipStream_t stream) {
  switch (func) {
#define AITAMD_EW_CASE(F) \
  case F:                 \
    return launch<T, F>(p, stream);
    AITAMD_EW_CASE(kAdd)
    AITAMD_EW_CASE(kSub)
    AITAMD_EW_CASE(kMul)
    AITAMD_EW_CASE(kDiv)
    AITAMD_EW_CASE(kTanh)
    AITAMD_EW_CASE(kAbs)
    AITAMD_EW_CASE(kExp)
    AITAMD_EW_CASE(kSqrt)
    AITAMD_EW_CASE(kMax)
    AITAMD_EW_CASE(kMin)
    AITAMD_EW_CASE(kSigmoid)
    AITAMD_EW_CASE(kRelu)
    AITAMD_EW_CASE(kSilu)
    AITAMD_EW_CASE(kGelu)
    AITAMD_EW_CASE(kFastGelu)
    AITAMD_EW_CASE(kCos)
    AITAMD_EW_CASE(kSin)
    AITAMD_EW_CASE(kSign)
    AITAMD_EW_CASE(kLog)
    AITAMD_EW_CASE(kLeakyRelu)
    AITAMD_EW_CASE(kPow)
    AITAMD_EW_CASE(kSoftsign)
    AITAMD_EW_CASE(kFloor)
    AITAMD_EW_CASE(kLog1p)
    AITAMD_EW_CASE(kReciprocal)
#undef AITAMD_EW_CASE
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace
}  // namespace aitamd

using namespace aitamd;

extern "C" int aitamd_elementwise_supported(int func) { return (is_binary(func) || is_unary(func)) ? 1 : 0; }

extern "C" int aitamd_elementwise(int func, int dtype, const void* a, const void* b, void* out, int64_t numel,
                                  int64_t b_period, float b_value, int swap_operands, void* stream) {
  if (dtype != 0 && dtype != 1) return fail("aitamd_elementwise: bad dtype %d", dtype);
  if (!is_binary(func) && !is_unary(func)) return fail("aitamd_elementwise: function %d is not supported", func);
  if (numel < 0) return fail("aitamd_elementwise: negative size");
  if (numel == 0) return 0;
  if (!a || !out) return fail("aitamd_elementwise: null pointer");
  if (is_unary(func)) {
    b = nullptr;
    b_period = 1;
  } else if (b != nullptr && (b_period < 1 || numel % b_period != 0)) {
    return fail("aitamd_elementwise: the second operand's %lld elements do not tile the output's %lld", (long long)b_period,
                (long long)numel);
  }
  ElementwiseParams p{a, b, out, numel, b != nullptr ? b_period : 1, b_value, swap_operands ? 1 : 0};
  const hipError_t e = dtype == 0 ? dispatch<f16>(func, p, reinterpret_cast<hipStream_t>(stream))
                                  : dispatch<bf16>(func, p, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail("aitamd_elementwise: launch failed: %s", hipGetErrorString(e));
  return 0;
}

// ---- strided row copy ----------------------------------------------------------------------------------------
// The copy a split or a concatenate needs when no GEMM-family op can take the piece as a view: `rows` rows of
// `row_bytes` bytes from src (rows `src_pitch` bytes apart) to dst (rows `dst_pitch` bytes apart).  Takes the place
// of the reference's generated split and concatenate kernels (python/aitemplate/backend/common/split_common.py,
// concatenate_common.py, instantiated by backend/rocm/tensor/split.py and concatenate.py).  Bound: HBM, 2 x
// rows x row_bytes; 16, 4 or 2 bytes per lane and access, whichever pointers, pitches and row length allow.
namespace aitamd {
namespace {

template <class V>
__global__ void __launch_bounds__(256) copy_rows_kernel(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst,
                                                       int64_t rows, int64_t row_units, int64_t src_pitch, int64_t dst_pitch) {
  // grid.x walks a row in units of V, grid.y (and a stride loop) the rows
  const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (u >= row_units) return;
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y)
    reinterpret_cast<V*>(dst + r * dst_pitch)[u] = reinterpret_cast<const V*>(src + r * src_pitch)[u];
}

// rows shorter than a workgroup: consecutive lanes run on through the rows (one division per lane)
template <class V>
__global__ void __launch_bounds__(256) copy_short_rows_kernel(const unsigned char* __restrict__ src,
                                                             unsigned char* __restrict__ dst, int64_t total_units,
                                                             uint32_t row_units, int64_t src_pitch, int64_t dst_pitch) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total_units; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / row_units;
    const int64_t u = i - r * row_units;
    reinterpret_cast<V*>(dst + r * dst_pitch)[u] = reinterpret_cast<const V*>(src + r * src_pitch)[u];
  }
}

template <class V>
hipError_t launch_copy_rows(const void* src, void* dst, int64_t rows, int64_t row_bytes, int64_t src_pitch,
                            int64_t dst_pitch, hipStream_t stream) {
  const int64_t units = row_bytes / (int64_t)sizeof(V);
  if (units < 256) {
    const int64_t total = rows * units;
    const int64_t blocks = (total + 255) / 256;
    hipLaunchKernelGGL(copy_short_rows_kernel<V>, dim3((unsigned)(blocks < (1 << 20) ? blocks : (1 << 20))), dim3(256), 0,
                       stream, static_cast<const unsigned char*>(src), static_cast<unsigned char*>(dst), total,
                       (uint32_t)units, src_pitch, dst_pitch);
    return hipGetLastError();
  }
  const int64_t gx = (units + 255) / 256;
  const int64_t gy = rows < 65535 ? rows : 65535;
  hipLaunchKernelGGL(copy_rows_kernel<V>, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, stream,
                     static_cast<const unsigned char*>(src), static_cast<unsigned char*>(dst), rows, units, src_pitch,
                     dst_pitch);
  return hipGetLastError();
}

}  // namespace
}  // namespace aitamd

extern "C" int aitamd_copy_rows(const void* src, void* dst, int64_t rows, int64_t row_bytes, int64_t src_pitch_bytes,
                                int64_t dst_pitch_bytes, void* stream) {
  using namespace aitamd;
  if (rows < 0 || row_bytes < 0) return fail("aitamd_copy_rows: negative size");
  if (rows == 0 || row_bytes == 0) return 0;
  if (!src || !dst) return fail("aitamd_copy_rows: null pointer");
  if (src_pitch_bytes < row_bytes || dst_pitch_bytes < row_bytes)
    return fail("aitamd_copy_rows: a row pitch (%lld, %lld) is smaller than the row (%lld bytes)",
                (long long)src_pitch_bytes, (long long)dst_pitch_bytes, (long long)row_bytes);
  if ((row_bytes + 255) / 256 > 0x7fffffffll) return fail("aitamd_copy_rows: row too long");
  const uintptr_t all = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | (uintptr_t)row_bytes |
      (uintptr_t)src_pitch_bytes | (uintptr_t)dst_pitch_bytes;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipError_t e;
  if ((all & 15) == 0)
    e = launch_copy_rows<uint4>(src, dst, rows, row_bytes, src_pitch_bytes, dst_pitch_bytes, s);
  else if ((all & 3) == 0)
    e = launch_copy_rows<uint32_t>(src, dst, rows, row_bytes, src_pitch_bytes, dst_pitch_bytes, s);
  else if ((all & 1) == 0)
    e = launch_copy_rows<uint16_t>(src, dst, rows, row_bytes, src_pitch_bytes, dst_pitch_bytes, s);
  else
    e = launch_copy_rows<unsigned char>(src, dst, rows, row_bytes, src_pitch_bytes, dst_pitch_bytes, s);
  if (e != hipSuccess) return fail("aitamd_copy_rows: launch failed: %s", hipGetErrorString(e));
  return 0;
}
