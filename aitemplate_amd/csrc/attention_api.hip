// C ABI launcher of the fused attention kernel (bmm_softmax_bmm_permute).
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/aitemplate_amd_kernels.h"
#include "attention_kernel.hpp"
#include "errors.hpp"

namespace aitamd {
namespace {

constexpr int kMaxDevices = 64;

// Variant forced by aitamd_attention_set_variant: -1 automatic, 0..3 a MODE below.  The environment variable
// AITAMD_ATTN_MODE gives the initial value and is read once, not on every launch.
constexpr int kVariantUnset = -2;
std::atomic<int> g_forced_variant{kVariantUnset};
int forced_variant() {
  int m = g_forced_variant.load(std::memory_order_relaxed);
  if (m == kVariantUnset) {
    const char* env = getenv("AITAMD_ATTN_MODE");
    const int from_env = env ? atoi(env) : -1;
    g_forced_variant.compare_exchange_strong(m, from_env >= 0 && from_env <= 3 ? from_env : -1);
    m = g_forced_variant.load(std::memory_order_relaxed);
  }
  return m;
}

// MODE 0: four waves (128 query rows), two LDS stages, two workgroups per CU.
// MODE 1: eight waves (256 query rows) share each K / V tile and four LDS stages keep three tiles in flight.
// MODE 2: as 1 with two groups of eight waves that take alternate tiles (sixteen waves per CU).
template <int KS, int OT, int MODE>
struct TileOf {
  using type = AttnTile<KS, OT>;
};
constexpr int wide_bn(int ks, int ot) { return (16 * ks + 32 * ot) <= 128 ? 128 : 64; }
constexpr bool wide_fits(int ks, int ot) {  // four stages of the wide tile within the LDS
  return 4 * wide_bn(ks, ot) * (16 * ks + 8 + 32 * ot) * 2 <= 160 * 1024;
}
template <int KS, int OT, bool FITS = wide_fits(KS, OT)>
struct WideTile {  // head dims too large for the wide forms keep the four-wave tile
  using one = AttnTile<KS, OT>;
  using two = AttnTile<KS, OT>;
};
template <int KS, int OT>
struct WideTile<KS, OT, true> {
  using one = AttnTile<KS, OT, wide_bn(KS, OT), 8, 4>;
  // (two groups only where the merge fits the ring's memory: the small head dims this mode is chosen for)
  static constexpr bool kMergeFits = (16 * KS + 32 * OT) <= 128 && (16 * OT + 2) * 8 * 64 * 4 <= one::kLdsBytes;
  using two = AttnTile<KS, OT, wide_bn(KS, OT), 8, 4, kMergeFits ? 2 : 1>;
};
template <int KS, int OT>
struct TileOf<KS, OT, 1> {
  using type = typename WideTile<KS, OT>::one;
};
template <int KS, int OT>
struct TileOf<KS, OT, 2> {
  using type = typename WideTile<KS, OT>::two;
};

// MODE 3: as 0 with two groups of four waves on alternate tiles and four LDS stages: for grids that leave CUs idle.
template <int KS, int OT>
struct TileOf<KS, OT, 3> {
  using Base = AttnTile<KS, OT>;
  static constexpr bool kFits = (16 * OT + 2) * 4 * 64 * 4 <= 2 * Base::kLdsBytes && 2 * Base::kLdsBytes <= 160 * 1024;
  using type = AttnTile<KS, OT, Base::BN, 4, kFits ? 4 : 2, kFits ? 2 : 1>;
};

template <class T, int KS, int OT, bool VEC, bool DMA, int MODE>
hipError_t launch_attention(const AttnParams& p, hipStream_t stream) {
  using Tile = typename TileOf<KS, OT, MODE>::type;
  auto kernel = attention_kernel<T, Tile, VEC, DMA>;
  static std::once_flag once[kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  // the outcome is kept per device: a failed opt-in must fail every later call too, not only the first
  static hipError_t attr_errs[kMaxDevices];
  hipError_t& attr_err = attr_errs[dev % kMaxDevices];
  std::call_once(once[dev % kMaxDevices], [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, Tile::kLdsBytes);
  });
  if (attr_err != hipSuccess) return attr_err;
  const int64_t m_tiles = (p.M + Tile::BM - 1) / Tile::BM;
  dim3 grid((unsigned)m_tiles, (unsigned)(p.B < 65535 ? p.B : 65535), 1);
  hipLaunchKernelGGL(kernel, grid, dim3(Tile::NT), Tile::kLdsBytes, stream, p);
  return hipGetLastError();
}

typedef hipError_t (*AttnLaunch)(const AttnParams&, hipStream_t);

template <class T, bool VEC, bool DMA, int MODE>
AttnLaunch pick(int ks, int ot) {
#define AITAMD_ATTN_CASE(KS, OT) \
  if (ks <= KS && ot <= OT) return &launch_attention<T, KS, OT, VEC, DMA, MODE>;
  // smallest padded head dims first; (K <= 16 KS, O <= 32 OT)
  AITAMD_ATTN_CASE(2, 1)
  AITAMD_ATTN_CASE(3, 2)
  AITAMD_ATTN_CASE(4, 2)
  AITAMD_ATTN_CASE(4, 4)
  AITAMD_ATTN_CASE(6, 3)
  AITAMD_ATTN_CASE(8, 4)
  AITAMD_ATTN_CASE(10, 5)  // head dim 160: the deepest attention of Stable Diffusion v1 (1280 channels, 8 heads)
#undef AITAMD_ATTN_CASE
  return nullptr;
}

// x rounded to the nearest fp16 (dtype 0) or bf16 value, ties to even, as a float.  Done on the bits: host-side
// conversions through _Float16 / __bf16 would call compiler-runtime routines that a model library linked by the
// host C++ compiler does not have.
float round_to_elem(float x, int dtype) {
  uint32_t u;
  memcpy(&u, &x, 4);
  const uint32_t sign = u & 0x80000000u, mag = u & 0x7fffffffu;
  if (mag >= 0x7f800000u) return x;  // infinities and NaNs stay what they are
  uint32_t r;
  if (dtype != 0) {
    r = mag + 0x7fffu + ((mag >> 16) & 1u);  // keep 8 bits of mantissa
    r &= 0xffff0000u;
  } else {
    const int e = (int)(mag >> 23) - 127;
    if (e > 15) {
      r = 0x7f800000u;  // beyond the largest half
    } else if (e >= -14) {
      r = mag + 0xfffu + ((mag >> 13) & 1u);  // normal half: keep 10 bits of mantissa
      r &= 0xffffe000u;
      if (r >= 0x47800000u) r = 0x7f800000u;  // rounded up past 65504
    } else {
      // subnormal half: a multiple of 2^-24
      float f;
      memcpy(&f, &mag, 4);
      const float q = f * 16777216.0f;          // exact scaling
      const float n = __builtin_rintf(q);       // ties to even in the default rounding mode
      f = n * (1.0f / 16777216.0f);
      memcpy(&r, &f, 4);
    }
  }
  r |= sign;
  float out;
  memcpy(&out, &r, 4);
  return out;
}

}  // namespace
}  // namespace aitamd

using namespace aitamd;

namespace {

int attention_entry(const char* who, int dtype, const void* q, const void* k, const void* v, void* out, int64_t B,
                    int64_t M, int64_t N, int64_t K, int64_t O, int64_t G, float scale, int causal,
                    const int32_t* kv_len, const int32_t* q_len, bool nan_reset, void* stream) {
  if (dtype != 0 && dtype != 1) return fail("%s: bad dtype %d", who, dtype);
  if (B < 0 || M < 0 || N < 0 || K < 0 || O < 0) return fail("%s: negative dimension", who);
  if (G <= 0 || (B % G) != 0) return fail("%s: batch %lld is not a multiple of heads %lld", who,
                                          (long long)B, (long long)G);
  if (B == 0 || M == 0 || O == 0) return 0;
  if (B > 0x7fffffffll || M > 0x7fffffffll || N > 0x7fffffffll) return fail("%s: dimension too large", who);
  if (K > 160 || O > 160) return fail("%s: head dims above 160 are not supported (K=%lld O=%lld)", who,
                                      (long long)K, (long long)O);
  if (!out || (N > 0 && (!q || !k || !v))) return fail("%s: null pointer", who);
  AttnParams p{};
  p.q = q;
  p.k = k;
  p.v = v;
  p.out = out;
  p.B = (int32_t)B;
  p.M = (int32_t)M;
  p.N = (int32_t)N;
  p.K = (int32_t)K;
  p.O = (int32_t)O;
  p.G = (int32_t)G;
  // the reference hands alpha to its kernel in the element type
  // (python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:47-51)
  p.scale_log2e = round_to_elem(scale, dtype) * 1.4426950408889634f;
  p.causal = causal ? 1 : 0;
  p.kv_len = kv_len;
  p.q_len = q_len;
  p.nan_reset = nan_reset ? 1 : 0;
  const int ks = (int)((K + 15) / 16) > 0 ? (int)((K + 15) / 16) : 1;
  const int ot = (int)((O + 31) / 32);
  const bool vec = (K % 8 == 0) && (O % 8 == 0) && ((reinterpret_cast<uintptr_t>(q) & 15) == 0) &&
      ((reinterpret_cast<uintptr_t>(k) & 15) == 0) && ((reinterpret_cast<uintptr_t>(v) & 15) == 0);
  // direct-to-LDS tiles address K and V of one batch entry with 32-bit byte offsets
  const int64_t kv_dim = K > O ? K : O;
  // (tiles are issued up to three past the last one, hence the slack)
  const bool dma = vec && (N + 4 * 128) * kv_dim * 2 < 0x7fffffffll;
  // 256-row workgroups for small head dims (where re-streaming K / V per 128 query rows costs most; measured
  // slower at head dims 64 and 128) once there are enough of them to fill the CUs
  const bool wide = dma && (16 * ks + 32 * ot) <= 112 && ((M + 255) / 256) * B >= 256;
  // two wave groups pay when a CU holds one workgroup anyway: measured 4.5 % faster with 256 workgroups
  // (16 heads x 4096 rows, head dim 40), 2 % slower with 512
  // (wave groups take alternate key tiles: with fewer than four tiles there is nothing to share out - the 77 text
  // tokens of a cross-attention are a single tile)
  const int64_t bn = (16 * ks + 32 * ot) <= 112 ? 128 : 64;
  const bool groups_pay = N >= 4 * bn;
  int mode = wide ? ((((M + 255) / 256) * B <= 256 && groups_pay) ? 2 : 1) : 0;
  // grids of 128-row workgroups that leave CUs idle take the two-group form of those too: 8-19 % faster from 48 to
  // 256 workgroups (head dims 40 and 64), 7 % slower at 384
  if (mode == 0 && dma && groups_pay && ((M + 127) / 128) * B <= 256) mode = 3;
  // head dim 64: the 256-row form with two wave groups when its grid is at most one workgroup per CU (and the
  // 128-row grid is too large for the rule above): 5-10 % faster on 4 x 16384^2, 8 x 8192^2, 16 x 4096^2, 32 x 2048^2;
  // no gain from 512 workgroups on
  if (mode == 0 && dma && groups_pay && (16 * ks + 32 * ot) <= 128 && ((M + 255) / 256) * B <= 256) mode = 2;
  // aitamd_attention_set_variant(0|1|2|3) forces a variant where the shape allows it (a test and measurement knob)
  {
    const int m = forced_variant();
    if (m >= 0 && m <= 2 && dma && (16 * ks + 32 * ot) <= 128) mode = m;
    if (m == 3 && dma) mode = 3;
  }
  AttnLaunch fn = nullptr;
  if (dtype == 0)
    fn = mode == 3 ? pick<f16, true, true, 3>(ks, ot)
       : mode == 2 ? pick<f16, true, true, 2>(ks, ot)
                   : (mode == 1 ? pick<f16, true, true, 1>(ks, ot)
                                : (dma ? pick<f16, true, true, 0>(ks, ot)
                                       : (vec ? pick<f16, true, false, 0>(ks, ot) : pick<f16, false, false, 0>(ks, ot))));
  else
    fn = mode == 3 ? pick<bf16, true, true, 3>(ks, ot)
       : mode == 2 ? pick<bf16, true, true, 2>(ks, ot)
                   : (mode == 1 ? pick<bf16, true, true, 1>(ks, ot)
                                : (dma ? pick<bf16, true, true, 0>(ks, ot)
                                       : (vec ? pick<bf16, true, false, 0>(ks, ot) : pick<bf16, false, false, 0>(ks, ot))));
  if (!fn) return fail("%s: no instance for K=%lld O=%lld", who, (long long)K, (long long)O);
  const hipError_t e = fn(p, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail("%s: launch failed: %s", who, hipGetErrorString(e));
  return 0;
}

}  // namespace

extern "C" int aitamd_attention_set_variant(int variant) {
  if (variant < -1 || variant > 3) return fail("aitamd_attention_set_variant: variant %d is not one of -1, 0, 1, 2, 3", variant);
  g_forced_variant.store(variant, std::memory_order_relaxed);
  return 0;
}

extern "C" int aitamd_bmm_softmax_bmm_permute(int dtype, const void* q, const void* k, const void* v, void* out,
                                              int64_t B, int64_t M, int64_t N, int64_t K, int64_t O, int64_t G,
                                              float scale, int causal, void* stream) {
  // NaN scores count as -inf: the reference gives this op's kernel ScaleAndResetNaNToMinusInfinity
  // (python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:106, bmm_softmax_bmm.py:99)
  return attention_entry("aitamd_bmm_softmax_bmm_permute", dtype, q, k, v, out, B, M, N, K, O, G, scale, causal, nullptr,
                         nullptr, true, stream);
}

extern "C" int aitamd_mem_eff_attention(int dtype, const void* q, const void* k, const void* v, void* out,
                                        int64_t batch, int64_t heads, int64_t seq_q, int64_t seq_kv, int64_t head_dim,
                                        int64_t head_dim_v, float scale, int causal, const int32_t* lengths_kv,
                                        const int32_t* lengths_q, void* stream) {
  if (batch < 0 || heads <= 0) return fail("aitamd_mem_eff_attention: bad batch %lld or heads %lld", (long long)batch,
                                           (long long)heads);
  if (batch > 0x7fffffffll / heads) return fail("aitamd_mem_eff_attention: dimension too large");
  // (a NaN score stays a NaN: the reference's kernel for this op scales only,
  // python/aitemplate/backend/rocm/attention/mem_eff_attention.py:74)
  return attention_entry("aitamd_mem_eff_attention", dtype, q, k, v, out, batch * heads, seq_q, seq_kv, head_dim,
                         head_dim_v, heads, scale, causal, lengths_kv, lengths_q, false, stream);
}
