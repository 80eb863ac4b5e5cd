// RCR GEMM / batched GEMM for gfx950:  C[b][m][n] = epi( sum_k A[b][m][k] * B[b][n][k] ).
// A is row-major [M,K], B is row-major [N,K] (so both operands are K-contiguous),
// C is row-major [M,N]; fp16 or bf16 in/out, fp32 accumulate.
//
// One workgroup owns a BM x BN output tile.  Per BK-slab of K:
//   global --(128-bit buffer loads, zero-filled past M/N/K)--> registers
//          --(128-bit ds_write, XOR-swizzled 16-byte chunks)--> LDS (2 stages)
//          --(128-bit ds_read)--> v_mfma_f32_32x32x16 operand fragments.
// The slab for step k+1 is in flight from HBM/L2 while step k is multiplied.
// The MFMA is issued with the operands swapped (B fragment first), so each lane
// ends up holding 4 consecutive output columns of one row: bias / residual
// loads and the output store are 8-byte vector accesses straight from the
// accumulator registers, with the epilogue evaluated in fp32 in between.
//
// Replaces the Composable Kernel device ops the reference instantiates for this
// family (python/aitemplate/utils/mk_ck_lib/gemm_operation.py:56-66, tile table
// python/aitemplate/utils/mk_ck_lib/generator.py:517-601,604-785,788-861).
#pragma once

#include "common.hpp"
#include "epilogue.hpp"

namespace aitamd {

struct GemmParams {
  const void* a;
  const void* b;
  void* c;
  const void* bias;  // [N]
  const void* d0;    // [M, ldd]
  const void* d1;    // [M, ldd]
  int32_t M, N, K;
  int32_t batch;
  int64_t lda, ldb, ldc, ldd;  // row pitches, in elements
  int64_t sa, sb, sc, sd;      // batch strides, in elements (0 broadcasts)
  int32_t tiles_m, tiles_n;
  // Permuted store (kernels built with PERM; perm_on tells the launcher to pick them).  The row index splits as
  // m = (m0 * perm_m1 + m1) * perm_m2 + m2 and the column index as n = (n0 * perm_n1 + n1) * perm_n2 + n2,
  // and C[m, n] goes to element m0*sm0 + m1*sm1 + m2*sm2 + n0*sn0 + n1*sn1 + n2 of a contiguous buffer.
  // That covers the reference's 5-D output permutations
  // (python/aitemplate/backend/rocm/gemm/permute_common.py:20-130): "m2n3" has perm_m2 = 1, "m3n2" perm_n1 = 1.
  int32_t perm_on, perm_m1, perm_m2, perm_n1, perm_n2;
  int64_t perm_sm0, perm_sm1, perm_sm2, perm_sn0, perm_sn1;
  // Non-zero: the output is written with streaming (non-temporal) stores.  Set by the launcher for outputs
  // too large to be still cached when a consumer runs; such stores do not push the operand tiles out of
  // the L2 and reach HBM at a higher rate (bmm_rcr 768x384x384x64: 4.1 -> 6.4 TB/s).
  int32_t nt_store;
  // Batched output whose batch index splits as b = b0 * batch_inner + b1 (0: plain batch stride sc): batch b
  // starts at element b0 * sc_outer + b1 * sc.  This is the [B/d1, d1, M, N] -> [B/d1, M, d1, N] store of
  // bmm_rcr_permute with batch_inner = d1, sc = N, sc_outer = M * d1 * N and ldc = d1 * N.
  int32_t batch_inner;
  int64_t sc_outer;
  // operand layout: 0 rcr (A [M, K], B [N, K]), 1 rrr (B [K, N]), 2 ccr (A [K, M]), 3 crr (both); lda / ldb
  // are the row pitches of the matrices as stored
  int32_t layout;
  // Scratch memory of the split-K instances (null for every other instance): arrival counters, then slots for
  // fp32 partial tiles; see gemm_kernel_dma.hpp.  The counters are zero before a launch and zero after it.
  void* ws;
  int64_t ws_bytes;
  int32_t split_k;  // number of workgroups that share a tile along K (set by the launcher of a split-K instance)
  // Persistent kernels, one batch: when non-zero, XCD x owns the block of tiles_n / xcd_cols tile columns number
  // x % xcd_cols and tiles_m * xcd_cols / 8 tile rows number x / xcd_cols, and walks it row by row (see
  // map_tile_block).  Set by the launcher where the grid divides so and a block's B panels fit half an L2.
  int32_t xcd_cols;
  // Persistent kernels without the block mapping: tile rows per group of the grouped walk (0: eight).  An XCD's run
  // of consecutive tiles is walked group by group, column by column inside a group.
  int32_t group_m;
};

AITAMD_DEVICE int64_t out_batch_offset(const GemmParams& p, int batch) {
  if (p.batch_inner == 0) return (int64_t)batch * p.sc;
  const int b0 = batch / p.batch_inner;
  return b0 * p.sc_outer + (batch - b0 * p.batch_inner) * p.sc;
}

// Output store of 8 or 16 bytes at element `idx` of the buffer `rc` describes (base `base`).  The streaming
// form is a buffer store with the non-temporal bit; it is a different instruction from the plain store on
// purpose, so that the two branches cannot be folded into one plain store.
template <class T, class V>
AITAMD_DEVICE void store_out(T* base, int64_t idx, V v, bool streaming, __amdgpu_buffer_rsrc_t rc) {
  constexpr int kNonTemporal = 2;
  if (streaming) {
    if constexpr (sizeof(V) == 16)
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rc, (uint32_t)(idx * 2), 0, kNonTemporal);
    else
      __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), rc, (uint32_t)(idx * 2), 0, kNonTemporal);
  } else {
    *reinterpret_cast<V*>(base + idx) = v;
  }
}
// descriptor for store_out: the launcher sets nt_store only when one batch of the output spans < 2 GiB
constexpr uint32_t kStoreRecords = 0x7fffffffu;

// Element index of C[m, n] in the output buffer.  PERM is a template flag rather than a run-time test so
// that the plain kernels carry none of the index arithmetic (in the large tiles the extra live values
// cost registers the main loop needs).  The row and the column parts are separate so that a lane that
// keeps one of them fixed across stores evaluates it once.
template <bool PERM>
AITAMD_DEVICE int64_t out_index(const GemmParams& p, int m, int n) {
  if constexpr (!PERM) {
    return (int64_t)m * p.ldc + n;
  } else {
    const int m01 = m / p.perm_m2, m2 = m - m01 * p.perm_m2;
    const int m0 = m01 / p.perm_m1, m1 = m01 - m0 * p.perm_m1;
    const int n01 = n / p.perm_n2, n2 = n - n01 * p.perm_n2;
    const int n0 = n01 / p.perm_n1, n1 = n01 - n0 * p.perm_n1;
    return (m0 * p.perm_sm0 + m1 * p.perm_sm1 + m2 * p.perm_sm2) + (n0 * p.perm_sn0 + n1 * p.perm_sn1 + n2);
  }
}

// KVEC = number of K-contiguous elements that may be fetched with one load:
// 8 -> 128-bit loads (K % 8 == 0, 16-byte aligned rows), 4/2/1 -> narrower
// pieces for odd K or unaligned views.
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int KVEC_>
struct GemmTile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_;
  static constexpr int WGM = WGM_, WGN = WGN_, KVEC = KVEC_;
  static constexpr int NT = WGM * WGN * kWaveSize;
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;  // per-wave tile
  static constexpr int MI = WTM / 32, NI = WTN / 32;    // 32x32 MFMA blocks per wave
  static constexpr int CPR = BK / 8;                    // 16-byte chunks per LDS row
  static constexpr int RPW = (256 / (BK * 2)) > 0 ? (256 / (BK * 2)) : 1;  // rows per 256-byte bank window
  static constexpr int A_IT = BM * CPR / NT;
  static constexpr int B_IT = BN * CPR / NT;
  static constexpr int ROWS_PER_PASS = NT / CPR;
  static constexpr int kLdsBytes = 2 * (BM + BN) * BK * 2;
  static_assert(BM % (WGM * 32) == 0 && BN % (WGN * 32) == 0, "wave tile must be whole MFMA blocks");
  static_assert(BK % 16 == 0, "BK must be a multiple of the MFMA K");
  static_assert((BM * CPR) % NT == 0 && (BN * CPR) % NT == 0, "loads must divide evenly");
  static_assert(NT % CPR == 0, "a load pass must cover whole rows");
};

// 16-byte chunk `chunk` of LDS row `row` lives at chunk ^ swz(row): any 16
// consecutive rows read at one logical chunk index touch all 64 banks once.
template <class Tile>
AITAMD_DEVICE int lds_chunk_elem(int row, int chunk) {
  const int swz = (row / Tile::RPW) % Tile::CPR;
  return row * Tile::BK + ((chunk ^ swz) << 3);
}

// LAYOUT as in gemm_rcr_dma_kernel (bit 1: A stored [K, M]; bit 0: B stored [K, N]); the element-wide
// loads (KVEC = 1) take any layout, pitch and alignment: the instance of last resort.
template <class T, class Tile, class Epi, bool PERM = false, int LAYOUT = 0>
__global__ void __launch_bounds__(Tile::NT) gemm_rcr_kernel(const GemmParams p) {
  static_assert(LAYOUT == 0 || Tile::KVEC == 1, "only the element-wide loads read operands that are not K-contiguous");
  constexpr bool A_T = (LAYOUT & 2) != 0, B_T = (LAYOUT & 1) != 0;
  using Tr = ElemTraits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int BM = Tile::BM, BN = Tile::BN, BK = Tile::BK;
  constexpr int MI = Tile::MI, NI = Tile::NI;
  constexpr int A_IT = Tile::A_IT, B_IT = Tile::B_IT;
  constexpr int KVEC = Tile::KVEC;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* const sA = reinterpret_cast<T*>(smem_raw);  // [2][BM*BK]
  T* const sB = sA + 2 * BM * BK;                // [2][BN*BK]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / Tile::WGN;
  const int wn = wave % Tile::WGN;
  const int r32 = lane & 31;
  const int h = lane >> 5;

  int batch, tm, tn;
  map_tile<8>(blockIdx.x, p.tiles_m, p.tiles_n, p.batch, batch, tm, tn);
  const int m0 = tm * BM;
  const int n0 = tn * BN;
  const int rows_a = (p.M - m0) < BM ? (p.M - m0) : BM;
  const int rows_b = (p.N - n0) < BN ? (p.N - n0) : BN;

  // Loop-invariant per-thread load coordinates.
  const int ld_row = tid / Tile::CPR;
  const int ld_chunk = tid % Tile::CPR;
  uint32_t a_off[A_IT], b_off[B_IT];
  int a_st[A_IT], b_st[B_IT];
#pragma unroll
  for (int i = 0; i < A_IT; ++i) {
    const int row = ld_row + i * Tile::ROWS_PER_PASS;
    // a transposed operand: element (row, k) lies at k * pitch + row; rows past the tile edge are masked here
    // because they are not past the end of the buffer
    a_off[i] = A_T ? (row < rows_a ? (uint32_t)((ld_chunk * 8 * p.lda + row) * 2) : kOobOffset)
                   : (uint32_t)(((int64_t)row * p.lda + ld_chunk * 8) * 2);
    a_st[i] = lds_chunk_elem<Tile>(row, ld_chunk);
  }
#pragma unroll
  for (int i = 0; i < B_IT; ++i) {
    const int row = ld_row + i * Tile::ROWS_PER_PASS;
    b_off[i] = B_T ? (row < rows_b ? (uint32_t)((ld_chunk * 8 * p.ldb + row) * 2) : kOobOffset)
                   : (uint32_t)(((int64_t)row * p.ldb + ld_chunk * 8) * 2);
    b_st[i] = lds_chunk_elem<Tile>(row, ld_chunk);
  }

  // Loop-invariant fragment read positions (elements), one per 16-wide k step.
  constexpr int KK = BK / 16;
  int a_rd[KK], b_rd[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    a_rd[kk] = lds_chunk_elem<Tile>(wm * Tile::WTM + r32, kk * 2 + h);
    b_rd[kk] = lds_chunk_elem<Tile>(wn * Tile::WTN + r32, kk * 2 + h);
  }

  const int k_tiles = (p.K + BK - 1) / BK;

  {
    const T* Ab = reinterpret_cast<const T*>(p.a) + (int64_t)batch * p.sa + (A_T ? (int64_t)m0 : (int64_t)m0 * p.lda);
    const T* Bb = reinterpret_cast<const T*>(p.b) + (int64_t)batch * p.sb + (B_T ? (int64_t)n0 : (int64_t)n0 * p.ldb);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(
        Ab, clamp_records((A_T ? ((int64_t)p.K - 1) * p.lda + rows_a : ((int64_t)rows_a - 1) * p.lda + p.K) * 2));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(
        Bb, clamp_records((B_T ? ((int64_t)p.K - 1) * p.ldb + rows_b : ((int64_t)rows_b - 1) * p.ldb + p.K) * 2));

    u32x4 ga[A_IT], gb[B_IT];

    auto load_global = [&](int k0) {
      if constexpr (KVEC == 8) {
        const uint32_t kadd = (k0 + ld_chunk * 8 < p.K) ? (uint32_t)(k0 * 2) : kOobOffset;
#pragma unroll
        for (int i = 0; i < A_IT; ++i) ga[i] = buffer_load_16B(ra, a_off[i] + kadd);
#pragma unroll
        for (int i = 0; i < B_IT; ++i) gb[i] = buffer_load_16B(rb, b_off[i] + kadd);
      } else {
        constexpr int PIECES = 8 / KVEC;
        auto load_pieces = [&](const __amdgpu_buffer_rsrc_t& r, uint32_t base, bool transposed, int64_t pitch) {
          union {
            u32x4 v;
            uint16_t s[8];
            uint32_t w[4];
          } u;
#pragma unroll
          for (int j = 0; j < PIECES; ++j) {
            const int ke = k0 + ld_chunk * 8 + j * KVEC;
            const uint32_t step = transposed ? (uint32_t)((k0 + j * KVEC) * pitch * 2) : (uint32_t)((k0 + j * KVEC) * 2);
            const uint32_t off = (ke < p.K && base != kOobOffset) ? base + step : kOobOffset;
            if constexpr (KVEC == 4) {
              const u32x2 t = buffer_load_8B(r, off);
              u.w[2 * j] = t.x;
              u.w[2 * j + 1] = t.y;
            } else if constexpr (KVEC == 2) {
              u.w[j] = buffer_load_4B(r, off);
            } else {
              u.s[j] = buffer_load_2B(r, off);
            }
          }
          return u.v;
        };
#pragma unroll
        for (int i = 0; i < A_IT; ++i) ga[i] = load_pieces(ra, a_off[i], A_T, p.lda);
#pragma unroll
        for (int i = 0; i < B_IT; ++i) gb[i] = load_pieces(rb, b_off[i], B_T, p.ldb);
      }
    };

    auto store_lds = [&](int stage) {
      T* dA = sA + stage * BM * BK;
      T* dB = sB + stage * BN * BK;
#pragma unroll
      for (int i = 0; i < A_IT; ++i) *reinterpret_cast<u32x4*>(dA + a_st[i]) = ga[i];
#pragma unroll
      for (int i = 0; i < B_IT; ++i) *reinterpret_cast<u32x4*>(dB + b_st[i]) = gb[i];
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[mi][ni][e] = 0.0f;

    load_global(0);
    store_lds(0);
    __syncthreads();

    for (int kt = 0; kt < k_tiles; ++kt) {
      const int cur = kt & 1;
      const bool has_next = (kt + 1) < k_tiles;
      if (has_next) load_global((kt + 1) * BK);

      const T* cA = sA + cur * BM * BK;
      const T* cB = sB + cur * BN * BK;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        vec8 af[MI], bf[NI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
          af[mi] = *reinterpret_cast<const vec8*>(cA + a_rd[kk] + mi * 32 * BK);
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
          bf[ni] = *reinterpret_cast<const vec8*>(cB + b_rd[kk] + ni * 32 * BK);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int ni = 0; ni < NI; ++ni)
            acc[mi][ni] = Tr::mfma32(bf[ni], af[mi], acc[mi][ni]);
      }

      if (has_next) store_lds(cur ^ 1);
      __syncthreads();
    }

    // ---------------- epilogue: registers -> fp32 math -> 8-byte stores -------------
    T* Cb = reinterpret_cast<T*>(p.c) + out_batch_offset(p, batch);
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(Cb, kStoreRecords);
    const T* D0b = Epi::kNumD >= 1 ? reinterpret_cast<const T*>(p.d0) + (int64_t)batch * p.sd : nullptr;
    const T* D1b = Epi::kNumD >= 2 ? reinterpret_cast<const T*>(p.d1) + (int64_t)batch * p.sd : nullptr;
    const T* bias = reinterpret_cast<const T*>(p.bias);

    // vector form for the lanes whose 4 columns lie inside the row: multi-dword global and buffer accesses need
    // dword alignment only, so even pitches and 4-byte aligned pointers are enough
    bool vec_ok = ((p.ldc & 1) == 0) && ((p.sc & 1) == 0) && (!PERM || ((p.perm_n2 & 3) == 0 && (p.N & 3) == 0)) &&
        ((reinterpret_cast<uintptr_t>(p.c) & 3) == 0);
    if (Epi::kHasBias) vec_ok = vec_ok && ((reinterpret_cast<uintptr_t>(p.bias) & 3) == 0);
    if (Epi::kNumD >= 1)
      vec_ok = vec_ok && ((p.ldd & 1) == 0) && ((p.sd & 1) == 0) && ((reinterpret_cast<uintptr_t>(p.d0) & 3) == 0);
    if (Epi::kNumD >= 2) vec_ok = vec_ok && ((reinterpret_cast<uintptr_t>(p.d1) & 3) == 0);

    using vec4 = typename Tr::vec4;
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      const int m = m0 + wm * Tile::WTM + mi * 32 + r32;
      if (m >= p.M) continue;
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = n0 + wn * Tile::WTN + ni * 32 + g * 8 + h * 4;
          if (n >= p.N) continue;
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = acc[mi][ni][g * 4 + j];
          const int64_t c_idx = out_index<PERM>(p, m, n);
          const int64_t d_idx = (int64_t)m * p.ldd + n;
          if (vec_ok && n + 4 <= p.N) {
            vec4 bv = {}, d0v = {}, d1v = {};
            if constexpr (Epi::kHasBias) bv = *reinterpret_cast<const vec4*>(bias + n);
            if constexpr (Epi::kNumD >= 1) d0v = *reinterpret_cast<const vec4*>(D0b + d_idx);
            if constexpr (Epi::kNumD >= 2) d1v = *reinterpret_cast<const vec4*>(D1b + d_idx);
            vec4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j)
              o[j] = Tr::from_float(
                  Epi::apply(v[j], Tr::to_float(bv[j]), Tr::to_float(d0v[j]), Tr::to_float(d1v[j])));
            // always cached: these are 8-byte pieces in the MFMA's own layout, and streaming stores of partial
            // lines reach memory at a third of the rate the L2 gets by merging them (300000x64x64: 80 us against 25)
            store_out(Cb, c_idx, o, false, rc);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if (n + j < p.N) {
                float bj = 0.f, d0j = 0.f, d1j = 0.f;
                if constexpr (Epi::kHasBias) bj = Tr::to_float(bias[n + j]);
                if constexpr (Epi::kNumD >= 1) d0j = Tr::to_float(D0b[d_idx + j]);
                if constexpr (Epi::kNumD >= 2) d1j = Tr::to_float(D1b[d_idx + j]);
                Cb[out_index<PERM>(p, m, n + j)] = Tr::from_float(Epi::apply(v[j], bj, d0j, d1j));
              }
            }
          }
        }
      }
    }
  }
}

}  // namespace aitamd
