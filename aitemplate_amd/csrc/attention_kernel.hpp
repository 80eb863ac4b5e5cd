// Fused  out = softmax(scale * Q K^T) V  with the [B,M,O] -> [B/G, M, G, O] permute
// folded into the store (bmm_softmax_bmm_permute), gfx950.
//
// The score matrix never leaves the chip.  One wave owns 32 query rows and walks
// the keys/values in blocks of 32 (64 for the smallest head dims); a workgroup of 4 or
// 8 waves shares each 64- or 128-row K / V tile through LDS, and the 16-wave form runs
// two such groups on alternate tiles of the same rows and merges them at the end.
//
//  * S^T = K Q^T is computed with v_mfma_f32_32x32x16 (K tile rows as the A
//    operand, the wave's Q rows - kept in registers for the whole kernel - as
//    the B operand).  In the accumulator layout of the transposed product a
//    lane holds 16 keys of ONE query row, so the online-softmax state (running
//    max, running sum, rescale factor) is one scalar per lane and the row
//    reductions are 15 in-lane ops plus a single v_permlane32_swap.
//  * The probabilities, rounded to the element type, are already laid out as the
//    B operand of the second MFMA  O^T = V^T P^T : no shuffle, no LDS round trip.
//  * V stays row-major [key][o] in LDS exactly as it sits in memory; the V^T
//    operand fragments are fetched with ds_read_b64_tr_b16 (LDS transpose read).
//  * head dims that are not MFMA multiples (40) are zero-padded inside the LDS
//    tiles only: K to 16*KS columns, V to 32*OT columns.
//
// Replaces DeviceBatchedGemmSoftmaxGemmPermute_Xdl_CShuffle as instantiated by
// the reference (python/aitemplate/utils/mk_ck_lib/gemm_operation.py:64,415-424;
// arguments python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:84-110).
#pragma once

#include <type_traits>

#include "common.hpp"

#ifndef AITAMD_ATTN_FAST
#define AITAMD_ATTN_FAST 1
#endif
#ifndef AITAMD_ATTN_BATCH_READS
#define AITAMD_ATTN_BATCH_READS 0
#endif
#ifndef AITAMD_ATTN_KB
#define AITAMD_ATTN_KB(KS, OT) (((KS) + 2 * (OT)) <= 7 ? 2 : 1)
#endif

namespace aitamd {

struct AttnParams {
  const void* q;  // [B, M, K]
  const void* k;  // [B, N, K]
  const void* v;  // [B, N, O]
  void* out;      // [B / G, M, G, O]
  int32_t B, M, N, K, O, G;
  float scale_log2e;  // scale (already rounded to the element type) * log2(e)
  int32_t causal;
  // Optional, device memory, B / G entries: batch entry b only attends to its first kv_len[b / G] keys (clamped to
  // [0, N]); the later rows of K and V are never read.  Null: all N keys.
  const int32_t* kv_len;
  // Optional, same form: rows m >= q_len[b / G] of batch entry b are written as zeros, and a workgroup whose rows
  // all lie past that length visits no keys.
  const int32_t* q_len;
  // Non-zero: a NaN score counts as -inf (its key is left out of the row's softmax) instead of making the row NaN.
  int32_t nan_reset;
};

// NW_ waves (32 query rows each) share the K / V tiles; NS_ LDS stages.  The register-staged
// loaders use two stages; the direct-to-LDS path keeps NS_ - 1 tiles in flight.
// NG_ groups of NW_ waves each take every NG_-th tile of the same query rows and merge their running
// sums at the end: twice the waves per SIMD for the same K / V traffic.
template <int KS_, int OT_, int BN_ = ((16 * KS_ + 32 * OT_) <= 112 ? 128 : 64), int NW_ = 4, int NS_ = 2, int NG_ = 1>
struct AttnTile {
  static constexpr int KS = KS_;          // K padded to 16 * KS
  static constexpr int OT = OT_;          // O padded to 32 * OT
  static constexpr int KP = 16 * KS;
  static constexpr int OP = 32 * OT;
  static constexpr int NW = NW_, NS = NS_, NG = NG_;
  static constexpr int BM = 32 * NW;      // query rows per workgroup
  static constexpr int BN = BN_;          // keys per LDS tile: 128 while two workgroups still fit one CU's LDS
  static constexpr int NT = 64 * NW * NG;
  static constexpr int K_PITCH = KP + 8;  // halves; keeps 16 consecutive rows on distinct banks
  // V rows carry no pad.  The transposing read fetches, per 32 lanes, 64 bytes of each of 4 consecutive rows; the
  // four pieces have to fall into four different quarters of the 64 banks.  Rows of 64 or 192 bytes do that as
  // they lie; rows of 128 or 256 bytes get the 64-byte pieces of a row exchanged by a row-dependent XOR.
  static constexpr int V_PITCH = OP;
  static constexpr int V_CR = OP / 8;                                             // 16-byte chunks per V row
  static constexpr int V_SWZ_GROUPS = (V_CR == 8 || V_CR == 16) ? V_CR / 4 : 1;  // 64-byte pieces exchanged
  static constexpr int V_SWZ_ROWS = V_CR == 8 ? 2 : 1;                            // rows per 256 bytes
  // chunk index -> chunk index ^ v_swz(row)
  static constexpr int v_swz(int row) { return 4 * ((row / V_SWZ_ROWS) % V_SWZ_GROUPS); }
  static constexpr int K_CHUNKS = BN * KP / 8;  // 16-byte chunks per tile (pads included)
  static constexpr int V_CHUNKS = BN * OP / 8;
  static constexpr int K_IT = (K_CHUNKS + NT - 1) / NT;
  static constexpr int V_IT = (V_CHUNKS + NT - 1) / NT;
  static constexpr int kLdsBytes = NS * BN * (K_PITCH + V_PITCH) * 2;
  static_assert(kLdsBytes <= 160 * 1024, "LDS budget");
  static_assert(NG == 1 || (NS % NG == 0 && NS >= 2 * NG), "the groups' tiles and the next ones in flight need a stage each");
  static_assert(NG == 1 || (16 * OT + 2) * NW * 64 * 4 <= kLdsBytes, "the merge goes through the ring's memory");
};

// LDS transpose read: 4 x 16-bit per lane, gathered across the 16 lanes of a block
template <class T>
struct AttnVec;
template <>
struct AttnVec<f16> {
  typedef __fp16 raw4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
  static AITAMD_DEVICE f16x4 tr_read(const f16* p) {
    const raw4 r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((__attribute__((address_space(3))) raw4*)p);
    return __builtin_bit_cast(f16x4, r);
  }
  static AITAMD_DEVICE f16x4 tr_read(__attribute__((address_space(3))) const f16* p) {
    const raw4 r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((__attribute__((address_space(3))) raw4*)p);
    return __builtin_bit_cast(f16x4, r);
  }
};
template <>
struct AttnVec<bf16> {
  typedef __bf16 raw4 __attribute__((__vector_size__(4 * sizeof(__bf16))));
  static AITAMD_DEVICE bf16x4 tr_read(const bf16* p) {
    const raw4 r = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) raw4*)p);
    return __builtin_bit_cast(bf16x4, r);
  }
  static AITAMD_DEVICE bf16x4 tr_read(__attribute__((address_space(3))) const bf16* p) {
    const raw4 r = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) raw4*)p);
    return __builtin_bit_cast(bf16x4, r);
  }
};

// acc + the 8 elements of v: four v_dot2 against (1, 1) on the packed pairs as they lie in the registers
AITAMD_DEVICE float add_elements(f16x8 v, float acc) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  struct Quads {
    h2 q[4];
  };
  const Quads u = __builtin_bit_cast(Quads, v);
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2(u.q[i], h2{(f16)1.0f, (f16)1.0f}, acc, false);
  return acc;
}
AITAMD_DEVICE float add_elements(bf16x8 v, float acc) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  struct Quads {
    b2 q[4];
  };
  const Quads u = __builtin_bit_cast(Quads, v);
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(u.q[i], b2{(bf16)1.0f, (bf16)1.0f}, acc, false);
  return acc;
}

AITAMD_DEVICE float max_across_halves(float x) {
  // lane l and lane l^32 hold the two halves of one query row
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
AITAMD_DEVICE float sum_across_halves(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// VEC: K and O are multiples of 8 and all base pointers 16-byte aligned -> 128-bit
// loads; otherwise elements are gathered one by one (slow, any shape).
// DMA (needs VEC, and each K / V matrix of a batch entry below 2 GiB): the K / V tiles go
// global -> LDS directly (buffer_load ... lds) instead of through registers: lane i of a wave-load
// fills the i-th 16-byte chunk of a 1 KiB LDS block, the rows' pad chunk and the rows past N are
// out-of-range lanes (zero fill), and one s_waitcnt vmcnt(0) + s_barrier per tile replaces the
// register staging, the LDS stores and the full __syncthreads().
template <int N>
AITAMD_DEVICE void attn_wait_vmcnt() {
  // s_waitcnt simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]; only vmcnt is waited for
  constexpr int imm = (N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8);
  __builtin_amdgcn_s_waitcnt(imm);
}
template <int N>
AITAMD_DEVICE void attn_wait_vmcnt_upto(int n) {
  // wave-uniform n: waits until at most min(n, N) vector-memory operations are outstanding
  if constexpr (N == 0) {
    attn_wait_vmcnt<0>();
  } else {
    if (n >= N)
      attn_wait_vmcnt<N>();
    else
      attn_wait_vmcnt_upto<N - 1>(n);
  }
}

template <class T, class Tile, bool VEC, bool DMA = false>
__global__ void __launch_bounds__(Tile::NT, Tile::NW == 4 ? 2 : 1) attention_kernel(const AttnParams p) {
  static_assert(!DMA || VEC, "the direct-to-LDS path needs 16-byte chunks");
  static_assert(DMA || Tile::NS == 2, "the register-staged loaders double-buffer");
  static_assert(DMA || Tile::NG == 1, "wave groups need the direct-to-LDS loader");
  constexpr int NS = Tile::NS, NW = Tile::NW, NG = Tile::NG, NWT = NW * NG;
  using Tr = ElemTraits<T>;
  using vec8 = typename Tr::vec8;
  using vec4 = typename Tr::vec4;
  constexpr int KS = Tile::KS, OT = Tile::OT, KP = Tile::KP, OP = Tile::OP;
  constexpr int BN = Tile::BN, KPI = Tile::K_PITCH, VPI = Tile::V_PITCH;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* const sK = reinterpret_cast<T*>(smem_raw);  // [NS][BN][K_PITCH]
  T* const sV = sK + NS * BN * KPI;              // [NS][BN][V_PITCH]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_all = tid >> 6;
  const int grp = __builtin_amdgcn_readfirstlane(wave_all / NW);  // which tiles this wave takes
  const int wave = wave_all % NW;                                 // which 32 query rows
  const int r32 = lane & 31;
  const int h = lane >> 5;
  // Workgroup -> (query tile, batch entry).  The hardware deals consecutive workgroup ids round-robin over the
  // 8 XCDs, each with its own L2; dealt plainly, the workgroups of one batch entry land on all of them and every
  // L2 fetches that entry's K and V.  When the grid divides evenly, XCD x takes the x-th eighth of the
  // (batch entry, query tile) pairs instead, so the workgroups that stream the same K / V share one L2.
  int bx = blockIdx.x, by = blockIdx.y;
  {
    const int total = gridDim.x * gridDim.y;
    if ((int)gridDim.y == p.B && (total & 7) == 0) {
      const int id = blockIdx.x + gridDim.x * blockIdx.y;
      const int v = (id & 7) * (total >> 3) + (id >> 3);
      by = v / (int)gridDim.x;
      bx = v - by * (int)gridDim.x;
    }
  }
  const int m0 = bx * Tile::BM;
  const int q_row = m0 + wave * 32 + r32;  // this lane's query row

  for (int b = by; b < p.B; b += gridDim.y) {
    const T* Qb = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.M * p.K;
    const T* Kb = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.N * p.K;
    const T* Vb = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.N * p.O;
    // keys of this batch entry (uniform over the workgroup)
    int N = p.N;
    if (p.kv_len != nullptr) {
      const int len = __builtin_amdgcn_readfirstlane(p.kv_len[b / p.G]);
      N = len < 0 ? 0 : (len < N ? len : N);
    }
    int m_rows = p.M;
    if (p.q_len != nullptr) {
      const int len = __builtin_amdgcn_readfirstlane(p.q_len[b / p.G]);
      m_rows = len < 0 ? 0 : (len < m_rows ? len : m_rows);
      if (m0 >= m_rows) N = 0;  // nothing but padding rows here: no keys, zeros out
    }

    // ---- Q fragments (B operand of S^T = K Q^T): lane (q = r32, k = 16 ks + 8 h + j)
    vec8 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int k0 = ks * 16 + h * 8;
      vec8 v = {};
      if (q_row < p.M) {
        if (VEC) {
          if (k0 < p.K) v = *reinterpret_cast<const vec8*>(Qb + (int64_t)q_row * p.K + k0);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (k0 + j < p.K) v[j] = Qb[(int64_t)q_row * p.K + k0 + j];
        }
      }
      // a negative scale changes sides: (-Q) K^T with |scale| gives the same scaled scores, and the
      // softmax below only ever sees a positive scale (negation is exact)
      if (p.scale_log2e < 0.0f) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = -v[j];
      }
      qf[ks] = v;
    }

    // ---- tile loaders: global -> registers -> LDS, zero-filled past N / K / O
    u32x4 kreg[Tile::K_IT], vreg[Tile::V_IT];
    auto gather = [&](const T* base, int row, int col, int rows, int cols) -> u32x4 {
      union {
        u32x4 v;
        T e[8];
      } u;
      u.v = u32x4{0, 0, 0, 0};
      if (row < rows) {
        if (VEC) {
          if (col < cols) u.v = *reinterpret_cast<const u32x4*>(base + (int64_t)row * cols + col);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (col + j < cols) u.e[j] = base[(int64_t)row * cols + col + j];
        }
      }
      return u.v;
    };
    auto load_tiles = [&](int n0) {
#pragma unroll
      for (int i = 0; i < Tile::K_IT; ++i) {
        const int c = tid + i * Tile::NT;
        const int row = c / (KP / 8), col = (c % (KP / 8)) * 8;
        kreg[i] = (c < Tile::K_CHUNKS) ? gather(Kb, n0 + row, col, N, p.K) : u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int i = 0; i < Tile::V_IT; ++i) {
        const int c = tid + i * Tile::NT;
        const int row = c / (OP / 8), col = (c % (OP / 8)) * 8;
        vreg[i] = (c < Tile::V_CHUNKS) ? gather(Vb, n0 + row, col, N, p.O) : u32x4{0, 0, 0, 0};
      }
    };
    auto store_tiles = [&](int stage) {
      T* dK = sK + stage * BN * KPI;
      T* dV = sV + stage * BN * VPI;
#pragma unroll
      for (int i = 0; i < Tile::K_IT; ++i) {
        const int c = tid + i * Tile::NT;
        const int row = c / (KP / 8), col = (c % (KP / 8)) * 8;
        if (c < Tile::K_CHUNKS) *reinterpret_cast<u32x4*>(dK + row * KPI + col) = kreg[i];
      }
#pragma unroll
      for (int i = 0; i < Tile::V_IT; ++i) {
        const int c = tid + i * Tile::NT;
        const int row = c / (OP / 8), col = (c % (OP / 8)) * 8;
        if (c < Tile::V_CHUNKS) *reinterpret_cast<u32x4*>(dV + row * VPI + (col ^ (Tile::v_swz(row) * 8))) = vreg[i];
      }
    };

    // ---- direct-to-LDS tile loader: the KL + VL wave-loads of a tile are dealt round-robin to the waves
    constexpr int KC1 = KP / 8 + 1, VC1 = OP / 8;            // chunks per LDS row (K: pad chunk included)
    constexpr int KL = BN * KC1 / 64, VL = BN * VC1 / 64;     // wave-loads per K / V tile
    constexpr int L_W = (KL + VL + NWT - 1) / NWT;
    static_assert((BN * KC1) % 64 == 0 && (BN * VC1) % 64 == 0, "tiles must be whole wave-loads");
    static_assert(Tile::K_PITCH == KC1 * 8 && Tile::V_PITCH == VC1 * 8, "LDS rows are whole chunks");
    typedef __attribute__((address_space(3))) void lds_void;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int wave_ld = __builtin_amdgcn_readfirstlane(wave_all);  // the loads are dealt over all waves
    uint32_t d_off[L_W];  // byte offset of the lane's chunk inside K (or V) for n0 = 0; kOobOffset = always zero
    if constexpr (DMA) {
#pragma unroll
      for (int i = 0; i < L_W; ++i) {
        const int j = wave_ld + NWT * i;
        const bool is_k = j < KL;
        const int idx = (is_k ? j : j - KL) * 64 + lane;
        const int c1 = is_k ? KC1 : VC1;
        const int dim = is_k ? p.K : p.O;
        const int row = idx / c1;
        // the lane fills chunk slot idx - row * c1 of the row; for V that slot holds chunk slot ^ v_swz(row)
        const int c = is_k ? idx - row * c1 : (idx - row * c1) ^ Tile::v_swz(row);
        d_off[i] = (c * 8 < dim) ? (uint32_t)((row * dim + c * 8) * 2) : kOobOffset;
      }
    }
    // (the K / V choice of a wave-load is wave-uniform: scalar selects, no branches)
    auto issue_tile = [&](int n0, int stage) {
      T* dK = sK + stage * BN * KPI;
      T* dV = sV + stage * BN * VPI;
#pragma unroll
      for (int i = 0; i < L_W; ++i) {
        const int j = wave_ld + NWT * i;
        if ((i + 1) * NWT > KL + VL && j >= KL + VL) continue;  // only the last round can run past the tile
        const bool is_k = j < KL;
        const uint32_t off =
            d_off[i] != kOobOffset ? d_off[i] + (uint32_t)(n0 * (is_k ? p.K : p.O) * 2) : kOobOffset;
        T* dst = is_k ? dK + j * 512 : dV + (j - KL) * 512;
        const __amdgpu_buffer_rsrc_t r = make_rsrc(is_k ? Kb : Vb, (uint32_t)((int64_t)N * (is_k ? p.K : p.O) * 2));
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)dst, 16, off, 0, 0, 0);
      }
    };

    // keys this workgroup has to visit (causal: nothing right of the last query row)
    int n_end = N;
    if (p.causal) {
      const int last = m0 + Tile::BM;
      n_end = last < n_end ? last : n_end;
    }
    const int n_tiles = (n_end + BN - 1) / BN;

    f32x16 oacc[OT];
#pragma unroll
    for (int ot = 0; ot < OT; ++ot)
#pragma unroll
      for (int e = 0; e < 16; ++e) oacc[ot][e] = 0.0f;
    // running maximum of the raw scores of this lane's row (of the negated scores when the scale is
    // negative: see the Q fragments)
    const float c = __builtin_fabsf(p.scale_log2e);
    float m_run = -INFINITY;
    float l_run = 0.0f;       // running sum over this lane's half of the keys
#if AITAMD_ATTN_FAST
    bool ref_ok = false;      // (wave-uniform) every row of the wave has a finite reference point
#endif

    // wave-loads this wave issues per tile
    const int my_loads = (KL + VL - wave_ld + NWT - 1) / NWT;
    if constexpr (DMA && NG > 1) {
      // every group's first tile; later tiles are issued one iteration ahead (see the loop)
#pragma unroll
      for (int g = 0; g < NG; ++g)
        if (g < n_tiles) issue_tile(g * BN, g);
    } else if constexpr (DMA) {
      // NS - 1 tiles in flight; tiles past the last one are all out of range (zero fill, no traffic),
      // issued all the same so that the number of loads per tile stays constant for the waits
      if (n_tiles > 0) {
#pragma unroll
        for (int s0 = 0; s0 < NS - 1; ++s0) issue_tile(s0 * BN, s0);
      }
    } else {
      if (n_tiles > 0) {
        load_tiles(0);
        store_tiles(0);
      }
      __syncthreads();
    }

    // source-lane address pattern of the LDS transpose read (see file header):
    // 16-lane block = one 4-key x 16-column patch; lane i of the block points at
    // key i/4, columns 4*(i%4)..+3 of the patch.
    const int tr_i = lane & 15;
    const int tr_row = tr_i >> 2;
    const int tr_col = ((lane >> 4) & 1) * 16 + (tr_i & 3) * 4;
    // every row a lane reads is its tr_row plus a multiple of 4: one swizzle value per lane
    const int tr_swz = Tile::v_swz(tr_row) * 8;

    // 32-key sub-blocks per softmax step: two for head dims up to 48, which halves the per-step work (exchange
    // across halves, rescale test, branches) per key: 3.7 % faster at head dim 40; at 64 the 16 extra
    // registers cost a resident workgroup and it measures equal, so one there
    constexpr int KB = AITAMD_ATTN_KB(KS, OT);
    static_assert(BN % (32 * KB) == 0, "a tile is whole blocks");
    int cur = 0;
    const int n_iters = (n_tiles + NG - 1) / NG;
    for (int it = 0; it < n_iters; ++it) {
      const int t = it * NG + grp;  // this wave's tile
      const bool has_next = (t + 1) < n_tiles;
      if constexpr (DMA && NG > 1) {
        // the tiles of this iteration were issued one iteration ago; past the barrier the stages of the
        // previous iteration are free and take the next iteration's tiles
        attn_wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          const int tn = (it + 1) * NG + g;
          if (tn < n_tiles) issue_tile(tn * BN, tn % NS);
        }
        cur = t % NS;
        if (t >= n_tiles) continue;  // the last iteration can be short of tiles
      } else if constexpr (DMA) {
        // this wave's part of tile t has landed once only the NS - 2 younger tiles are in flight; past
        // the barrier everybody's has, and nobody reads the stage of tile t - 1 any more, so tile
        // t + NS - 1 starts landing there
        attn_wait_vmcnt_upto<(NS - 2) * L_W>((NS - 2) * my_loads);
        __builtin_amdgcn_s_barrier();
        issue_tile((t + NS - 1) * BN, cur == 0 ? NS - 1 : cur - 1);
      } else {
        if (has_next) load_tiles((t + 1) * BN);
      }
      const T* cK = sK + cur * BN * KPI;
      const T* cV = sV + cur * BN * VPI;
      // The lane's LDS addresses of the tile, one per operand (and per 32-column block of V, whose swizzle sits
      // in the column bits), taken once per tile and made opaque: every fragment read of the tile is then that
      // register plus an immediate offset.  Left to itself the compiler re-adds stage base, lane offset and block
      // offset in front of every read (22 vector instructions per 64 keys).
      typedef __attribute__((address_space(3))) const T lds_T;
      lds_T* k_lane = (lds_T*)(cK + r32 * KPI + h * 8);
      asm volatile("" : "+v"(k_lane));
      lds_T* v_lane[OT];
#pragma unroll
      for (int ot = 0; ot < OT; ++ot) {
        v_lane[ot] = (lds_T*)(cV + (h * 4 + tr_row) * VPI + ((ot * 32) ^ tr_swz) + tr_col);
        asm volatile("" : "+v"(v_lane[ot]));
      }

#pragma unroll
      for (int blk = 0; blk < BN / (32 * KB); ++blk) {
        const int nb = t * BN + blk * 32 * KB;  // first key of this block of KB x 32 keys
        // ---- S^T sub-blocks: rows = keys, columns = this wave's 32 query rows
        // (issuing the next block's product ahead of this block's softmax was measured: no gain at
        // head dim 40 and a quarter slower at head dim 64, where the extra live accumulator costs more)
        f32x16 s[KB];
#if AITAMD_ATTN_BATCH_READS
        // all K fragments of the block first, then its MFMAs: the reads overlap each other and the first MFMAs
        // instead of each being waited for right behind its issue
        {
          vec8 kf[KB][KS];
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
              kf[kb][ks] = *reinterpret_cast<const vec8*>(cK + ((blk * KB + kb) * 32 + r32) * KPI + ks * 16 + h * 8);
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) s[kb][e] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) s[kb] = Tr::mfma32(kf[kb][ks], qf[ks], s[kb]);
          }
        }
#else
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
          for (int e = 0; e < 16; ++e) s[kb][e] = 0.0f;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            typedef __attribute__((address_space(3))) const vec8 lds_vec8;
            const vec8 kf = *(lds_vec8*)(k_lane + (blk * KB + kb) * 32 * KPI + ks * 16);
            s[kb] = Tr::mfma32(kf, qf[ks], s[kb]);
          }
        }
#endif
        // lane holds keys nb + 32 kb + 8 g + 4 h + r (element 4 g + r of sub-block kb) of query row q_row.
        // The running maximum is kept on the raw scores and the scale is folded into the exponent:
        // p = exp2(s * c - m * c) is one FMA and one v_exp per score (c > 0: a negative scale was moved into
        // the Q fragments).  Only blocks that reach past N or touch the causal diagonal pay for masking; the
        // test is wave-uniform, so it costs one scalar branch per block.
        const bool need_mask = (nb + 32 * KB > N) || (p.causal && nb + 32 * KB - 1 > m0 + wave_u * 32);
        float alpha = 1.0f;
        vec8 pf[2 * KB];  // P^T fragments of the block's 16-key steps
        auto softmax_block = [&](auto masked_tag, auto nan_tag) {
          constexpr bool MASKED = decltype(masked_tag)::value;
          constexpr bool NAN_RESET = decltype(nan_tag)::value;  // (implies MASKED)
          bool dead[KB][16];
          if constexpr (MASKED) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
              for (int e = 0; e < 16; ++e) {
                const int n = nb + kb * 32 + (e >> 2) * 8 + h * 4 + (e & 3);
                dead[kb][e] = (n >= N) || (p.causal && n > q_row) || (NAN_RESET && s[kb][e] != s[kb][e]);
              }
          }
          float text = -INFINITY;
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) text = fmaxf(text, (MASKED && dead[kb][e]) ? -INFINITY : s[kb][e]);
          text = max_across_halves(text);
          const float m_cand = fmaxf(m_run, text);
          // The reference point of the exponent moves only when the row maximum has grown by more than
          // kLazyLog2 binary orders since it was last taken: until then p = exp2(s c - m c) may exceed 1 (by at
          // most 2^kLazyLog2, harmless in fp32 sums and in the fp16 / bf16 probabilities) and the accumulators
          // need no rescaling.  With random scores some row of a wave sets a new maximum in most blocks, so
          // rescaling on every change costs 2 multiplies per score; this way it is rare.
          constexpr float kLazyLog2 = 8.0f;
          const float drift = (m_run - m_cand) * c;  // <= 0; -inf (or NaN for inf - inf) on the first live block
          const bool move = !(drift >= -kLazyLog2);
          const float m_new = move ? m_cand : m_run;
          const float m_safe = __builtin_isinf(m_new) ? 0.0f : m_new;  // every key so far masked
          alpha = !move ? 1.0f : (__builtin_isinf(m_run) ? 0.0f : __builtin_amdgcn_exp2f(drift));
          const float mc = -m_safe * c;
          // the probabilities are rounded to the element type at once (the second product takes them so) and the
          // row sum adds the rounded values, two per instruction
          l_run *= alpha;
#pragma unroll
          for (int st = 0; st < 2 * KB; ++st) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const int kb = st >> 1, e = (st & 1) * 8 + j;
              pf[st][j] = Tr::from_float(
                  (MASKED && dead[kb][e]) ? 0.0f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][e], c, mc)));
            }
            l_run = add_elements(pf[st], l_run);
          }
          m_run = m_new;
        };
        const float m_before = m_run, l_before = l_run;
#if AITAMD_ATTN_FAST
        // Fast form of an unmasked block: no row maximum at all.  The probabilities are taken against the reference
        // point the row already has, p = exp2((s - m) c); that is exact whatever m is, as long as no p leaves the
        // element type's range, and a p beyond it shows as an infinite (or NaN) row sum, for which the block is
        // redone below in the full form (maximum, moved reference point, rescaled accumulators).  After a row's
        // first block - always the full form: there is no reference point yet - that takes a score 16 binary orders
        // above everything the row has seen (fp16; never in practice for bf16), so nearly every block saves the
        // maximum's 16 three-way compares, the exchange across the wave's halves and the bookkeeping of the
        // reference point: 96 instead of 128 vector instructions per 64 keys.
        bool full = need_mask || !ref_ok;
        if (!full) {
          const float mc = -m_run * c;
#pragma unroll
          for (int st = 0; st < 2 * KB; ++st) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const int kb = st >> 1, e = (st & 1) * 8 + j;
              pf[st][j] = Tr::from_float(__builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][e], c, mc)));
            }
            l_run = add_elements(pf[st], l_run);
          }
          if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(l_run <= 3.0e38f)) != 0, 0)) {
            l_run = l_before;
            full = true;
          }
        }
        if (full) {
          if (need_mask)
            softmax_block(std::true_type{}, std::false_type{});
          else
            softmax_block(std::false_type{}, std::false_type{});
          ref_ok = __builtin_amdgcn_ballot_w64(__builtin_isinf(m_run)) == 0;
        }
#else
        if (need_mask)
          softmax_block(std::true_type{}, std::false_type{});
        else
          softmax_block(std::false_type{}, std::false_type{});
#endif
        // A NaN score (a NaN in Q or in a K row) counts as -inf, i.e. its key is left out, as in the reference, whose
        // kernel applies ScaleAndResetNaNToMinusInfinity to the scores
        // (python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:106, bmm_softmax_bmm.py:99).  The running
        // maximum ignores NaNs as it is (fmaxf), and a NaN probability shows in the lane's row sum: the block is redone
        // with those keys masked.  One compare and one scalar branch per block where there is none.  (mem_eff_attention
        // runs without the reset: the reference's kernel for it only scales.)
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(l_run != l_run) != 0, 0) && p.nan_reset) {
          m_run = m_before;
          l_run = l_before;
          softmax_block(std::true_type{}, std::true_type{});
#if AITAMD_ATTN_FAST
          ref_ok = __builtin_amdgcn_ballot_w64(__builtin_isinf(m_run)) == 0;
#endif
        }
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
          for (int ot = 0; ot < OT; ++ot)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[ot][e] *= alpha;
        }
        // ---- O^T += V^T P^T over the block's 16-key steps
#if AITAMD_ATTN_BATCH_READS
        {
          // all V^T fragments of the block first (the score registers are free by now), then the MFMAs
          vec8 vfs[2 * KB][OT];
#pragma unroll
          for (int st = 0; st < 2 * KB; ++st)
#pragma unroll
            for (int ot = 0; ot < OT; ++ot) {
              const T* vb = cV + (blk * KB * 32 + st * 16 + h * 4 + tr_row) * VPI + ((ot * 32) ^ tr_swz) + tr_col;
              const vec4 lo = AttnVec<T>::tr_read(vb);
              const vec4 hi = AttnVec<T>::tr_read(vb + 8 * VPI);
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                vfs[st][ot][j] = lo[j];
                vfs[st][ot][4 + j] = hi[j];
              }
            }
#pragma unroll
          for (int st = 0; st < 2 * KB; ++st)
#pragma unroll
            for (int ot = 0; ot < OT; ++ot) oacc[ot] = Tr::mfma32(vfs[st][ot], pf[st], oacc[ot]);
        }
#else
#pragma unroll
        for (int st = 0; st < 2 * KB; ++st) {
#pragma unroll
          for (int ot = 0; ot < OT; ++ot) {
            lds_T* vb = v_lane[ot] + (blk * KB * 32 + st * 16) * VPI;
            const vec4 lo = AttnVec<T>::tr_read(vb);
            const vec4 hi = AttnVec<T>::tr_read(vb + 8 * VPI);
            vec8 vf;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              vf[j] = lo[j];
              vf[4 + j] = hi[j];
            }
            oacc[ot] = Tr::mfma32(vf, pf[st], oacc[ot]);
          }
        }
#endif
      }

      if constexpr (!DMA) {
        if (has_next) store_tiles(cur ^ 1);
        __syncthreads();
      }
      if constexpr (NG == 1) cur = cur + 1 == NS ? 0 : cur + 1;
    }

    // ---- wave groups: the other groups hand their running state to group 0 through the ring's memory
    if constexpr (NG > 1) {
      attn_wait_vmcnt<0>();
      __syncthreads();  // nobody reads tiles any more and nothing is landing
      float* xch = reinterpret_cast<float*>(smem_raw);
      constexpr int NV = 16 * OT + 2;
      static_assert(NG == 2, "the merge below pairs two groups");
      if (grp == 1) {
#pragma unroll
        for (int ot = 0; ot < OT; ++ot)
#pragma unroll
          for (int e = 0; e < 16; ++e) xch[((ot * 16 + e) * NW + wave) * 64 + lane] = oacc[ot][e];
        xch[((NV - 2) * NW + wave) * 64 + lane] = m_run;
        xch[((NV - 1) * NW + wave) * 64 + lane] = l_run;
      }
      __syncthreads();
      if (grp == 0) {
        const float m1 = xch[((NV - 2) * NW + wave) * 64 + lane];
        const float l1 = xch[((NV - 1) * NW + wave) * 64 + lane];
        // both states are sums of exp2((s - m) c) terms for their own reference m: bring them to the larger one
        const float m = fmaxf(m_run, m1);
        const float a0 = __builtin_isinf(m_run) ? 0.0f : __builtin_amdgcn_exp2f((m_run - m) * c);
        const float a1 = __builtin_isinf(m1) ? 0.0f : __builtin_amdgcn_exp2f((m1 - m) * c);
        l_run = l_run * a0 + l1 * a1;
#pragma unroll
        for (int ot = 0; ot < OT; ++ot)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            oacc[ot][e] = oacc[ot][e] * a0 + xch[((ot * 16 + e) * NW + wave) * 64 + lane] * a1;
      }
    }

    // ---- normalise and store permuted: out[b / G][m][b % G][o]
    const float l_tot = sum_across_halves(l_run);
    const float inv = (l_tot > 0.0f && q_row < m_rows) ? 1.0f / l_tot : 0.0f;
    if (q_row < p.M && grp == 0) {
      T* orow = reinterpret_cast<T*>(p.out) + (((int64_t)(b / p.G) * p.M + q_row) * p.G + (b % p.G)) * p.O;
      const bool vec_ok = ((p.O & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 7) == 0);
#pragma unroll
      for (int ot = 0; ot < OT; ++ot)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int o = ot * 32 + g * 8 + h * 4;
          if (o >= p.O) continue;
          if (vec_ok) {
            vec4 ov;
#pragma unroll
            for (int j = 0; j < 4; ++j) ov[j] = Tr::from_float(oacc[ot][g * 4 + j] * inv);
            *reinterpret_cast<vec4*>(orow + o) = ov;
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (o + j < p.O) orow[o + j] = Tr::from_float(oacc[ot][g * 4 + j] * inv);
          }
        }
    }
    if constexpr (DMA) attn_wait_vmcnt<0>();  // the zero-fill tiles issued past the last one
    __syncthreads();  // LDS stage 0 is refilled by the next batch iteration
  }
}

}  // namespace aitamd
