// RCR GEMM main loop with direct global->LDS loads (buffer_load_dwordx4 ... lds)
// and an NS-deep LDS ring, plus an LDS-transposed epilogue with 128-bit stores.
//
// Differences from gemm_kernel.hpp (same math, same operand layout):
//  * A/B slabs never pass through VGPRs: each wave's load instruction fills one
//    contiguous 1 KiB of LDS (64 lanes x 16 bytes); the XOR swizzle is applied
//    on the *global* side by choosing which 16-byte chunk of the row each lane
//    fetches, so the ds_read side stays bank-conflict free.
//  * NS slabs are resident: the slab for step k+NS-1 is issued while step k is
//    multiplied, and one s_waitcnt vmcnt + one barrier per step orders them.
//  * MT selects the MFMA: 32 -> v_mfma_f32_32x32x16, 16 -> v_mfma_f32_16x16x32.
//  * the accumulator tile goes registers -> LDS (row-major, padded) -> registers
//    so that each lane owns 8 consecutive output columns: bias / residual loads
//    and the store are 16-byte accesses.
#pragma once

#include "common.hpp"
#include "epilogue.hpp"
#include "gemm_kernel.hpp"

namespace aitamd {

// SPLITK_ = 1: GemmParams::split_k workgroups share each tile, each multiplying a contiguous part of the K-slabs;
// every one of them leaves its fp32 partial tile in the scratch memory (GemmParams::ws) and counts itself on the
// tile's counter, and the one that finds all the others counted sums the partial tiles in slab order (its own
// included, so the result does not depend on who came last) and runs the epilogue.  Nobody waits for anybody.
// For grids that leave most CUs idle and tiles small enough that a partial tile is a few KiB.
//
// MODE 2, K in dwords (3: both): K, the row pitches and the operand pointers need to be whole dwords only (K % 8 in {2, 4, 6}:
// rows that start 4, 8 or 12 bytes off a 16-byte boundary).  The 16-byte slab loads take dword-aligned addresses
// as they are; the K loop runs over the whole 16-byte pieces of a row, and the 2, 4 or 6 elements behind them are
// fetched once per tile with dword loads straight into MFMA operands (lanes of the first k-chunk, zeros elsewhere)
// and multiplied after the loop.  Nothing is read past the end of a row.
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int NS_, int OCC_, int PIPE_ = 0, int MT_ = 32, int AUX_ = 0,
          int MODE_ = 0>
struct GemmTileDma {
  static constexpr int SPLITK = MODE_ & 1;          // MODE bit 0
  static constexpr int KTAIL = (MODE_ >> 1) & 1;    // MODE bit 1
  static constexpr int64_t kSlotBytes = (int64_t)BM_ * BN_ * 4;
  static constexpr int64_t kCounterAlign = 4096;
  // scratch bytes for `tiles` (batch x tile) pairs shared by `splits` workgroups each: one counter per pair,
  // padded to 4 KiB, then one slot per workgroup
  static constexpr int64_t ws_bytes(int64_t tiles, int splits) {
    return SPLITK ? (tiles * 4 + kCounterAlign - 1) / kCounterAlign * kCounterAlign + tiles * splits * kSlotBytes : 0;
  }
  // cache-policy bits of the slab loads: 1 = sc0, 2 = nt, 16 = sc1
  static constexpr int AUX = AUX_;
  // PIPE 0: barrier at the top of every K-slab.  PIPE 1: barrier inside the last
  // MFMA step of a slab, so the first fragments of the next slab are read from
  // LDS under the current slab's last MFMAs (needs NS >= 3).
  static constexpr int PIPE = PIPE_;
  static constexpr int MT = MT_;                     // MFMA output tile edge
  static constexpr int KSTEP = MT == 32 ? 16 : 32;   // K consumed by one MFMA
  static constexpr int QN = 64 / MT;                 // k-chunks (of 8) per MFMA operand = lane / MT range
  static constexpr int ACC_N = MT * MT / 64;         // fp32 accumulators per lane per MFMA tile
  static constexpr int BM = BM_, BN = BN_, BK = BK_;
  static constexpr int WGM = WGM_, WGN = WGN_, NS = NS_, OCC = OCC_;
  static constexpr int KVEC = KTAIL ? 2 : 8;
  static constexpr int NW = WGM * WGN;
  static constexpr int NT = NW * kWaveSize;
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;
  static constexpr int MI = WTM / MT, NI = WTN / MT;
  static constexpr int KK = BK / KSTEP;
  static constexpr int CPR = BK / 8;                 // 16-byte chunks per LDS row
  static constexpr int RPW = (256 / (BK * 2)) > 0 ? (256 / (BK * 2)) : 1;
  static constexpr int ROWS_PER_LOAD = 64 / CPR;     // rows one wave-load covers (1 KiB)
  static constexpr int A_LOADS = BM / ROWS_PER_LOAD; // wave-loads per slab
  static constexpr int B_LOADS = BN / ROWS_PER_LOAD;
  // the A_LOADS + B_LOADS wave-loads of a slab are dealt round-robin to the waves
  static constexpr int LOADS_PER_STEP = (A_LOADS + B_LOADS) / NW;  // per wave
  static constexpr int STAGE_ELEMS = (BM + BN) * BK;
  // epilogue staging: one MT-row strip per wave, fp32, padded by 4 floats per row
  static constexpr int EPI_PITCH = WTN + 4;
  static constexpr int EPI_BYTES = NW * MT * EPI_PITCH * 4;
  static constexpr int MAIN_BYTES = NS * STAGE_ELEMS * 2;
  static constexpr int kLdsBytes = MAIN_BYTES > EPI_BYTES ? MAIN_BYTES : EPI_BYTES;
  // operands that are not K-contiguous need whole k-rows per 1 KiB wave-load and at least 8 chunks per row
  static constexpr bool kTransposable = MT == 32 && (BM == 64 || BM == 128 || BM == 256) &&
      (BN == 64 || BN == 128 || BN == 256);
  static_assert(MT == 32 || MT == 16, "MFMA tile is 32x32 or 16x16");
  static_assert(WTM % MT == 0 && WTN % MT == 0, "wave tile must be whole MFMA tiles");
  static_assert(BM % ROWS_PER_LOAD == 0 && BN % ROWS_PER_LOAD == 0, "slab rows must fill whole wave-loads");
  static_assert((A_LOADS + B_LOADS) % NW == 0, "slab loads must divide over the waves");
  static_assert(BK % KSTEP == 0 && 64 % CPR == 0, "BK must be a multiple of the MFMA K");
  static_assert((NS - 2) * LOADS_PER_STEP <= 63, "vmcnt field is 6 bits");
  static_assert(PIPE == 0 || (NS >= 3 && (KK == 1 || KK % 2 == 0)), "cross-slab prefetch needs 3 stages");
  static_assert(WTN % 8 == 0, "epilogue needs 8-column groups");
};

template <class Tile>
AITAMD_DEVICE int dma_lds_chunk_elem(int row, int chunk) {
  const int swz = (row / Tile::RPW) % Tile::CPR;
  return row * Tile::BK + ((chunk ^ swz) << 3);
}

template <int N>
AITAMD_DEVICE void wait_vmcnt() {
  // s_waitcnt simm16 on gfx9: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]
  constexpr int imm = (N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8);
  __builtin_amdgcn_s_waitcnt(imm);
}

template <class T, int MT>
struct MfmaOp;
template <class T>
struct MfmaOp<T, 32> {
  using acc_t = f32x16;
  static AITAMD_DEVICE acc_t run(typename ElemTraits<T>::vec8 a, typename ElemTraits<T>::vec8 b, acc_t c) {
    return ElemTraits<T>::mfma32(a, b, c);
  }
};
template <class T>
struct MfmaOp<T, 16> {
  using acc_t = f32x4;
  static AITAMD_DEVICE acc_t run(typename ElemTraits<T>::vec8 a, typename ElemTraits<T>::vec8 b, acc_t c) {
    return ElemTraits<T>::mfma16(a, b, c);
  }
};

// Scheduling hints for one MFMA step of MFMAS matrix instructions that also
// issues READS LDS fragment reads (for the next step) and VM direct-to-LDS
// loads.  The reads go first, two behind each of the first MFMAs, so they have
// the rest of the step to arrive; the VM loads are spread evenly over the
// remaining MFMAs so that the waves of a CU never burst more than the L1 can
// take per clock.
template <int N>
AITAMD_DEVICE void sched_mfma() {
  if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(0x008, N, 0);
}
template <int VM, int LEFT, int PER>
AITAMD_DEVICE void sched_spread_vmem() {
  if constexpr (VM > 0) {
    constexpr int take = LEFT < PER ? LEFT : PER;
    sched_mfma<take>();
    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // 1 VMEM read
    sched_spread_vmem<VM - 1, LEFT - take, PER>();
  } else {
    sched_mfma<LEFT>();
  }
}
template <int PAIRS>
AITAMD_DEVICE void sched_front_reads() {
  if constexpr (PAIRS > 0) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // 2 DS reads
    sched_front_reads<PAIRS - 1>();
  }
}
template <int MFMAS, int READS, int VM>
AITAMD_DEVICE void sched_step() {
  constexpr int PAIRS = (READS + 1) / 2 < MFMAS ? (READS + 1) / 2 : MFMAS;
  sched_front_reads<PAIRS>();
  constexpr int REST = MFMAS - PAIRS;
  constexpr int PER = VM > 0 ? (REST / VM > 0 ? REST / VM : 1) : 1;
  sched_spread_vmem<VM, REST, PER>();
}

// LAYOUT selects how the operands lie in memory (the result is always row-major):
//   0 "rcr": A [M, K], B [N, K]  - both K-contiguous, the native form of the MFMA operands
//   1 "rrr": A [M, K], B [K, N]      2 "ccr": A [K, M], B [N, K]      3 "crr": A [K, M], B [K, N]
// An operand that is not K-contiguous is copied to LDS as it lies in memory (k-rows of BM or BN elements,
// 16-byte chunks XOR-swizzled by 2 * (k % 4) so that four consecutive k-rows fall into four different
// 32-byte bank groups) and its fragments are gathered with the transposing LDS read: per 16 lanes, lane
// 4 i + e receives element e of the four 8-byte rows i, i + 4, i + 8, i + 12 addressed by the 16 lanes, so
// when lane r points at (k-row r / 4, elements 4 (r % 4) .. + 4) lane d ends up with one element column d
// of four consecutive k-rows: two such reads give the 8 k-values of an MFMA operand.
template <class T, class Tile, class Epi, bool PERM = false, int LAYOUT = 0>
__global__ void __launch_bounds__(Tile::NT, Tile::OCC) gemm_rcr_dma_kernel(const GemmParams p) {
  using Tr = ElemTraits<T>;
  using vec8 = typename Tr::vec8;
  using vec4 = typename Tr::vec4;
  constexpr bool A_T = (LAYOUT & 2) != 0, B_T = (LAYOUT & 1) != 0;
  static_assert(LAYOUT == 0 || Tile::kTransposable, "this tile has no transposed-operand form");
  using Mfma = MfmaOp<T, Tile::MT>;
  using acc_t = typename Mfma::acc_t;
  constexpr int BM = Tile::BM, BN = Tile::BN, BK = Tile::BK, NS = Tile::NS;
  constexpr int MI = Tile::MI, NI = Tile::NI, MT = Tile::MT, QN = Tile::QN, ACC_N = Tile::ACC_N;
  constexpr int L_IT = Tile::LOADS_PER_STEP;
  constexpr int KK = Tile::KK;
  constexpr int AUX = Tile::AUX;
  typedef __attribute__((address_space(3))) void lds_void;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* const smem = reinterpret_cast<T*>(smem_raw);  // [NS][ A: BM*BK | B: BN*BK ]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Tile::WGN;
  const int wn = wave % Tile::WGN;
  const int fr = lane % MT;  // row of the MFMA operand / column of the transposed result
  const int fq = lane / MT;  // which 8-wide k chunk of the MFMA step this lane feeds

  // split-K: the workgroups of one split form one full grid of tiles (split s = workgroups [s * tiles, (s + 1) * tiles))
  const int grid_tiles = p.tiles_m * p.tiles_n * p.batch;
  const int split = Tile::SPLITK ? (int)blockIdx.x / grid_tiles : 0;
  const int tile_wg = Tile::SPLITK ? (int)blockIdx.x - split * grid_tiles : (int)blockIdx.x;
  int batch, tm, tn;
  map_tile<8>(tile_wg, p.tiles_m, p.tiles_n, p.batch, batch, tm, tn);
  const int m0 = tm * BM;
  const int n0 = tn * BN;
  const int rows_a = (p.M - m0) < BM ? (p.M - m0) : BM;
  const int rows_b = (p.N - n0) < BN ? (p.N - n0) : BN;

  // Per-lane source coordinates of the wave-loads: lane -> (row in the 1 KiB
  // block, physical chunk slot); the logical chunk fetched is slot ^ swz(row).
  const int l_row = lane / Tile::CPR;
  const int l_slot = lane % Tile::CPR;
  // wave-load j (j = wave + i * NW) fills 1 KiB block j of the slab; blocks
  // [0, A_LOADS) belong to A, the rest to B.  j is wave-uniform.
  uint32_t l_off[L_IT];
  int l_chunk_k[L_IT];      // k offset inside the slab of the lane's chunk (its k-row for a transposed operand)
  uint32_t l_kbytes[L_IT];  // bytes one step in k moves the lane's source address
#pragma unroll
  for (int i = 0; i < L_IT; ++i) {
    const int j = wave + i * Tile::NW;
    // (with A_LOADS a multiple of the wave count, whether load i fetches A or B is the same for every wave)
    const bool is_a = Tile::A_LOADS % Tile::NW == 0 ? i * Tile::NW < Tile::A_LOADS : j < Tile::A_LOADS;
    const int64_t ld = is_a ? p.lda : p.ldb;
    if ((is_a && A_T) || (!is_a && B_T)) {
      // 1 KiB of the operand's slab = 512 / BX whole k-rows of BX elements
      const int bx = is_a ? BM : BN;
      const int cpr = bx / 8;
      const int k_row = (is_a ? j : j - Tile::A_LOADS) * (512 / bx) + lane / cpr;
      const int chunk = (lane % cpr) ^ (2 * (k_row & 3));
      l_off[i] = (uint32_t)(((int64_t)k_row * ld + chunk * 8) * 2);
      l_chunk_k[i] = k_row;
      l_kbytes[i] = (uint32_t)(ld * 2);
    } else {
      const int row = (is_a ? j : j - Tile::A_LOADS) * Tile::ROWS_PER_LOAD + l_row;
      const int chunk = l_slot ^ ((row / Tile::RPW) % Tile::CPR);
      l_off[i] = (uint32_t)(((int64_t)row * ld + chunk * 8) * 2);
      l_chunk_k[i] = chunk * 8;
      l_kbytes[i] = 2;
    }
  }

  int a_rd[KK], b_rd[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    a_rd[kk] = dma_lds_chunk_elem<Tile>(wm * Tile::WTM + fr, kk * QN + fq);
    b_rd[kk] = BM * BK + dma_lds_chunk_elem<Tile>(wn * Tile::WTN + fr, kk * QN + fq);
  }
  // transposed operands: lane r of a 16-lane block addresses k-row (r / 4) and the 8-byte piece (r % 4) of
  // the block's 16 element columns; blocks 0 / 1 take the lower / upper 16 columns of a 32-wide MFMA
  // operand, blocks 2 / 3 the second 8 k-values (lane / 32, as for the K-contiguous operands)
  const int t_r = lane & 15;
  const int t_swz = 2 * ((t_r >> 2) & 3);
  const int t_piece = ((lane >> 4) & 1) * 2 + ((t_r & 3) >> 1);  // 16-byte chunk inside the 32 columns
  int at_col[A_T ? MI : 1], bt_col[B_T ? NI : 1];
  if constexpr (A_T) {
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
      at_col[mi] = (((wm * Tile::WTM / 8 + mi * 4 + t_piece) ^ t_swz) << 3) + (t_r & 1) * 4 +
          (fq * 8 + (t_r >> 2)) * BM;
  }
  if constexpr (B_T) {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
      bt_col[ni] = BM * BK + (((wn * Tile::WTN / 8 + ni * 4 + t_piece) ^ t_swz) << 3) + (t_r & 1) * 4 +
          (fq * 8 + (t_r >> 2)) * BN;
  }

  static_assert(!Tile::KTAIL || LAYOUT == 0, "the dword K tail is written for K-contiguous operands");
  // K covered by the slab loop: all of it, or its whole 16-byte pieces
  const int k_main = Tile::KTAIL ? (p.K & ~7) : p.K;
  const int k_tiles_all = (k_main + BK - 1) / BK;
  // this workgroup's K-slabs [k_lo, k_lo + k_tiles)
  const int splits = Tile::SPLITK ? p.split_k : 1;
  const int k_lo = Tile::SPLITK ? (int)((int64_t)split * k_tiles_all / splits) : 0;
  const int k_tiles = Tile::SPLITK ? (int)((int64_t)(split + 1) * k_tiles_all / splits) - k_lo : k_tiles_all;

  {
    // a transposed operand starts at its first column of the tile and ends with the tile's columns of row K-1
    const T* Ab = reinterpret_cast<const T*>(p.a) + (int64_t)batch * p.sa + (A_T ? (int64_t)m0 : (int64_t)m0 * p.lda);
    const T* Bb = reinterpret_cast<const T*>(p.b) + (int64_t)batch * p.sb + (B_T ? (int64_t)n0 : (int64_t)n0 * p.ldb);
    const int64_t bytes_a = A_T ? (((int64_t)p.K - 1) * p.lda + rows_a) * 2 : (((int64_t)rows_a - 1) * p.lda + p.K) * 2;
    const int64_t bytes_b = B_T ? (((int64_t)p.K - 1) * p.ldb + rows_b) * 2 : (((int64_t)rows_b - 1) * p.ldb + p.K) * 2;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ab, clamp_records(bytes_a));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bb, clamp_records(bytes_b));

    // Issue the wave-loads of K-slab `kt` into ring slot `stage`.  Slabs past
    // the end of K are still issued (every chunk out of range -> zero fill) so
    // the number of loads in flight per step stays constant for s_waitcnt.
    auto issue_loads = [&](int kt, int stage, int i0, int i1) {
      const int k0 = (Tile::SPLITK && kt >= k_tiles) ? k_main : (k_lo + kt) * BK;  // (past the own range: nothing to fetch)
      T* sbase = smem + stage * Tile::STAGE_ELEMS;
#pragma unroll
      for (int i = 0; i < L_IT; ++i) {
        if (i < i0 || i >= i1) continue;
        const int j = wave + i * Tile::NW;
        const uint32_t step = (A_T || B_T) ? (uint32_t)k0 * l_kbytes[i] : (uint32_t)(k0 * 2);
        const uint32_t off = (k0 + l_chunk_k[i] < k_main) ? l_off[i] + step : kOobOffset;
        T* dst = sbase + j * 512;  // 1 KiB = 512 elements per wave-load; A blocks then B blocks
        const bool is_a = Tile::A_LOADS % Tile::NW == 0 ? i * Tile::NW < Tile::A_LOADS : j < Tile::A_LOADS;
        if (is_a)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)dst, 16, off, 0, 0, AUX);
        else
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_void*)dst, 16, off, 0, 0, AUX);
      }
    };

    constexpr int kFragReads = MI * (A_T ? 2 : 1) + NI * (B_T ? 2 : 1);  // LDS reads per MFMA step
    acc_t acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) acc[mi][ni][e] = 0.0f;

    // dword K tail: the up to three dwords behind the last whole 16-byte piece of each of the lane's operand rows,
    // requested before the slab loads (so every wait of the loop covers them) and used after the loop
    uint32_t tail_a[Tile::KTAIL ? MI : 1][3], tail_b[Tile::KTAIL ? NI : 1][3];
    if constexpr (Tile::KTAIL != 0) {
#pragma unroll
      for (int d = 0; d < 3; ++d) {
        const int k = k_main + 2 * d;
        const bool on = fq == 0 && k < p.K;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
          const int row = wm * Tile::WTM + mi * MT + fr;
          tail_a[mi][d] = buffer_load_4B(ra, on ? (uint32_t)(((int64_t)row * p.lda + k) * 2) : kOobOffset);
        }
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
          const int row = wn * Tile::WTN + ni * MT + fr;
          tail_b[ni][d] = buffer_load_4B(rb, on ? (uint32_t)(((int64_t)row * p.ldb + k) * 2) : kOobOffset);
        }
      }
    }

    // the L_IT wave-loads of a slab are issued in KK equal portions, one per MFMA step
    constexpr int L_PER = (L_IT + KK - 1) / KK;
    constexpr int L_P0 = L_PER < L_IT ? L_PER : L_IT;  // size of portion 0
    if constexpr (Tile::PIPE == 0) {
#pragma unroll
      for (int s = 0; s < NS - 1; ++s) issue_loads(s, s, 0, L_IT);
    } else {
      // steady state at the top of slab 0: slabs 0..NS-3 whole, slab NS-2 up to portion 0
#pragma unroll
      for (int s = 0; s < NS - 2; ++s) issue_loads(s, s, 0, L_IT);
      issue_loads(NS - 2, NS - 2, 0, L_P0);
    }

    auto load_frags = [&](const T* st, int kk, vec8* af, vec8* bf) {
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
        if constexpr (A_T) {
          const T* at = st + at_col[mi] + kk * Tile::KSTEP * BM;
          af[mi] = join_halves<T>(tr_read16(at), tr_read16(at + 4 * BM));
        } else {
          af[mi] = *reinterpret_cast<const vec8*>(st + a_rd[kk] + mi * MT * BK);
        }
      }
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
        if constexpr (B_T) {
          const T* bt = st + bt_col[ni] + kk * Tile::KSTEP * BN;
          bf[ni] = join_halves<T>(tr_read16(bt), tr_read16(bt + 4 * BN));
        } else {
          bf[ni] = *reinterpret_cast<const vec8*>(st + b_rd[kk] + ni * MT * BK);
        }
      }
    };
    // operands swapped: the MFMA produces the transposed tile, so a lane holds
    // 4 consecutive output columns of one row
    auto mfmas = [&](const vec8* af, const vec8* bf) {
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = Mfma::run(bf[ni], af[mi], acc[mi][ni]);
    };
    // fragments are double-buffered in registers: step kk+1 is read from LDS
    // while step kk is multiplied
    vec8 af[2][MI], bf[2][NI];
    if constexpr (Tile::PIPE == 0) {
      for (int kt = 0; kt < k_tiles; ++kt) {
        // slab kt has landed once at most the (NS-2) younger slabs are in flight
        wait_vmcnt<(NS - 2) * Tile::LOADS_PER_STEP>();
        __builtin_amdgcn_s_barrier();
        const T* cur = smem + (kt % NS) * Tile::STAGE_ELEMS;
        load_frags(cur, 0, af[0], bf[0]);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const int cb = kk & 1, nb = cb ^ 1;
          const int i0 = kk * L_PER, i1 = (kk + 1) * L_PER < L_IT ? (kk + 1) * L_PER : L_IT;
          issue_loads(kt + NS - 1, (kt + NS - 1) % NS, i0, i1);
          if (kk + 1 < KK) load_frags(cur, kk + 1, af[nb], bf[nb]);
          mfmas(af[cb], bf[cb]);
          if (kk + 1 < KK)
            sched_step<MI * NI, kFragReads, L_PER>();
          else
            sched_step<MI * NI, 0, L_PER>();
        }
      }
    } else {
      wait_vmcnt<(NS - 3) * Tile::LOADS_PER_STEP + L_P0>();
      __builtin_amdgcn_s_barrier();
      load_frags(smem, 0, af[0], bf[0]);
      // with a single MFMA step per slab the register buffers alternate per slab
      constexpr int KT_UNROLL = (KK % 2 == 0) ? 1 : 2;
      for (int kt0 = 0; kt0 < k_tiles; kt0 += KT_UNROLL) {
#pragma unroll
        for (int u = 0; u < KT_UNROLL; ++u) {
          const int kt = kt0 + u;
          if (KT_UNROLL > 1 && kt >= k_tiles) break;
          const T* cur = smem + (kt % NS) * Tile::STAGE_ELEMS;
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) {
            const int cb = (u * KK + kk) & 1, nb = cb ^ 1;
            // portion `pi` of the slab being loaded during this period: the period
            // starts at the barrier in a slab's last step and covers the next KK-1 steps
            if (kk + 1 < KK) {
              const int pi = kk + 1;
              const int i0 = pi * L_PER, i1 = (pi + 1) * L_PER < L_IT ? (pi + 1) * L_PER : L_IT;
              issue_loads(kt + NS - 2, (kt + NS - 2) % NS, i0, i1);
              load_frags(cur, kk + 1, af[nb], bf[nb]);
              mfmas(af[cb], bf[cb]);
              sched_step<MI * NI, kFragReads, L_PER>();
            } else {
              // slab kt+1 has landed once at most (NS-3) younger slabs are in flight;
              // past the barrier nobody reads slab kt-1 any more, so its ring slot
              // starts taking slab kt+NS-1, and the next slab's first fragments are
              // fetched under this slab's last MFMAs.
              wait_vmcnt<(NS - 3) * Tile::LOADS_PER_STEP>();
              __builtin_amdgcn_s_barrier();
              const int i1 = L_P0;
              issue_loads(kt + NS - 1, (kt + NS - 1) % NS, 0, i1);
              load_frags(smem + ((kt + 1) % NS) * Tile::STAGE_ELEMS, 0, af[nb], bf[nb]);
              mfmas(af[cb], bf[cb]);
              sched_step<MI * NI, kFragReads, L_P0>();
            }
          }
        }
      }
    }
    // drain the zero-fill slabs still in flight before LDS is reused
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    if constexpr (Tile::KTAIL != 0) {
      // (of the workgroups that share a tile's K range the last one takes the tail)
      if (k_main < p.K && (Tile::SPLITK == 0 || split == splits - 1)) {
        vec8 ta[MI], tb[NI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
          ta[mi] = __builtin_bit_cast(vec8, u32x4{tail_a[mi][0], tail_a[mi][1], tail_a[mi][2], 0u});
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
          tb[ni] = __builtin_bit_cast(vec8, u32x4{tail_b[ni][0], tail_b[ni][1], tail_b[ni][2], 0u});
        mfmas(ta, tb);
      }
    }

    if constexpr (Tile::SPLITK != 0) {
      // ---------------- split-K: partial tile to the scratch memory; the last workgroup of the tile sums ----
      // ws: int32 counter per (batch, tile) pair, padded to 4 KiB, then slot (pair * splits + split) of BM * BN
      // floats.  A lane's 16-byte pieces lie as ((wave * PIECES + q) * 64 + lane) * 16 bytes: every wave-store and
      // wave-load is one contiguous KiB.  The slots may be read on another XCD than they were written on, whose L2
      // does not see this one's lines: they are written through to memory and read from there (sc1), and a store
      // is complete when vmcnt says so - no cache write-back or invalidate.
      if (splits > 1) {
        constexpr int PIECES = MI * NI * (ACC_N / 4);
        constexpr int kCoherent = 16;
        const int pair = batch * (p.tiles_m * p.tiles_n) + tm * p.tiles_n + tn;
        int* const counters = reinterpret_cast<int*>(p.ws);
        const int64_t counter_bytes = ((int64_t)grid_tiles * 4 + Tile::kCounterAlign - 1) / Tile::kCounterAlign * Tile::kCounterAlign;
        unsigned char* const slots = reinterpret_cast<unsigned char*>(p.ws) + counter_bytes;
        auto slot_rsrc = [&](int s_idx) {
          const uint64_t a = reinterpret_cast<uint64_t>(slots + ((int64_t)pair * splits + s_idx) * Tile::kSlotBytes);
          const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
          return make_rsrc(reinterpret_cast<void*>(((uint64_t)hi << 32) | lo), (uint32_t)Tile::kSlotBytes);
        };
        const uint32_t lane_off = (uint32_t)((wave * PIECES * 64 + lane) * 16);
        {
          const __amdgpu_buffer_rsrc_t rs = slot_rsrc(split);
#pragma unroll
          for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
              for (int q = 0; q < ACC_N / 4; ++q) {
                f32x4 v4;
#pragma unroll
                for (int j = 0; j < 4; ++j) v4[j] = acc[mi][ni][q * 4 + j];
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v4), rs, lane_off,
                                                       ((mi * NI + ni) * (ACC_N / 4) + q) * 1024, kCoherent);
              }
        }
        wait_vmcnt<0>();  // this lane's part of the partial tile is in memory
        __syncthreads();  // ... and so is every other lane's
        int* const word = reinterpret_cast<int*>(smem_raw);
        if (tid == 0) *word = __hip_atomic_fetch_add(&counters[pair], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __syncthreads();
        const bool last = *word == splits - 1;
        __syncthreads();
        if (!last) return;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int e = 0; e < ACC_N; ++e) acc[mi][ni][e] = 0.0f;
        for (int s_idx = 0; s_idx < splits; ++s_idx) {
          const __amdgpu_buffer_rsrc_t rs = slot_rsrc(s_idx);
#pragma unroll
          for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
              for (int q = 0; q < ACC_N / 4; ++q) {
                const f32x4 v4 = __builtin_bit_cast(
                    f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, lane_off, ((mi * NI + ni) * (ACC_N / 4) + q) * 1024, kCoherent));
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[mi][ni][q * 4 + j] += v4[j];
              }
        }
        // the counter is zero again for the next launch (which starts after this kernel has ended)
        if (tid == 0) __hip_atomic_store(&counters[pair], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __syncthreads();  // (the broadcast word shares LDS with the epilogue's strips)
      }
    }

    // ---------------- epilogue: acc -> LDS (fp32, per-wave strip) -> 16-byte stores --------
    T* Cb = reinterpret_cast<T*>(p.c) + out_batch_offset(p, batch);
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(Cb, kStoreRecords);
    const T* D0b = Epi::kNumD >= 1 ? reinterpret_cast<const T*>(p.d0) + (int64_t)batch * p.sd : nullptr;
    const T* D1b = Epi::kNumD >= 2 ? reinterpret_cast<const T*>(p.d1) + (int64_t)batch * p.sd : nullptr;
    const T* bias = reinterpret_cast<const T*>(p.bias);

    // vector form for the lanes whose 8 columns lie inside the row: multi-dword global and buffer accesses need
    // dword alignment only, so even pitches and 4-byte aligned pointers are enough
    bool vec_ok = ((p.ldc & 1) == 0) && ((p.sc & 1) == 0) && (!PERM || ((p.perm_n2 & 7) == 0 && (p.N & 7) == 0)) &&
        ((reinterpret_cast<uintptr_t>(p.c) & 3) == 0);
    if (Epi::kHasBias) vec_ok = vec_ok && ((reinterpret_cast<uintptr_t>(p.bias) & 3) == 0);
    if (Epi::kNumD >= 1)
      vec_ok = vec_ok && ((p.ldd & 1) == 0) && ((p.sd & 1) == 0) && ((reinterpret_cast<uintptr_t>(p.d0) & 3) == 0);
    if (Epi::kNumD >= 2) vec_ok = vec_ok && ((reinterpret_cast<uintptr_t>(p.d1) & 3) == 0);

    float one = 1.0f;
    asm volatile("" : "+s"(one));  // (opaque to the optimizer: see to_float_plus)
    constexpr int PITCH = Tile::EPI_PITCH;
    float* strip = reinterpret_cast<float*>(smem_raw) + wave * MT * PITCH;
    constexpr int LANES_PER_ROW = Tile::WTN / 8;             // lanes covering one strip row
    constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;        // rows read back per pass
    constexpr int ACTIVE = ROWS_PER_PASS * LANES_PER_ROW;    // lanes used in a pass
    constexpr int PASSES = (MT + ROWS_PER_PASS - 1) / ROWS_PER_PASS;
    const int rd_row = lane / LANES_PER_ROW;
    const int rd_col = (lane % LANES_PER_ROW) * 8;
    constexpr int NG = ACC_N / 4;  // groups of 4 consecutive columns per lane per MFMA tile

#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      // this wave's MT x WTN strip, row-major fp32
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          f32x4 v;
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = acc[mi][ni][g * 4 + j];
          *reinterpret_cast<f32x4*>(strip + fr * PITCH + ni * MT + g * (QN * 4) + fq * 4) = v;
        }
      // the strip is private to the wave: a wave-level LDS fence suffices
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) {
        const int row = ps * ROWS_PER_PASS + rd_row;
        const bool lane_on = (ACTIVE == 64 || lane < ACTIVE) && (MT % ROWS_PER_PASS == 0 || row < MT);
        const int m = m0 + wm * Tile::WTM + mi * MT + row;
        const int n = n0 + wn * Tile::WTN + rd_col;
        if (lane_on && m < p.M && n < p.N) {
          const f32x4 v0 = *reinterpret_cast<const f32x4*>(strip + row * PITCH + rd_col);
          const f32x4 v1 = *reinterpret_cast<const f32x4*>(strip + row * PITCH + rd_col + 4);
          float v[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
          const int64_t c_idx = out_index<PERM>(p, m, n);
          const int64_t d_idx = (int64_t)m * p.ldd + n;
          if (vec_ok && n + 8 <= p.N) {
            vec8 bv = {}, d0v = {}, d1v = {};
            if constexpr (Epi::kHasBias) bv = *reinterpret_cast<const vec8*>(bias + n);
            if constexpr (Epi::kNumD >= 1) d0v = *reinterpret_cast<const vec8*>(D0b + d_idx);
            if constexpr (Epi::kNumD >= 2) d1v = *reinterpret_cast<const vec8*>(D1b + d_idx);
            vec8 o;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              // bias conversion and add as one instruction where the type has one; -0.0 is the bias that adds nothing
              const float xb = Epi::kHasBias ? Tr::to_float_plus(bv[j], one, v[j]) : v[j];
              o[j] = Tr::from_float(apply_folded<Epi, T>(xb, d0v[j], d1v[j], one));
            }
            store_out(Cb, c_idx, o, p.nt_store != 0, rc);
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
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
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }
}

}  // namespace aitamd
