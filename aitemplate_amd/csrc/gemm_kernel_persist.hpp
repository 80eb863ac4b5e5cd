// Persistent variant of the direct-to-LDS RCR GEMM: one workgroup per CU walks its
// tiles and the LDS ring never drains.
//
// gemm_rcr_dma_kernel starts every tile cold: the first K-slab needs a full trip to
// memory (about 6 k cycles per 256x256 tile on MI355X) before the first MFMA
// can issue, which is a tenth of a BERT-FFN-sized tile (K = 768).  Here the slab
// stream runs across tile boundaries - while a tile's epilogue runs, the first
// slabs of the workgroup's next tile are already landing - so only the first
// tile of a workgroup pays the fill.
//
// Main loop: as gemm_rcr_dma_kernel with PIPE = 1 (barrier inside the last MFMA
// step of a slab, first fragments of the next slab prefetched across it, loads
// issued in two portions per slab).
//
// Epilogue: the accumulators are rounded to the output type, transposed through a
// wave-private LDS strip outside the ring (32 rows at a time, 16-byte chunks XOR-
// swizzled: the 16-byte reads are free of bank conflicts, the 8-byte writes take 1.3
// times the conflict-free time), read back as 8 consecutive columns per lane,
// combined with bias / residuals in fp32 and stored with 16-byte stores.  Rounding
// the accumulator before the element-wise functor is what the reference's
// Composable-Kernel path does too (C-shuffle to the C type, then the functor;
// python/aitemplate/utils/mk_ck_lib/gemm_operation.py:487).
#pragma once

#include <type_traits>

#include "gemm_kernel_dma.hpp"


namespace aitamd {

// MT_: edge of the MFMA's output block.  32: v_mfma_f32_32x32x16, two K-steps per 32-deep slab.  16:
// v_mfma_f32_16x16x32, one K-step per slab, whose blocks are multiplied in two halves (upper and lower block rows)
// around the slab's barrier; the 16x16x32 form moves half the accumulator registers per multiply-add and sustains
// 13 % more under the board's power limit on random operands (1.93 against 1.71 PFLOP/s in a loop of MFMAs alone).
// LBM_: rows of the A slab a ring stage holds.  A tile of BM rows whose 16-row blocks do not divide over the waves
// (224 rows: 14 blocks) takes the next size that does (256: rows past BM are cut off by the panel's buffer
// descriptor - zero fill, nothing fetched - and no wave reads them).
// PAIR_: the loader requests a K-slab and its successor together, 16 rows at a time (see the kernel): a row's two
// 64-byte pieces are the halves of one 128-byte line of memory, and asked for back to back by one wave the second
// finds the line in the CU's vector cache.  Needs a ring of five stages (two slabs can only be requested when two
// stages are free), which leaves no room beside it: the epilogue's strips take the stage that is free then.
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int NS_, int MT_ = 32, int LBM_ = BM_, int PAIR_ = 0>
struct GemmTilePersist {
  static constexpr int LBM = LBM_;
  static constexpr int PAIR = PAIR_;
  static constexpr int MT = MT_, KSTEP = MT == 32 ? 16 : 32, QN = 64 / MT, ACC_N = MT * MT / 64;
  static constexpr int BM = BM_, BN = BN_, BK = BK_;
  static constexpr int WGM = WGM_, WGN = WGN_, NS = NS_;
  static constexpr int NW = WGM * WGN;
  static constexpr int NT = NW * kWaveSize;
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;
  static constexpr int MI = WTM / MT, NI = WTN / MT;
  static constexpr int KK = BK / KSTEP;
  static constexpr int CPR = BK / 8;
  // Rows that share one value of the chunk swizzle.  The 32-row fragment reads of the 32x32 MFMAs are free of bank
  // conflicts with the rows of one 256-byte line of banks sharing it; the 16-row reads of the 16x16 MFMAs (four
  // chunks of each row at once) with half as many (measured with a loop of ds_read_b128 alone: 1.95x the time of
  // a conflict-free read with four rows per value, 1.00x with two).
  static constexpr int RPW32 = (256 / (BK * 2)) > 0 ? (256 / (BK * 2)) : 1;
  static constexpr int RPW = (MT == 16 && RPW32 > 1) ? RPW32 / 2 : RPW32;
  static constexpr int ROWS_PER_LOAD = 64 / CPR;
  static constexpr int A_LOADS = LBM / ROWS_PER_LOAD;
  static constexpr int B_LOADS = BN / ROWS_PER_LOAD;
  // Wave-loads per slab per wave.  L_MAIN consecutive blocks for every wave; where the blocks do not divide over the
  // waves (320 rows of A: 36 blocks on 8 waves) the last XTRA blocks of A go out as one more load of every wave,
  // block A_MAIN + wave % XTRA (fetched by NW / XTRA waves each: the same bytes to the same place).
  static constexpr int L_MAIN = (A_LOADS + B_LOADS) / NW;
  static constexpr int XTRA = (A_LOADS + B_LOADS) - L_MAIN * NW;
  static constexpr int A_MAIN = A_LOADS - XTRA;
  static constexpr int LOADS_PER_STEP = L_MAIN + (XTRA > 0 ? 1 : 0);
  static constexpr int L_P0 = (LOADS_PER_STEP + 1) / 2;            // issued in a slab's last step
  static constexpr int STAGE_ELEMS = (LBM + BN) * BK;
  static constexpr int RING_BYTES = NS * STAGE_ELEMS * 2;
  // wave-private epilogue strip: 32 rows x WTN elements of the output type
  static constexpr int STRIP_CHUNKS = WTN / 8;  // 16-byte chunks per strip row
  static constexpr int STRIP_PITCH = WTN * 2;
  // rows of an epilogue strip pass: 32 (one or two block rows) where the LDS has room for it beside the ring
  // (and where a wave's rows are whole 32-row passes)
  static constexpr bool kStripsFit32 =
      PAIR ? NW * 32 * STRIP_PITCH <= STAGE_ELEMS * 2 : RING_BYTES + NW * 32 * STRIP_PITCH <= 160 * 1024;
  static constexpr int SB = (kStripsFit32 && WTM % 32 == 0) ? 32 : 16;
  static constexpr int STRIP_BYTES = SB * STRIP_PITCH;
  static constexpr int ROWS_PER_PASS = 64 / STRIP_CHUNKS;
  static constexpr int PASSES = SB / ROWS_PER_PASS;
  static constexpr int kLdsBytes = PAIR ? RING_BYTES : RING_BYTES + NW * STRIP_BYTES;
  // a slab-pair form of this tile exists (five of its stages fit the LDS, its waves load four blocks each)
  static constexpr bool kPairable = PAIR == 0 && MT == 16 && NS == 4 && BK == 32 && XTRA == 0 && L_MAIN == 4 &&
      5 * STAGE_ELEMS * 2 <= 160 * 1024;
  // fewest K-slabs per tile for which the launcher takes the slab-pair form (it needs an even number; below 16
  // the longer fill and the peeled first pair cost what the loads gain: M=N=1000 K=256 0.0156 against 0.0150 ms)
  static constexpr int kPairMinSlabs = 16;
  static_assert(MT == 32 || MT == 16, "MFMA block is 32x32 or 16x16");
  static_assert((MT == 32 && KK == 2) || (MT == 16 && KK == 1 && MI >= 2), "a slab is multiplied in two halves");
  static_assert(LBM >= BM && LBM % ROWS_PER_LOAD == 0, "the A slab in LDS holds the tile's rows");
  static_assert(PAIR == 0 || (MT == 16 && NS == 5 && XTRA == 0 && L_MAIN == 4 && BK == 32 &&
                              NW * STRIP_BYTES <= STAGE_ELEMS * 2),
                "slab pairs: five stages of one-step slabs, four blocks per wave, the strips within one stage");
  static_assert(WTM % SB == 0, "a wave's rows are whole strip passes");
  static_assert(NS >= 4, "needs one slab in flight behind the one being waited for");
  static_assert(XTRA == 0 || (XTRA <= A_LOADS && NW % XTRA == 0 && L_P0 < LOADS_PER_STEP - 1),
                "left-over blocks: all of A, fetched as the last load of the slab's second portion");
  static_assert(SB % MT == 0, "a strip pass is whole block rows");
  static_assert(STRIP_CHUNKS == 4 || STRIP_CHUNKS == 8 || STRIP_CHUNKS == 16, "strip swizzle needs 2^k chunks");
  static_assert(kLdsBytes <= 160 * 1024, "LDS budget");
};

// SHORT_K: the instantiation for tiles of fewer K-slabs than ring stages (the launcher picks by K)
template <class T, class Tile, class Epi, bool PERM = false, bool SHORT_K = false>
__global__ void __launch_bounds__(Tile::NT, 1) gemm_rcr_persist_kernel(const GemmParams p) {
  using Tr = ElemTraits<T>;
  using vec8 = typename Tr::vec8;
  using Mfma = MfmaOp<T, Tile::MT>;
  using acc_t = typename Mfma::acc_t;
  constexpr int BM = Tile::BM, BN = Tile::BN, BK = Tile::BK, NS = Tile::NS;
  constexpr int MI = Tile::MI, NI = Tile::NI, MT = Tile::MT, KK = Tile::KK, QN = Tile::QN, SB = Tile::SB;
  // block rows multiplied in the first / second half of a slab (one-step slabs: the upper rows, then the lower
  // ones, one fewer where their number is odd; two-step slabs: all rows in both)
  constexpr int MH = KK == 1 ? (MI + 1) / 2 : MI;
  constexpr int MH2 = KK == 1 ? MI - MH : MI;
  constexpr int L = Tile::LOADS_PER_STEP, L_P0 = Tile::L_P0;
  constexpr int SC = Tile::STRIP_CHUNKS;
  typedef __attribute__((address_space(3))) void lds_void;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* const smem = reinterpret_cast<T*>(smem_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Tile::WGN;
  const int wn = wave % Tile::WGN;
  const int fr = lane % MT;
  const int fq = lane / MT;
  // (beside the ring; the slab-pair form moves it into the ring stage that is free during a tile's epilogue)
  unsigned char* strip = smem_raw + (Tile::PAIR ? 0 : Tile::RING_BYTES) + wave * Tile::STRIP_BYTES;

  const int tiles_per_batch = p.tiles_m * p.tiles_n;
  const int total_tiles = tiles_per_batch * p.batch;
  const int G = gridDim.x;
  const int g = blockIdx.x;
  const int k_tiles = (p.K + BK - 1) / BK;
  // Work items of this workgroup: one tile per full round, then its share of the last, partly
  // filled round.  When at most half the workgroups would get a tile there, every leftover tile is
  // split into an upper and a lower half (the waves of the other half idle through it): two
  // workgroups finish a leftover tile in about half a tile time instead of one working while
  // another waits.  Both halves of a tile go to workgroups of the same XCD.
  const int full_rounds = total_tiles / G;
  const int left = total_tiles - full_rounds * G;
  const bool split = Tile::WGM == 2 && left > 0 && 2 * left <= G && (G % 16) == 0;
  const int split_tile = ((g >> 4) << 3) + (g & 7);  // leftover tile of this workgroup when splitting
  const int split_half = (g >> 3) & 1;
  const int my_tiles = full_rounds + (split ? (split_tile < left ? 1 : 0) : (g < left ? 1 : 0));

  // (Every lambda below is force-inlined: left to its size heuristics the compiler has kept the slab lambda of a
  // four-wave instantiation as a real function, with the accumulators passed through scratch memory.)
  // ---- loader: a stream of slabs that runs across this workgroup's tiles ------------------------
  // A ring stage holds A_LOADS + B_LOADS blocks of 1 KiB (ROWS_PER_LOAD rows of a slab each, A then B); a wave
  // fetches the L consecutive blocks wave * L ... with one direct-to-LDS load each, so it reads only A or only B.
  // The loads of one portion ([0, L_P0) or [L_P0, L)) share one LDS base: the instruction's immediate offset
  // places the later ones (it shifts the global address as well, which the lane offsets take back).  Writing
  // the LDS base register before every load instead costs a fifth of the whole kernel's time.
  constexpr int LM = Tile::L_MAIN, XTRA = Tile::XTRA;
  static_assert(Tile::A_MAIN % LM == 0, "a wave's consecutive blocks must not straddle A and B");
  const bool loads_a = wave * LM < Tile::A_MAIN;
  // first LDS block of the wave's consecutive loads (A's blocks come first in a stage, its left-over ones last)
  const int l_block0 = wave * LM + (loads_a ? 0 : XTRA);
  const int l_block_x = Tile::A_MAIN + (XTRA > 0 ? wave % (XTRA > 0 ? XTRA : 1) : 0);
  const int l_row = lane / Tile::CPR;
  const int l_slot = lane % Tile::CPR;
  uint32_t l_off[L];
  int l_chunk_k[L];
#pragma unroll
  for (int i = 0; i < L; ++i) {
    const bool extra = XTRA > 0 && i == LM;  // the left-over block of A: always A, placed by its own LDS base
    const int j = wave * LM + i;
    const int row = (extra ? l_block_x : (loads_a ? j : j - Tile::A_MAIN)) * Tile::ROWS_PER_LOAD + l_row;
    const int chunk = l_slot ^ ((row / Tile::RPW) % Tile::CPR);
    const int in_portion = (SHORT_K || extra) ? 0 : (i < L_P0 ? i : i - L_P0);
    l_off[i] = (uint32_t)(((int64_t)row * ((loads_a || extra) ? p.lda : p.ldb) + chunk * 8) * 2 - in_portion * 1024);
    l_chunk_k[i] = chunk * 8;
  }

  struct TileCoord {
    int m0, n0, batch;
    int rows;  // rows of the tile this workgroup computes: BM, or BM / 2 for half a leftover tile
  };
  auto tile_coord = [&](int i) __attribute__((always_inline)) {
    TileCoord c;
    // virtual workgroup index: with one workgroup per CU, g % 8 is the XCD and stays it for every i
    int b, tm, tn;
    const bool half = split && i == full_rounds;
    const int vwg = half ? full_rounds * G + split_tile : g + i * G;
    if (p.xcd_cols > 0) {
      b = 0;
      map_tile_block(vwg, p.tiles_m, p.tiles_n, p.xcd_cols, tm, tn);
    } else {
      map_tile_grouped(vwg, p.tiles_m, p.tiles_n, p.batch, p.group_m > 0 ? p.group_m : 8, b, tm, tn);
    }
    c.m0 = tm * BM + (half ? split_half * (BM / 2) : 0);
    c.n0 = tn * BN;
    c.batch = b;
    c.rows = half ? BM / 2 : BM;
    return c;
  };

  // Descriptor of the operand panel (A or B) this wave fetches for the workgroup's i-th tile.  Past the last tile
  // the ring keeps turning on a zero-sized buffer: every lane is out of range, nothing is fetched, and the number
  // of loads in flight per step stays constant.
  // (dx: the A panel, for the left-over block every wave fetches; only tiles with such blocks use it)
  auto tile_desc = [&](int i, __amdgpu_buffer_rsrc_t& d, __amdgpu_buffer_rsrc_t& dx) __attribute__((always_inline)) {
    if (i < my_tiles) {
      const TileCoord c = tile_coord(i);
      const int rows_a = (p.M - c.m0) < c.rows ? (p.M - c.m0) : c.rows;
      const int rows_b = (p.N - c.n0) < BN ? (p.N - c.n0) : BN;
      const T* Ab = reinterpret_cast<const T*>(p.a) + (int64_t)c.batch * p.sa + (int64_t)c.m0 * p.lda;
      const T* Bb = reinterpret_cast<const T*>(p.b) + (int64_t)c.batch * p.sb + (int64_t)c.n0 * p.ldb;
      // (the lower half of a leftover tile can lie wholly below M: nothing to fetch then)
      const uint32_t bytes_a = rows_a > 0 ? clamp_records((((int64_t)rows_a - 1) * p.lda + p.K) * 2) : 0u;
      const uint32_t bytes_b = clamp_records((((int64_t)rows_b - 1) * p.ldb + p.K) * 2);
      d = make_rsrc(loads_a ? Ab : Bb, loads_a ? bytes_a : bytes_b);
      if constexpr (XTRA > 0) dx = make_rsrc(Ab, bytes_a);
    } else {
      d = make_rsrc(p.a, 0);
      if constexpr (XTRA > 0) dx = d;
    }
  };

  // Issue wave-loads [I0, I1) of K-slab `kt` of the tile behind `d` into ring stage `stage`.  No state, no
  // branches: the slab loop calls it between MFMAs and has to stay one basic block for the interleave to hold.
  auto issue_part = [&](auto i0_c, auto i1_c, const __amdgpu_buffer_rsrc_t& d, const __amdgpu_buffer_rsrc_t& dx, int kt,
                        int stage) __attribute__((always_inline)) {
    constexpr int I0 = decltype(i0_c)::value, I1 = decltype(i1_c)::value;
    const int k0 = kt * BK;
    T* dst = smem + stage * Tile::STAGE_ELEMS + (l_block0 + I0) * 512;  // 1 KiB per wave-load
    static_for<I0, I1>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      const uint32_t off = (k0 + l_chunk_k[i] < p.K) ? l_off[i] + (uint32_t)(k0 * 2) : kOobOffset;
      if constexpr (XTRA > 0 && i == LM)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(dx, (lds_void*)(smem + stage * Tile::STAGE_ELEMS + l_block_x * 512), 16,
                                                 off, 0, 0, 0);
      else if constexpr (SHORT_K)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(d, (lds_void*)(dst + (i - I0) * 512), 16, off, 0, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(d, (lds_void*)dst, 16, off, 0, (i - I0) * 1024, 0);
    });
  };

  // ---- fragments ------------------------------------------------------------------------------
  int a_rd[KK], b_rd[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    a_rd[kk] = dma_lds_chunk_elem<Tile>(wm * Tile::WTM + fr, kk * QN + fq);
    b_rd[kk] = Tile::LBM * BK + dma_lds_chunk_elem<Tile>(wn * Tile::WTN + fr, kk * QN + fq);
  }
  // KK == 2: half `hh` of a slab is K-step hh over all block rows (af[hh][0 .. MI), bf[hh][0 .. NI)).
  // KK == 1: half `hh` is block rows hh * MH ... of the one K-step (af[hh][0 .. MH)); both halves use bf[0].
  auto load_a = [&](const T* st, int hh, vec8* af) __attribute__((always_inline)) {
#pragma unroll
    for (int mi = 0; mi < MH; ++mi)
      if (mi < (hh == 0 ? MH : MH2))
        af[mi] = *reinterpret_cast<const vec8*>(st + a_rd[KK == 1 ? 0 : hh] + ((KK == 1 ? hh * MH : 0) + mi) * MT * BK);
  };
  auto load_b1 = [&](const T* st, int hh, int ni) __attribute__((always_inline)) {
    return *reinterpret_cast<const vec8*>(st + b_rd[KK == 1 ? 0 : hh] + ni * MT * BK);
  };
  auto load_frags = [&](const T* st, int hh, vec8* af, vec8* bf) __attribute__((always_inline)) {
    load_a(st, hh, af);
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) bf[ni] = load_b1(st, hh, ni);
  };
  acc_t acc[MI][NI];
  vec8 af[2][MH], bf[KK][NI];
  // operands swapped: the MFMA produces the transposed block, so a lane holds 4 consecutive
  // output columns of one row
  // (m0: first block row of the half: 0, or MH for the lower half of a one-step slab)
  auto mfmas = [&](const vec8* a, const vec8* b, int m0 = 0) __attribute__((always_inline)) {
#pragma unroll
    for (int mi = 0; mi < MH; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) acc[m0 + mi][ni] = Mfma::run(b[ni], a[mi], acc[m0 + mi][ni]);
  };
  auto mfmas_first = [&](const vec8* a, const vec8* b, int m0 = 0) __attribute__((always_inline)) {
    const acc_t zero = {};
#pragma unroll
    for (int mi = 0; mi < MH; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) acc[m0 + mi][ni] = Mfma::run(b[ni], a[mi], zero);
  };

  // The two halves of a slab.  The first fetches what the second needs and multiplies K-step 0 (the upper block
  // rows of a one-step slab); the second multiplies the rest and fetches the first half of the next slab.  With
  // one K-step per slab the B fragments serve both halves and are single-buffered: each is replaced by the next
  // slab's as soon as the MFMAs of its block column have been issued.
  auto half1_reads = [&](const T* cur_st) __attribute__((always_inline)) {
    if constexpr (KK == 2)
      load_frags(cur_st, 1, af[1], bf[1]);
    else
      load_a(cur_st, 1, af[1]);
  };
  auto half1_mfmas = [&](auto first_c) __attribute__((always_inline)) {
    if constexpr (decltype(first_c)::value)
      mfmas_first(af[0], bf[0]);
    else
      mfmas(af[0], bf[0]);
  };
  auto half2_reads = [&](const T* nxt_st) __attribute__((always_inline)) {
    if constexpr (KK == 2)
      load_frags(nxt_st, 0, af[0], bf[0]);
    else
      load_a(nxt_st, 0, af[0]);
  };
  // (FETCH = false: the next slab's fragments are not fetched - a tile's last slab, where they would have to live
  // through the epilogue; see kRefetch)
  auto half2_mfmas = [&](auto first_c, const T* nxt_st, auto fetch_c) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(first_c)::value;
    constexpr bool FETCH = decltype(fetch_c)::value;
    if constexpr (KK == 2) {
      mfmas(af[1], bf[1]);
    } else {
      const acc_t zero = {};
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
        for (int mi = 0; mi < MH2; ++mi)
          acc[MH + mi][ni] = Mfma::run(bf[0][ni], af[1][mi], FIRST ? zero : acc[MH + mi][ni]);
        if constexpr (FETCH) bf[0][ni] = load_b1(nxt_st, 0, ni);
      }
    }
  };

  // ---- epilogue -------------------------------------------------------------------------------
  const T* bias = reinterpret_cast<const T*>(p.bias);
  // vector form for the lanes whose 8 columns lie inside the row: multi-dword global and buffer accesses need
  // dword alignment only, so even pitches and 4-byte aligned pointers are enough
  bool vec_ok = ((p.ldc & 1) == 0) && ((p.sc & 1) == 0) && (!PERM || ((p.perm_n2 & 7) == 0 && (p.N & 7) == 0)) &&
      ((reinterpret_cast<uintptr_t>(p.c) & 3) == 0);
  if (Epi::kHasBias) vec_ok = vec_ok && ((reinterpret_cast<uintptr_t>(p.bias) & 3) == 0);
  if (Epi::kNumD >= 1)
    vec_ok = vec_ok && ((p.ldd & 1) == 0) && ((p.sd & 1) == 0) && ((reinterpret_cast<uintptr_t>(p.d0) & 3) == 0);
  if (Epi::kNumD >= 2) vec_ok = vec_ok && ((reinterpret_cast<uintptr_t>(p.d1) & 3) == 0);
  // strip addressing: row r, 16-byte chunk c lives at r * PITCH + ((c ^ (r % SC)) << 4)
  const int r_row = lane / SC;
  const int r_c = lane % SC;
  // Strip block `sb` (SB = 32 rows of the wave's part: one block row of 32x32 MFMAs, two of 16x16) goes to the
  // strip in the output type.  A lane holds, per MFMA block and group g, 4 consecutive columns
  // ni * MT + g * 4 QN + 4 fq of row fr.
  auto write_strip = [&](int sb) __attribute__((always_inline)) {
    constexpr int SUB = SB / MT;       // block rows per strip block
    constexpr int NG = Tile::ACC_N / 4;
#pragma unroll
    for (int sub = 0; sub < SUB; ++sub) {
      const int row = sub * MT + fr;
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int gq = 0; gq < NG; ++gq) {
          typename Tr::vec4 h;
#pragma unroll
          for (int j = 0; j < 4; ++j) h[j] = Tr::from_float(acc[sb * SUB + sub][ni][gq * 4 + j]);
          const int col = ni * MT + gq * (QN * 4) + fq * 4;
          *reinterpret_cast<u32x2*>(strip + row * Tile::STRIP_PITCH + (((col >> 3) ^ (row & (SC - 1))) << 4) +
                                    (col & 7) * 2) = __builtin_bit_cast(u32x2, h);
        }
    }
  };

  // Fast form of the epilogue's addressing (plain store, N a multiple of 8, a tile's rows span less than
  // 2 GiB): the output and the residuals are addressed through buffer descriptors that start at the wave's
  // corner of the tile, with 32-bit byte offsets that advance by a scalar per 8-row pass - no 64-bit index
  // arithmetic per pass, rows past M cut off by the descriptor's size, columns past N by an out-of-range offset.
  const bool fast_addr = !PERM && vec_ok && (p.N & 7) == 0 && (int64_t)BM * p.ldc * 2 < 0x7fffffffll &&
      (Epi::kNumD == 0 || (int64_t)BM * p.ldd * 2 < 0x7fffffffll);
  const uint32_t lane_off_c = (uint32_t)((r_row * (int)p.ldc + r_c * 8) * 2);
  const uint32_t lane_off_d = (uint32_t)((r_row * (int)p.ldd + r_c * 8) * 2);

  // NT: cache-policy bits of the stores, a template value so that the choice is made once per tile and the
  // passes of a strip stay one basic block (math of one pass schedules around the stores of the one before)
  auto epilogue_fast = [&](const TileCoord& c, auto nt_bits) __attribute__((always_inline)) {
    constexpr int NT_BITS = decltype(nt_bits)::value;
    const int m_w = c.m0 + wm * Tile::WTM;  // first row and column of the wave's part of the tile
    const int n_w = c.n0 + wn * Tile::WTN;
    const int rows_left = p.M - m_w;
    const uint32_t rows_valid = rows_left <= 0 ? 0u : (uint32_t)(rows_left < Tile::WTM ? rows_left : Tile::WTM);
    T* Cw = reinterpret_cast<T*>(p.c) + out_batch_offset(p, c.batch) + (int64_t)m_w * p.ldc + n_w;
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(Cw, rows_valid * (uint32_t)p.ldc * 2u);
    __amdgpu_buffer_rsrc_t rd0 = rc, rd1 = rc;
    if constexpr (Epi::kNumD >= 1) {
      const T* Dw = reinterpret_cast<const T*>(p.d0) + (int64_t)c.batch * p.sd + (int64_t)m_w * p.ldd + n_w;
      rd0 = make_rsrc(Dw, rows_valid * (uint32_t)p.ldd * 2u);
    }
    if constexpr (Epi::kNumD >= 2) {
      const T* Dw = reinterpret_cast<const T*>(p.d1) + (int64_t)c.batch * p.sd + (int64_t)m_w * p.ldd + n_w;
      rd1 = make_rsrc(Dw, rows_valid * (uint32_t)p.ldd * 2u);
    }
    const int n = n_w + r_c * 8;  // the lane's 8 columns: the same in every pass
    const bool col_ok = n < p.N;
    const uint32_t off_c0 = col_ok ? lane_off_c : kOobOffset;
    const uint32_t off_d0 = col_ok ? lane_off_d : kOobOffset;
    float one = 1.0f;
    asm volatile("" : "+s"(one));  // (opaque to the optimizer: see to_float_plus)
    float bf8[8] = {};
    if constexpr (Epi::kHasBias) {
      if (col_ok) {
        const vec8 bv = *reinterpret_cast<const vec8*>(bias + n);
#pragma unroll
        for (int j = 0; j < 8; ++j) bf8[j] = Tr::to_float(bv[j]);
      }
    }
#pragma unroll
    for (int sb = 0; sb < Tile::WTM / SB; ++sb) {
      write_strip(sb);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      // passes in flight at once: all of a strip's, or half of them with two residual operands (three 16-byte
      // values per pass and lane: all four passes of a 32-row strip at once spilled registers)
      constexpr int PG = (Epi::kNumD >= 2 && Tile::PASSES >= 4) ? Tile::PASSES / 2 : Tile::PASSES;
#pragma unroll
      for (int p0 = 0; p0 < Tile::PASSES; p0 += PG) {
        vec8 raw[PG], d0v[PG], d1v[PG];
#pragma unroll
        for (int q = 0; q < PG; ++q) {
          const int ps = p0 + q;
          const int row = ps * Tile::ROWS_PER_PASS + r_row;
          raw[q] = *reinterpret_cast<const vec8*>(strip + row * Tile::STRIP_PITCH + ((r_c ^ (row & (SC - 1))) << 4));
          const uint32_t step_d = (uint32_t)((sb * SB + ps * Tile::ROWS_PER_PASS) * (int)p.ldd * 2);
          if constexpr (Epi::kNumD >= 1) d0v[q] = __builtin_bit_cast(vec8, buffer_load_16B(rd0, off_d0 + step_d));
          if constexpr (Epi::kNumD >= 2) d1v[q] = __builtin_bit_cast(vec8, buffer_load_16B(rd1, off_d0 + step_d));
        }
#pragma unroll
        for (int q = 0; q < PG; ++q) {
          const int ps = p0 + q;
          vec8 o;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            // conversion and bias add as one instruction where the type has one; -0.0 is the bias that adds nothing
            const float xb = Epi::kHasBias ? Tr::to_float_plus(raw[q][j], one, bf8[j]) : Tr::to_float(raw[q][j]);
            o[j] = Tr::from_float(apply_folded<Epi, T>(xb, d0v[q][j], d1v[q][j], one));
          }
          const uint32_t off = off_c0 + (uint32_t)((sb * SB + ps * Tile::ROWS_PER_PASS) * (int)p.ldc * 2);
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o), rc, off, 0, NT_BITS);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  };

  auto epilogue = [&](const TileCoord& c) __attribute__((always_inline)) {
    if (fast_addr) {
      if (p.nt_store)
        epilogue_fast(c, std::integral_constant<int, 2>{});
      else
        epilogue_fast(c, std::integral_constant<int, 0>{});
      return;
    }
    T* Cb = reinterpret_cast<T*>(p.c) + out_batch_offset(p, c.batch);
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(Cb, kStoreRecords);
    const T* D0b = Epi::kNumD >= 1 ? reinterpret_cast<const T*>(p.d0) + (int64_t)c.batch * p.sd : nullptr;
    const T* D1b = Epi::kNumD >= 2 ? reinterpret_cast<const T*>(p.d1) + (int64_t)c.batch * p.sd : nullptr;
    const int n = c.n0 + wn * Tile::WTN + r_c * 8;  // the lane's 8 columns: the same in every pass
    float bf8[8] = {};  // the lane's 8 bias values, converted once per tile
    if constexpr (Epi::kHasBias) {
      if (vec_ok && n + 8 <= p.N) {
        const vec8 bv = *reinterpret_cast<const vec8*>(bias + n);
#pragma unroll
        for (int j = 0; j < 8; ++j) bf8[j] = Tr::to_float(bv[j]);
      }
    }
#pragma unroll
    for (int sb = 0; sb < Tile::WTM / SB; ++sb) {
      write_strip(sb);
      // the strip is private to the wave and LDS executes one wave's accesses in order
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int ps = 0; ps < Tile::PASSES; ++ps) {
        const int row = ps * Tile::ROWS_PER_PASS + r_row;
        const vec8 raw =
            *reinterpret_cast<const vec8*>(strip + row * Tile::STRIP_PITCH + ((r_c ^ (row & (SC - 1))) << 4));
        const int m = c.m0 + wm * Tile::WTM + sb * SB + row;
        if (m < p.M && n < p.N) {
          const int64_t c_idx = out_index<PERM>(p, m, n);
          const int64_t d_idx = (int64_t)m * p.ldd + n;
          if (vec_ok && n + 8 <= p.N) {
            vec8 d0v = {}, d1v = {};
            if constexpr (Epi::kNumD >= 1) d0v = *reinterpret_cast<const vec8*>(D0b + d_idx);
            if constexpr (Epi::kNumD >= 2) d1v = *reinterpret_cast<const vec8*>(D1b + d_idx);
            vec8 o;
#pragma unroll
            for (int j = 0; j < 8; ++j)
              o[j] = Tr::from_float(Epi::apply(Tr::to_float(raw[j]), bf8[j], Tr::to_float(d0v[j]), Tr::to_float(d1v[j])));
            store_out(Cb, c_idx, o, p.nt_store != 0, rc);
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              if (n + j < p.N) {
                float bj = 0.f, d0j = 0.f, d1j = 0.f;
                if constexpr (Epi::kHasBias) bj = Tr::to_float(bias[n + j]);
                if constexpr (Epi::kNumD >= 1) d0j = Tr::to_float(D0b[d_idx + j]);
                if constexpr (Epi::kNumD >= 2) d1j = Tr::to_float(D1b[d_idx + j]);
                Cb[out_index<PERM>(p, m, n + j)] = Tr::from_float(Epi::apply(Tr::to_float(raw[j]), bj, d0j, d1j));
              }
            }
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  };

  // The loader runs ahead of the multiplying: while slab kt of a tile is multiplied, the rest of slab kt + NS - 2
  // goes out in the slab's first step and the first portion of slab kt + NS - 1 in its last step, into the ring
  // stage the barrier has just freed.  From slab k_tiles - (NS - 1) on those are slabs of the workgroup's next tile.
  // Which tile a step loads from is decided by the structure of the code (one slab loop for the bulk of a tile,
  // NS - 1 peeled slabs for its end), never by a test inside a slab: a conditional there splits the slab into
  // basic blocks, the loads bunch up behind the barrier instead of alternating with the MFMAs, and the matrix unit
  // waits for the address unit (measured: 44 us of a 139 us launch).  Needs k_tiles >= NS.
  constexpr int D1 = NS - 2, D2 = NS - 1;
  constexpr std::integral_constant<int, 0> c_0{};
  constexpr std::integral_constant<int, L_P0> c_P{};
  constexpr std::integral_constant<int, L> c_L{};
  static_assert(L_P0 > 0 && L_P0 < L, "a slab goes out in two portions");
  __amdgpu_buffer_rsrc_t rd, nrd;    // this wave's operand panel of the current and of the next tile
  __amdgpu_buffer_rsrc_t rdx, nrdx;  // and their A panels, for tiles with left-over blocks
  tile_desc(0, rd, rdx);
  if constexpr (SHORT_K) {
    // Short K: the loader is more than a tile ahead and wraps at places that depend on k_tiles, so it keeps its
    // position as state and tests for the wrap after every slab it has issued (the conditional costs the
    // interleave; with so few slabs per tile the epilogue dominates anyway).
    int ld_i = 0, ld_kt = 0;
    auto advance = [&]() __attribute__((always_inline)) {
      if (++ld_kt == k_tiles) {
        ld_kt = 0;
        ++ld_i;
        tile_desc(ld_i, rd, rdx);
      }
    };
#pragma unroll
    for (int s = 0; s < NS - 2; ++s) {
      issue_part(c_0, c_P, rd, rdx, ld_kt, s);
      issue_part(c_P, c_L, rd, rdx, ld_kt, s);
      advance();
    }
    issue_part(c_0, c_P, rd, rdx, ld_kt, NS - 2);
    wait_vmcnt<(NS - 3) * L + L_P0>();
    __builtin_amdgcn_s_barrier();
    int rd_stage = 0;
    load_frags(smem, 0, af[0], bf[0]);
    for (int i = 0; i < my_tiles; ++i) {
      const TileCoord cur = tile_coord(i);
      const bool active = wm * Tile::WTM < cur.rows;
      for (int kt = 0; kt < k_tiles; ++kt) {
        const T* cur_st = smem + rd_stage * Tile::STAGE_ELEMS;
        const int nx_stage = rd_stage + 1 == NS ? 0 : rd_stage + 1;
        const T* nxt_st = smem + nx_stage * Tile::STAGE_ELEMS;
        const int st1 = rd_stage + D1 >= NS ? rd_stage + D1 - NS : rd_stage + D1;
        const int st2 = rd_stage + D2 >= NS ? rd_stage + D2 - NS : rd_stage + D2;
        issue_part(c_P, c_L, rd, rdx, ld_kt, st1);
        advance();
        if (active) {
          half1_reads(cur_st);
          if (kt == 0)
            half1_mfmas(std::true_type{});
          else
            half1_mfmas(std::false_type{});
        }
        wait_vmcnt<(NS - 3) * L>();
        __builtin_amdgcn_s_barrier();
        issue_part(c_0, c_P, rd, rdx, ld_kt, st2);
        if (active) {
          half2_reads(nxt_st);
          if (kt == 0)
            half2_mfmas(std::true_type{}, nxt_st, std::true_type{});
          else
            half2_mfmas(std::false_type{}, nxt_st, std::true_type{});
        }
        rd_stage = nx_stage;
      }
      if (active) epilogue(cur);
    }
    wait_vmcnt<0>();
    return;
  } else if constexpr (Tile::PAIR != 0) {
    // ---- slab pairs ---------------------------------------------------------------------------------------
    // The K loop in units of two slabs (a, b), a even.  Multiplying is as in the loop below - every slab in two
    // halves around its barrier, the first fetching the lower A rows of its slab from LDS, the second the next
    // slab's upper A rows and B fragments (B alternates between two register sets, so these go out at the start
    // of the half, not as the last MFMAs release the registers).  Loading differs: a wave requests block i of
    // slab a' and block i of slab b' back to back - the same 16 rows, the two 64-byte halves of the same lines.
    // Measured with the loads alone (no MFMAs, constant operands), such pairs against one slab at a time:
    // M=N=8192 K=8192 0.67 against 0.73 ms, M=24576 N=3072 K=768 0.069 against 0.090 ms.
    // With slab t in ring stage t % 5, the two stages of the pair (a + 4, a + 5) are both free behind a's barrier
    // (a's own stage and that of the slab before it).  A wave requests its four blocks of that pair one per half
    // slab - second half of a, both halves of b, first half of a + 2 - so every half issues two loads, as in the
    // loop below, and a load has one to three slab times to arrive.  Which tile a request belongs to is a scalar
    // select per pair, so one loop body serves the whole K range of a tile and the hand-over to the next one.
    // Needs tiles of an even number of slabs, at least four.
    struct Panel {
      uint32_t lo, hi, bytes;
    };
    auto tile_panel = [&](int i) __attribute__((always_inline)) {
      Panel q;
      const void* base = p.a;
      uint32_t bytes = 0;
      if (i < my_tiles) {
        const TileCoord c = tile_coord(i);
        const int rows_a = (p.M - c.m0) < c.rows ? (p.M - c.m0) : c.rows;
        const int rows_b = (p.N - c.n0) < BN ? (p.N - c.n0) : BN;
        const T* Ab = reinterpret_cast<const T*>(p.a) + (int64_t)c.batch * p.sa + (int64_t)c.m0 * p.lda;
        const T* Bb = reinterpret_cast<const T*>(p.b) + (int64_t)c.batch * p.sb + (int64_t)c.n0 * p.ldb;
        const uint32_t bytes_a = rows_a > 0 ? clamp_records((((int64_t)rows_a - 1) * p.lda + p.K) * 2) : 0u;
        const uint32_t bytes_b = clamp_records((((int64_t)rows_b - 1) * p.ldb + p.K) * 2);
        base = loads_a ? (const void*)Ab : (const void*)Bb;
        bytes = loads_a ? bytes_a : bytes_b;
      }
      const uint64_t v = reinterpret_cast<uint64_t>(base);
      q.lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
      q.hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
      q.bytes = __builtin_amdgcn_readfirstlane(bytes);
      return q;
    };
    auto panel_rsrc = [&](const Panel& q) __attribute__((always_inline)) {
      return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uint64_t)q.hi << 32) | q.lo), 0, q.bytes,
                                               0x00020000);
    };
    // byte offset of the lane's chunk in block i of the wave (every load has its own LDS base here)
    uint32_t lp_off[L];
#pragma unroll
    for (int i = 0; i < L; ++i) {
      const int j = wave * LM + i;
      const int row = (loads_a ? j : j - Tile::A_MAIN) * Tile::ROWS_PER_LOAD + l_row;
      lp_off[i] = (uint32_t)(((int64_t)row * (loads_a ? p.lda : p.ldb) + l_chunk_k[i]) * 2);
    }
    auto ring_stage = [&](int st) __attribute__((always_inline)) { return smem + st * Tile::STAGE_ELEMS; };
    auto wrap = [](int st) __attribute__((always_inline)) { return st >= NS ? st - NS : st; };
    // blocks [I0, I1) of the wave for the slabs kt (even) and kt + 1 of the tile behind d, into stages sa_ and sb_
    auto issue_pair = [&](auto i0_c, auto i1_c, const __amdgpu_buffer_rsrc_t& d, int kt, int sa_, int sb_)
                          __attribute__((always_inline)) {
      constexpr int I0 = decltype(i0_c)::value, I1 = decltype(i1_c)::value;
      const int k0 = kt * BK;
      static_for<I0, I1>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        const uint32_t off_a = (k0 + l_chunk_k[i] < p.K) ? lp_off[i] + (uint32_t)(k0 * 2) : kOobOffset;
        const uint32_t off_b = (k0 + BK + l_chunk_k[i] < p.K) ? lp_off[i] + (uint32_t)((k0 + BK) * 2) : kOobOffset;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(d, (lds_void*)(ring_stage(sa_) + (l_block0 + i) * 512), 16, off_a, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(d, (lds_void*)(ring_stage(sb_) + (l_block0 + i) * 512), 16, off_b, 0, 0, 0);
      });
    };
    constexpr std::integral_constant<int, 0> b_0{};
    constexpr std::integral_constant<int, 1> b_1{};
    constexpr std::integral_constant<int, 2> b_2{};
    constexpr std::integral_constant<int, 3> b_3{};
    constexpr std::integral_constant<int, 4> b_4{};
    static_assert(L == 4, "four blocks per wave, one per half slab of a pair");
    Panel cur_p = tile_panel(0), nxt_p = cur_p;
    // prologue: pair 0 whole and blocks 0 to 2 of pair 1 (what the three halves before the loop would have
    // requested); slab 0 has landed when only its successor's last block and pair 1's six loads are outstanding
    {
      const __amdgpu_buffer_rsrc_t d0 = panel_rsrc(cur_p);
      issue_pair(b_0, b_4, d0, 0, 0, 1);
      issue_pair(b_0, b_3, d0, 2, 2, 3);
      wait_vmcnt<7>();
      __builtin_amdgcn_s_barrier();
    }
    vec8 bfn[NI];  // B fragments of a pair's second slab
    load_a(smem, 0, af[0]);
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) bf[0][ni] = load_b1(smem, 0, ni);
    int sa = 0;  // ring stage of the pair's first slab

    // One pair in stages sa, sa + 1.  (p1, kt1): panel and first slab of the next pair (its block 3 goes out in the
    // first half of a); (p2, kt2): of the pair after that (blocks 0 to 2, in the three halves behind a's barrier).
    auto pair = [&](auto active_c, auto first_c, const Panel& p1, int kt1, const Panel& p2, int kt2) __attribute__((always_inline)) {
      constexpr bool ACTIVE = decltype(active_c)::value;
      constexpr bool FIRST = decltype(first_c)::value;  // the tile's first pair: slab a starts the accumulators
      const int s1 = wrap(sa + 1), s2 = wrap(sa + 2), s3 = wrap(sa + 3), s4 = wrap(sa + 4);
      const T* st_a = ring_stage(sa);
      const T* st_b = ring_stage(s1);
      const T* st_n = ring_stage(s2);
      const __amdgpu_buffer_rsrc_t d2 = panel_rsrc(p2);
      // first half of a
      issue_pair(b_3, b_4, panel_rsrc(p1), kt1, s2, s3);
      if constexpr (ACTIVE) {
        load_a(st_a, 1, af[1]);
        if constexpr (FIRST)
          mfmas_first(af[0], bf[0]);
        else
          mfmas(af[0], bf[0]);
      }
      // slab b has landed: only the eight loads of the four halves since its last block are younger.  The LDS reads
      // of a are waited for as well (they were issued a half slab ago): a's stage is written to behind the barrier.
      __builtin_amdgcn_s_waitcnt((8 & 0xf) | (0x7 << 4) | (0 << 8));
      __builtin_amdgcn_s_barrier();
      // second half of a
      issue_pair(b_0, b_1, d2, kt2, s4, sa);
      if constexpr (ACTIVE) {
        load_a(st_b, 0, af[0]);
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) bfn[ni] = load_b1(st_b, 0, ni);
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
          for (int mi = 0; mi < MH2; ++mi)
            acc[MH + mi][ni] = Mfma::run(bf[0][ni], af[1][mi], FIRST ? acc_t{} : acc[MH + mi][ni]);
      }
      // first half of b
      issue_pair(b_1, b_2, d2, kt2, s4, sa);
      if constexpr (ACTIVE) {
        load_a(st_b, 1, af[1]);
        mfmas(af[0], bfn);
      }
      wait_vmcnt<5>();  // the next pair's first slab has landed: younger are its last block's other half and two blocks
      __builtin_amdgcn_s_barrier();
      // second half of b
      issue_pair(b_2, b_3, d2, kt2, s4, sa);
      if constexpr (ACTIVE) {
        load_a(st_n, 0, af[0]);
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) bf[0][ni] = load_b1(st_n, 0, ni);
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
          for (int mi = 0; mi < MH2; ++mi) acc[MH + mi][ni] = Mfma::run(bfn[ni], af[1][mi], acc[MH + mi][ni]);
      }
      sa = s2;
    };
    const int n_pairs = k_tiles / 2;  // (the launcher checks: an even number of slabs, at least four)
    auto tile_pairs = [&](auto active_c) __attribute__((always_inline)) {
      auto one = [&](auto first_c, int j) __attribute__((always_inline)) {
        const bool in1 = j + 1 < n_pairs, in2 = j + 2 < n_pairs;
        Panel p1, p2;
        p1.lo = in1 ? cur_p.lo : nxt_p.lo;
        p1.hi = in1 ? cur_p.hi : nxt_p.hi;
        p1.bytes = in1 ? cur_p.bytes : nxt_p.bytes;
        p2.lo = in2 ? cur_p.lo : nxt_p.lo;
        p2.hi = in2 ? cur_p.hi : nxt_p.hi;
        p2.bytes = in2 ? cur_p.bytes : nxt_p.bytes;
        pair(active_c, first_c, p1, in1 ? 2 * j + 2 : 0, p2, in2 ? 2 * j + 4 : 2 * (j + 2 - n_pairs));
      };
      one(std::true_type{}, 0);
      for (int j = 1; j < n_pairs; ++j) one(std::false_type{}, j);
    };
    for (int i = 0; i < my_tiles; ++i) {
      const TileCoord cur = tile_coord(i);
      nxt_p = tile_panel(i + 1);
      const bool active = wm * Tile::WTM < cur.rows;
      if (active) {
        tile_pairs(std::true_type{});
        // the stage of the tile's last slab is free until the next tile's first slab has passed its barrier, which
        // no wave reaches before every wave has left this epilogue
        strip = smem_raw + wrap(sa + NS - 1) * (Tile::STAGE_ELEMS * 2) + wave * Tile::STRIP_BYTES;
        epilogue(cur);
      } else {
        tile_pairs(std::false_type{});
      }
      cur_p = nxt_p;
    }
    wait_vmcnt<0>();
  } else {
  // prologue: slabs 0 .. NS-3 whole, slab NS-2 up to its first portion
#pragma unroll
  for (int s = 0; s < NS - 2; ++s) {
    // (portion by portion: the lane offsets assume the immediate offsets of a portion's loads)
    issue_part(c_0, c_P, rd, rdx, s, s);
    issue_part(c_P, c_L, rd, rdx, s, s);
  }
  issue_part(c_0, c_P, rd, rdx, NS - 2, NS - 2);
  wait_vmcnt<(NS - 3) * L + L_P0>();
  __builtin_amdgcn_s_barrier();
  int rd_stage = 0;
  load_frags(smem, 0, af[0], bf[0]);

  // one K-slab: ACTIVE waves multiply, the others only keep the ring turning
  // Tiles of more than 128 accumulator registers per lane: the first fragments of the next tile are not held in
  // registers through the epilogue (36 registers of a 10 x 4 block part, which the epilogue then spills around)
  // but fetched behind it; the slab they come from has landed and stays in its ring stage.
  constexpr bool kRefetch = KK == 1 && MI * NI * Tile::ACC_N > 128;
  auto slab = [&](auto active_c, auto first_c, const __amdgpu_buffer_rsrc_t& d1, const __amdgpu_buffer_rsrc_t& d1x, int kt1,
                  const __amdgpu_buffer_rsrc_t& d2, const __amdgpu_buffer_rsrc_t& d2x, int kt2,
                  auto last_c) __attribute__((always_inline)) {
    constexpr bool ACTIVE = decltype(active_c)::value, FIRST = decltype(first_c)::value;
    constexpr bool FETCH = !(decltype(last_c)::value && kRefetch);
    const T* cur_st = smem + rd_stage * Tile::STAGE_ELEMS;
    const int nx_stage = rd_stage + 1 == NS ? 0 : rd_stage + 1;
    const T* nxt_st = smem + nx_stage * Tile::STAGE_ELEMS;
    const int st1 = rd_stage + D1 >= NS ? rd_stage + D1 - NS : rd_stage + D1;
    const int st2 = rd_stage + D2 >= NS ? rd_stage + D2 - NS : rd_stage + D2;
    // first step: the rest of the slab whose first portion went out in the previous slab's last step
    issue_part(c_P, c_L, d1, d1x, kt1, st1);
    if constexpr (ACTIVE) {
      half1_reads(cur_st);
      half1_mfmas(first_c);
      if constexpr (KK == 2) sched_step<MI * NI, MI + NI, L - L_P0>();
    }
    // last step: the next slab has landed once at most (NS-3) younger slabs are in flight; past
    // the barrier nobody reads the previous slab any more, so its ring slot starts taking a new
    // slab, and the next slab's first fragments are fetched under this slab's last MFMAs
    wait_vmcnt<(NS - 3) * L>();
    __builtin_amdgcn_s_barrier();
    issue_part(c_0, c_P, d2, d2x, kt2, st2);
    if constexpr (ACTIVE) {
      if constexpr (FETCH) half2_reads(nxt_st);
      half2_mfmas(first_c, nxt_st, std::integral_constant<bool, FETCH>{});
      // (one-step slabs take no scheduling hints: reads in pairs behind the first MFMAs and loads spread over
      // the rest, the order the hints give two-step slabs, ran 3 to 5 % slower there than the compiler's own)
      if constexpr (KK == 2) sched_step<MI * NI, MI + NI, L_P0>();
    }
    rd_stage = nx_stage;
  };
  auto tile_slabs = [&](auto active_c) __attribute__((always_inline)) {
    constexpr std::false_type no{};
    slab(active_c, std::true_type{}, rd, rdx, D1, rd, rdx, D2, no);
    for (int kt = 1; kt < k_tiles - D2; ++kt) slab(active_c, no, rd, rdx, kt + D1, rd, rdx, kt + D2, no);
    slab(active_c, no, rd, rdx, k_tiles - 1, nrd, nrdx, 0, no);
    static_for<1, D2 - 1>([&](auto t_c) {
      constexpr int t = decltype(t_c)::value;
      slab(active_c, no, nrd, nrdx, t - 1, nrd, nrdx, t, no);
    });
    slab(active_c, no, nrd, nrdx, D2 - 2, nrd, nrdx, D2 - 1, std::true_type{});
  };

  for (int i = 0; i < my_tiles; ++i) {
    const TileCoord cur = tile_coord(i);
    tile_desc(i + 1, nrd, nrdx);
    // waves whose rows lie outside a half tile keep the ring turning (their share of the loads, the
    // waits and the barriers) but multiply and store nothing; a half tile is always the last item
    const bool active = wm * Tile::WTM < cur.rows;
    if (active) {
      tile_slabs(std::true_type{});
      epilogue(cur);
      if constexpr (kRefetch) load_frags(smem + rd_stage * Tile::STAGE_ELEMS, 0, af[0], bf[0]);
    } else {
      tile_slabs(std::false_type{});
    }
    rd = nrd;
    if constexpr (XTRA > 0) rdx = nrdx;
  }
  // no LDS-DMA may be in flight into a workgroup that has ended
  wait_vmcnt<0>();
  }
}

}  // namespace aitamd
