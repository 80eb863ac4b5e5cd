// One translation unit per (epilogue, dtype): compiled repeatedly by the
// Makefile with -DAITAMD_EPI=<EpilogueId> -DAITAMD_DT=<0 fp16 | 1 bf16>.
// It instantiates every tile of gemm_tiles.inc for that pair and exports the
// resulting launcher table under a C symbol the dispatcher looks up.
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "gemm_host.hpp"
#include "gemm_kernel_dma.hpp"
#include "gemm_kernel_persist.hpp"

#ifndef AITAMD_EPI
#error "compile with -DAITAMD_EPI=<id>"
#endif
#ifndef AITAMD_DT
#error "compile with -DAITAMD_DT=<0|1>"
#endif

namespace aitamd {
namespace {

#if AITAMD_DT == 0
using Elem = f16;
#define AITAMD_DT_NAME "f16"
#else
using Elem = bf16;
#define AITAMD_DT_NAME "bf16"
#endif

constexpr int kMaxDevices = 64;

using Epi = Epilogue<AITAMD_EPI>;

// Kernels with the permuted store exist for the two epilogues the permuting ops use.
constexpr bool kHasPermutedStore = AITAMD_EPI == kEpiNone || AITAMD_EPI == kEpiBias;

// Kernels for operands that are not K-contiguous exist on the direct-to-LDS tiles whose edges allow it, for the
// epilogues the reference's ops in those layouts use: plain and residual-add in all of rrr, ccr, crr; bias for
// rrr with the permuted store (gemm_rrr_bias_permute).  kLayoutBits: bit L set when layout L is compiled.
constexpr int kLayoutBits = (AITAMD_EPI == kEpiNone || AITAMD_EPI == kEpiAdd) ? 0xf : (AITAMD_EPI == kEpiBias ? 0x3 : 0x1);
constexpr bool kLayoutsArePermuted = AITAMD_EPI == kEpiBias;  // the bias kernels of the other layouts store permuted

constexpr int kShortK = 4;
template <class Tile, bool PERM, int LAYOUT>
struct KernelOf {
  static constexpr auto value = gemm_rcr_kernel<Elem, Tile, Epi, PERM, LAYOUT>;
};
template <int BM, int BN, int BK, int WM, int WN, int NS, int OCC, int PIPE, int MT, int AUX, int MODE, bool PERM,
          int LAYOUT>
struct KernelOf<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX, MODE>, PERM, LAYOUT> {
  static constexpr auto value =
      gemm_rcr_dma_kernel<Elem, GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX, MODE>, Epi, PERM, LAYOUT>;
};

template <int BM, int BN, int BK, int WM, int WN, int NS, int MT, int LBM, int PAIR, bool PERM, int LAYOUT>
struct KernelOf<GemmTilePersist<BM, BN, BK, WM, WN, NS, MT, LBM, PAIR>, PERM, LAYOUT> {
  // (LAYOUT 4 is not an operand layout: it names the instantiation for tiles of fewer K-slabs than ring stages)
  static constexpr auto value =
      gemm_rcr_persist_kernel<Elem, GemmTilePersist<BM, BN, BK, WM, WN, NS, MT, LBM, PAIR>, Epi, PERM, LAYOUT == kShortK>;
};
// the slab-pair form of a persistent tile (the tile itself where it has none)
template <class Tile>
struct PairOf {
  using type = Tile;
};
template <int BM, int BN, int BK, int WM, int WN, int MT, int LBM>
struct PairOf<GemmTilePersist<BM, BN, BK, WM, WN, 4, MT, LBM, 0>> {
  using Plain = GemmTilePersist<BM, BN, BK, WM, WN, 4, MT, LBM, 0>;
  using type = std::conditional_t<Plain::kPairable,
                                  GemmTilePersist<BM, BN, BK, WM, WN, 5, MT, LBM, Plain::kPairable ? 1 : 0>, Plain>;
};
// bit L set: the tile has a kernel for layout L (bit 0, rcr, always)
template <class Tile>
struct LayoutMask {
  static constexpr int value = 1;
};
// the element-wide loads take every layout: the instance of last resort for pitches and K that the
// 16-byte loads cannot take
template <int BM, int BN, int BK, int WM, int WN>
struct LayoutMask<GemmTile<BM, BN, BK, WM, WN, 1>> {
  static constexpr int value = kLayoutBits;
};
template <int BM, int BN, int BK, int WM, int WN, int NS, int OCC, int PIPE, int MT, int AUX>
struct LayoutMask<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX, 0>> {
  static constexpr int value =
      GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX>::kTransposable ? kLayoutBits : 1;
};
// split-K form: rcr only
template <class Tile>
struct IsSplitK {
  static constexpr bool value = false;
};
template <int BM, int BN, int BK, int WM, int WN, int NS, int OCC, int PIPE, int MT, int AUX, int MODE>
struct IsSplitK<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX, MODE>> {
  static constexpr bool value = (MODE & 1) != 0;
};
template <class Tile>
struct IsPersistent {
  static constexpr bool value = false;
};
template <int BM, int BN, int BK, int WM, int WN, int NS, int MT, int LBM, int PAIR>
struct IsPersistent<GemmTilePersist<BM, BN, BK, WM, WN, NS, MT, LBM, PAIR>> {
  static constexpr bool value = true;
};

// Workgroups per tile of a split-K launch: as many as bring the grid up to about one workgroup per CU, each with
// at least two K-slabs, at most 16; 1 (no splitting, nothing written to the scratch memory) for grids that fill
// the device anyway.
template <class Tile>
int split_k_factor(const GemmParams& p, int cus) {
  const int64_t tiles = (int64_t)((p.M + Tile::BM - 1) / Tile::BM) * ((p.N + Tile::BN - 1) / Tile::BN) * p.batch;
  const int64_t k_tiles = ((Tile::KVEC == 8 ? p.K : (p.K & ~7)) + Tile::BK - 1) / Tile::BK;
  return split_k_rule(tiles, k_tiles, cus);
}
template <class Tile>
int64_t workspace_of(const GemmParams& p) {
  if constexpr (IsSplitK<Tile>::value) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    const int64_t tiles = (int64_t)((p.M + Tile::BM - 1) / Tile::BM) * ((p.N + Tile::BN - 1) / Tile::BN) * p.batch;
    const int s = split_k_factor<Tile>(p, device_cus(dev));
    return s > 1 ? Tile::ws_bytes(tiles, s) : 0;
  }
  return 0;
}

// Column blocks of the per-XCD block mapping of the persistent kernels (GemmParams::xcd_cols; 0: the grouped
// mapping).  The grid of one batch is cut into xcd_cols column blocks times 8 / xcd_cols row blocks, one per XCD,
// where it divides so and the B panels of a block's columns take at most 2.5 MiB; the fewest column blocks that fit
// are taken, which share an A panel among the most tiles.  An XCD then reads few B panels over and over and every
// A panel once.  Measured on M=24576 N=3072 K=768 (two column blocks of six tile columns): 158 MB fetched per launch
// against 176 MB with the grouped mapping, 0.5 % (normally distributed operands) to 2 % (constant ones) less time.
// The B panels do not stay in the 4 MiB L2 from one block row to the next all the same: a round of 32 tiles streams
// 4.4 MB of distinct panel data between two uses of a B line (loading A with the non-temporal policy to protect B
// loses the sharing of A among the tiles of a row: 0.159 against 0.123 ms).
inline int xcd_column_blocks(const GemmParams& p, int bn, int grid) {
  if (p.batch != 1 || grid % 8 != 0 || p.tiles_m <= 0 || p.tiles_n <= 0) return 0;
  for (int a = 1; a <= 8; a *= 2) {
    if (p.tiles_n % a != 0 || p.tiles_m % (8 / a) != 0) continue;
    const int64_t b_bytes = (int64_t)(p.tiles_n / a) * bn * p.K * 2;
    if (b_bytes <= (5ll << 19)) return a;
  }
  return 0;
}

template <class Tile, bool PERM, int LAYOUT = 0>
hipError_t launch_kernel(const GemmParams& p_in, hipStream_t stream) {
  auto kernel = KernelOf<Tile, PERM, LAYOUT>::value;
  // LDS above 64 KiB has to be opted into once per device.
  static std::once_flag once[kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  // the outcome is kept per device: a failed opt-in must fail every later call too, not only the first
  static hipError_t attr_errs[kMaxDevices];
  hipError_t& attr_err = attr_errs[dev % kMaxDevices];
  std::call_once(once[dev % kMaxDevices], [&] {
    attr_err = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, Tile::kLdsBytes);
  });
  if (attr_err != hipSuccess) return attr_err;

  GemmParams p = p_in;
  // streaming stores for outputs that will not be cached anyway (the 8 L2s hold 32 MiB together); the
  // buffer form needs one batch of the output to span less than 2 GiB
  {
    static const long long nt_min = getenv("AITAMD_NT_MIN_BYTES") ? atoll(getenv("AITAMD_NT_MIN_BYTES")) : (32ll << 20);
    const long long span = p.perm_on ? (long long)p.M * p.N * 2 : ((long long)(p.M - 1) * p.ldc + p.N) * 2;
    p.nt_store = (long long)p.M * p.N * p.batch * 2 >= nt_min && span < 0x7fffffffll;
  }
  p.tiles_m = (p.M + Tile::BM - 1) / Tile::BM;
  p.tiles_n = (p.N + Tile::BN - 1) / Tile::BN;
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles <= 0 || p.batch <= 0) return hipSuccess;
  // one workgroup per (batch, tile) pair, or, for the persistent kernels, one per CU walking them
  const int64_t total = tiles * p.batch;
  if (total > 0x7fffffffll) return hipErrorInvalidValue;
  dim3 grid((unsigned)total, 1, 1);
  if constexpr (IsPersistent<Tile>::value) {
    const int cus = device_cus(dev);
    grid = dim3((unsigned)(total < cus ? total : cus), 1, 1);
    p.xcd_cols = xcd_column_blocks(p, Tile::BN, (int)grid.x);
    // few tile columns: the grouped walk goes row by row, so that the run of tiles of an XCD ends inside at most
    // one row of tiles whose A panel a second XCD then fetches too (eight rows with the default group height;
    // measured on M=24576 N=768 K=3072 and M=12608 N=1024 K=4096: 1 % less time)
    p.group_m = p.tiles_n <= 4 ? 1 : 8;
  }
  if constexpr (IsSplitK<Tile>::value) {
    // tiles are shared along K only with enough scratch memory to hold the partial tiles; without it the
    // instance runs as its plain counterpart (one workgroup per tile, nothing written to the scratch memory)
    p.split_k = split_k_factor<Tile>(p, device_cus(dev));
    if (p.ws == nullptr || p.ws_bytes < Tile::ws_bytes(total, p.split_k) || total * p.split_k > 0x7fffffffll)
      p.split_k = 1;
    grid = dim3((unsigned)(total * p.split_k), 1, 1);
  }
  hipLaunchKernelGGL(kernel, grid, dim3(Tile::NT), Tile::kLdsBytes, stream, p);
  return hipGetLastError();
}

template <class Tile>
hipError_t launch_tile(const GemmParams& p, hipStream_t stream) {
  if (p.layout != 0) {
    constexpr int mask = LayoutMask<Tile>::value;
    if ((p.perm_on != 0) != kLayoutsArePermuted) return hipErrorInvalidValue;
    if constexpr ((mask & 2) != 0) {
      if (p.layout == 1) return launch_kernel<Tile, kLayoutsArePermuted, 1>(p, stream);
    }
    if constexpr ((mask & 4) != 0) {
      if (p.layout == 2) return launch_kernel<Tile, kLayoutsArePermuted, 2>(p, stream);
    }
    if constexpr ((mask & 8) != 0) {
      if (p.layout == 3) return launch_kernel<Tile, kLayoutsArePermuted, 3>(p, stream);
    }
    return hipErrorInvalidValue;
  }
  if constexpr (IsPersistent<Tile>::value) {
    const int64_t k_tiles = ((int64_t)p.K + Tile::BK - 1) / Tile::BK;
    if (k_tiles < Tile::NS) {
      if (p.perm_on) {
        if constexpr (kHasPermutedStore) return launch_kernel<Tile, true, kShortK>(p, stream);
        return hipErrorInvalidValue;
      }
      return launch_kernel<Tile, false, kShortK>(p, stream);
    }
    // tiles of an even number of K-slabs go to the slab-pair form of the kernel where the tile has one: the same
    // products summed in the same order (the results are the same bit for bit), the loads better ordered
    using Pair = typename PairOf<Tile>::type;
    if constexpr (!std::is_same_v<Pair, Tile>) {
      // (AITAMD_NO_SLAB_PAIRS=1 keeps every tile on the one-slab form, for measuring one against the other)
      static const bool pairs_on = !(getenv("AITAMD_NO_SLAB_PAIRS") && atoi(getenv("AITAMD_NO_SLAB_PAIRS")) != 0);
      if (pairs_on && k_tiles % 2 == 0 && k_tiles >= Tile::kPairMinSlabs) {
        if (p.perm_on) {
          if constexpr (kHasPermutedStore) return launch_kernel<Pair, true>(p, stream);
          return hipErrorInvalidValue;
        }
        return launch_kernel<Pair, false>(p, stream);
      }
    }
  }
  if (p.perm_on) {
    if constexpr (kHasPermutedStore) return launch_kernel<Tile, true>(p, stream);
    return hipErrorInvalidValue;
  }
  return launch_kernel<Tile, false>(p, stream);
}

// Workgroups one CU can hold: limited by LDS (160 KiB) and by the register file
// (512 VGPRs per SIMD lane shared by the waves of a SIMD).
constexpr int kLdsPerCu = 160 * 1024;
constexpr int staged_wgs_per_cu(int bm, int bn, int nt, int lds) {
  const int acc = bm * bn / nt;                       // fp32 accumulators per lane
  const int regs = acc + 96;                          // plus staging / fragments / addresses
  const int waves_per_simd = 512 / regs > 0 ? 512 / regs : 1;
  const int by_regs = waves_per_simd * 4 / (nt / 64) > 0 ? waves_per_simd * 4 / (nt / 64) : 1;
  const int by_lds = kLdsPerCu / lds > 0 ? kLdsPerCu / lds : 1;
  return by_regs < by_lds ? by_regs : by_lds;
}
constexpr int dma_wgs_per_cu(int nt, int occ, int lds) {
  const int waves_per_wg_per_simd = nt / 64 / 4 > 0 ? nt / 64 / 4 : 1;
  const int by_regs = occ / waves_per_wg_per_simd > 0 ? occ / waves_per_wg_per_simd : 1;
  const int by_lds = kLdsPerCu / lds > 0 ? kLdsPerCu / lds : 1;
  return by_regs < by_lds ? by_regs : by_lds;
}

#define AITAMD_STR2(x) #x
#define AITAMD_STR(x) AITAMD_STR2(x)

const GemmAlgo kAlgos[] = {
#define AITAMD_GEMM_TILE(BM, BN, BK, WM, WN, KV)                                              \
  {"gemm_rcr_" AITAMD_DT_NAME "_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_v" #KV,                \
   BM, BN, BK, GemmTile<BM, BN, BK, WM, WN, KV>::NT, KV, GemmTile<BM, BN, BK, WM, WN, KV>::kLdsBytes, \
   staged_wgs_per_cu(BM, BN, GemmTile<BM, BN, BK, WM, WN, KV>::NT,                                  \
                     GemmTile<BM, BN, BK, WM, WN, KV>::kLdsBytes),                                  \
   0, LayoutMask<GemmTile<BM, BN, BK, WM, WN, KV>>::value, &launch_tile<GemmTile<BM, BN, BK, WM, WN, KV>>, nullptr},
#define AITAMD_GEMM_TILE_DMA(BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX)                                 \
  {"gemm_rcr_" AITAMD_DT_NAME "_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_dma" #NS "_o" #OCC "_p" #PIPE "_m" #MT \
   "_c" #AUX,                                                                                              \
   BM, BN, BK, GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX>::NT, 8,                             \
   GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX>::kLdsBytes,                                     \
   dma_wgs_per_cu(GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX>::NT, OCC,                        \
                  GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX>::kLdsBytes),                      \
   1, LayoutMask<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX>>::value,                            \
   &launch_tile<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, AUX>>, nullptr},
#define AITAMD_GEMM_TILE_PERSIST(BM, BN, BK, WM, WN, NS, MT, LBM)                                         \
  {"gemm_rcr_" AITAMD_DT_NAME "_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_persist" #NS "_m" #MT,                \
   BM, BN, BK, GemmTilePersist<BM, BN, BK, WM, WN, NS, MT, LBM>::NT, 8,                                     \
   GemmTilePersist<BM, BN, BK, WM, WN, NS, MT, LBM>::kLdsBytes,                                             \
   1, 2, 1, &launch_tile<GemmTilePersist<BM, BN, BK, WM, WN, NS, MT, LBM>>, nullptr},
#define AITAMD_GEMM_TILE_DMA_SPLITK(BM, BN, BK, WM, WN, NS, OCC, PIPE, MT)                                   \
  {"gemm_rcr_" AITAMD_DT_NAME "_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_dma" #NS "_o" #OCC "_p" #PIPE "_m" #MT \
   "_splitk",                                                                                             \
   BM, BN, BK, GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 1>::NT, 8,                             \
   GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 1>::kLdsBytes,                                     \
   dma_wgs_per_cu(GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 1>::NT, OCC,                        \
                  GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 1>::kLdsBytes),                      \
   4, 1, &launch_tile<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 1>>,                             \
   &workspace_of<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 1>>},
#define AITAMD_GEMM_TILE_DMA_K2(BM, BN, BK, WM, WN, NS, OCC, PIPE, MT)                                      \
  {"gemm_rcr_" AITAMD_DT_NAME "_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_dma" #NS "_o" #OCC "_p" #PIPE "_m" #MT \
   "_k2",                                                                                                 \
   BM, BN, BK, GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 2>::NT, 2,                             \
   GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 2>::kLdsBytes,                                     \
   dma_wgs_per_cu(GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 2>::NT, OCC,                        \
                  GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 2>::kLdsBytes),                      \
   1, 1, &launch_tile<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 2>>, nullptr},
#define AITAMD_GEMM_TILE_DMA_SPLITK_K2(BM, BN, BK, WM, WN, NS, OCC, PIPE, MT)                                \
  {"gemm_rcr_" AITAMD_DT_NAME "_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_dma" #NS "_o" #OCC "_p" #PIPE "_m" #MT \
   "_k2_splitk",                                                                                          \
   BM, BN, BK, GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 3>::NT, 2,                             \
   GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 3>::kLdsBytes,                                     \
   dma_wgs_per_cu(GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 3>::NT, OCC,                        \
                  GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 3>::kLdsBytes),                      \
   4, 1, &launch_tile<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 3>>,                             \
   &workspace_of<GemmTileDma<BM, BN, BK, WM, WN, NS, OCC, PIPE, MT, 0, 3>>},
#include "gemm_tiles.inc"
#undef AITAMD_GEMM_TILE
#undef AITAMD_GEMM_TILE_DMA
#undef AITAMD_GEMM_TILE_DMA_K2
#undef AITAMD_GEMM_TILE_DMA_SPLITK_K2
#undef AITAMD_GEMM_TILE_PERSIST
#undef AITAMD_GEMM_TILE_DMA_SPLITK
};

}  // namespace
}  // namespace aitamd

#define AITAMD_CAT3(a, b, c) a##b##_##c
#define AITAMD_TABLE_SYM(e, d) AITAMD_CAT3(aitamd_gemm_table_, e, d)

extern "C" __attribute__((visibility("hidden"))) aitamd::GemmAlgoTable AITAMD_TABLE_SYM(AITAMD_EPI, AITAMD_DT)() {
  return {aitamd::kAlgos, (int)(sizeof(aitamd::kAlgos) / sizeof(aitamd::kAlgos[0]))};
}
