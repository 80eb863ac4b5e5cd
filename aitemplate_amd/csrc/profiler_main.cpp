// Profiler executable of the GEMM family: times every compiled instance that
// supports the given problem and prints one line per instance,
//     OP:<instance name>,TIME:<ms>,WS:<workspace bytes>
// which is the protocol the host-side runner parses
// (python/aitemplate/backend/profiler_runner.py:40).  It replaces the profiler
// programs the reference renders and compiles per op
// (python/aitemplate/backend/rocm/gemm/common.py:313-488, bmm_common.py:155-175,
// bmm_softmax_bmm_permute.py:113-158): being one prebuilt binary over the
// kernel library's C ABI, nothing is compiled at profiling time.
//
// usage:
//   aitamd_profiler gemm <op_name> <dtype:0|1> M N K [split_k]
//   aitamd_profiler bmm  bmm_rcr   <dtype> B M N K
//   aitamd_profiler attn bmm_softmax_bmm_permute <dtype> B M N K O heads [causal]
//   aitamd_profiler ew   <FuncEnum value> <dtype> numel [b_period]   (stand-alone element-wise kernel)
//   aitamd_profiler copy rows <dtype, unused> rows row_bytes pitch_bytes  (row copy out of a pitched buffer)
// environment: AITAMD_PROF_WARMUP (default 3), AITAMD_PROF_ITERS (default 10),
//              AITAMD_PROF_ALGO=<name or index> restricts the run to one instance.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "../../include/aitemplate_amd_kernels.h"

#define HIP_OK(call)                                                                       \
  do {                                                                                     \
    hipError_t e_ = (call);                                                                \
    if (e_ != hipSuccess) {                                                                \
      fprintf(stderr, "%s failed: %s (%s:%d)\n", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
      exit(2);                                                                             \
    }                                                                                      \
  } while (0)

namespace {

// Operands rotate through a pool larger than the 256 MiB Infinity Cache so that
// every timed launch reads its inputs from HBM, as the reference's rotating
// ProfilerMemoryPool does for L2 (backend/rocm/gemm/common.py:315-325).
constexpr size_t kPoolTargetBytes = 512ull << 20;
constexpr int kMaxSets = 16;

uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  uint16_t b;
  memcpy(&b, &h, 2);
  return b;
}
uint16_t f32_to_bf16_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

struct Rng {
  uint64_t s;
  float uniform() {  // [-1, 1)
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    return (float)((s >> 40) & 0xffffff) / 8388608.0f - 1.0f;
  }
};

struct DeviceBuf {
  void* p = nullptr;
  size_t bytes = 0;
};

DeviceBuf alloc_random(size_t elems, int dtype, float scale, uint64_t seed) {
  DeviceBuf d;
  d.bytes = elems * 2;
  if (elems == 0) return d;
  HIP_OK(hipMalloc(&d.p, d.bytes));
  std::vector<uint16_t> h(elems);
  Rng r{seed * 0x9e3779b97f4a7c15ull + 1};
  for (size_t i = 0; i < elems; ++i) {
    const float v = r.uniform() * scale;
    h[i] = dtype == 0 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
  }
  HIP_OK(hipMemcpy(d.p, h.data(), d.bytes, hipMemcpyHostToDevice));
  return d;
}

DeviceBuf alloc_copy_of(const DeviceBuf& src) {
  DeviceBuf d;
  d.bytes = src.bytes;
  if (src.bytes == 0) return d;
  HIP_OK(hipMalloc(&d.p, d.bytes));
  HIP_OK(hipMemcpy(d.p, src.p, d.bytes, hipMemcpyDeviceToDevice));
  return d;
}

int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return v && *v ? atoi(v) : dflt;
}

int epilogue_of(const std::string& op) {
  static const char* names[] = {"gemm_rcr", "gemm_rcr_bias", "gemm_rcr_bias_relu", "gemm_rcr_bias_gelu",
                                "gemm_rcr_bias_add", "gemm_rcr_bias_add_add", "gemm_rcr_bias_add_relu",
                                "gemm_rcr_bias_add_add_relu", "gemm_rcr_bias_sigmoid", "gemm_rcr_bias_tanh",
                                "gemm_rcr_bias_swish", "gemm_rcr_bias_hardswish", "gemm_rcr_bias_mul",
                                "gemm_rcr_bias_mul_add", "gemm_rcr_bias_sigmoid_mul",
                                "gemm_rcr_bias_sigmoid_mul_tanh", "gemm_rcr_bias_mul_tanh"};
  if (op == "gemm_rcr_bias_fast_gelu") return AITAMD_EPI_BIAS_GELU;
  if (op == "bmm_rcr") return AITAMD_EPI_NONE;
  if (op == "bmm_add") return AITAMD_EPI_ADD;
  for (int i = 0; i < AITAMD_NUM_EPILOGUES; ++i)
    if (op == names[i]) return i;
  return -1;
}

int num_residuals(int epi) {
  switch (epi) {
    case AITAMD_EPI_BIAS_ADD:
    case AITAMD_EPI_BIAS_ADD_RELU:
    case AITAMD_EPI_BIAS_MUL:
    case AITAMD_EPI_BIAS_SIGMOID_MUL:
    case AITAMD_EPI_BIAS_SIGMOID_MUL_TANH:
    case AITAMD_EPI_BIAS_MUL_TANH:
    case AITAMD_EPI_ADD:
      return 1;
    case AITAMD_EPI_BIAS_ADD_ADD:
    case AITAMD_EPI_BIAS_ADD_ADD_RELU:
    case AITAMD_EPI_BIAS_MUL_ADD:
      return 2;
    default:
      return 0;
  }
}

struct OperandSet {
  DeviceBuf a, b, bias, d0, d1, c;
};

// layout 0 = plain store; otherwise the permuting launcher with the op's (g1, g2, g3)
struct PermuteSpec {
  int layout = 0;
  int64_t g[3] = {1, 1, 1};
  int operands = 0;  // operand layout of the batched launcher: AITAMD_LAYOUT_*
};

// permuting op name -> base op (which names the epilogue) and layout id; false when `op` does not permute
bool permute_op(const std::string& op, std::string* base, int* layout) {
  static const struct {
    const char* op;
    const char* base;
    int layout;
  } table[] = {{"gemm_rcr_permute_m2n3", "gemm_rcr", AITAMD_PERMUTE_M2N3},
               {"gemm_rcr_bias_permute_m2n3", "gemm_rcr_bias", AITAMD_PERMUTE_M2N3},
               {"gemm_rcr_bias_permute_m3n2", "gemm_rcr_bias", AITAMD_PERMUTE_M3N2},
               {"gemm_rcr_bias_permute", "gemm_rcr_bias", AITAMD_PERMUTE_M3N2},
               {"gemm_rrr_bias_permute", "gemm_rcr_bias", AITAMD_PERMUTE_M3N2}};
  for (const auto& t : table)
    if (op == t.op) {
      *base = t.base;
      *layout = t.layout;
      return true;
    }
  return false;
}

int profile_gemm_like(const std::string& op, int dtype, int64_t B, int64_t M, int64_t N, int64_t K, bool batched,
                      const PermuteSpec& perm = PermuteSpec()) {
  const int epi = epilogue_of(op);
  if (epi < 0) {
    fprintf(stderr, "unknown op %s\n", op.c_str());
    return 2;
  }
  const int n_algos = aitamd_gemm_num_algos(epi, dtype);
  if (n_algos == 0) {
    fprintf(stderr, "no instances for %s dtype %d\n", op.c_str(), dtype);
    return 2;
  }
  const int nres = num_residuals(epi);
  const size_t set_bytes = 2 * (size_t)(B * (M * K + N * K + (1 + nres) * M * N) + N);
  int sets = (int)(kPoolTargetBytes / (set_bytes ? set_bytes : 1)) + 1;
  if (sets > kMaxSets) sets = kMaxSets;
  if (sets < 1) sets = 1;
  std::vector<OperandSet> pool(sets);
  const float wscale = K > 0 ? 1.0f / sqrtf((float)K) * 1.7320508f : 1.0f;  // unit-variance outputs
  for (int s = 0; s < sets; ++s) {
    OperandSet& o = pool[s];
    if (s == 0) {
      o.a = alloc_random((size_t)(B * M * K), dtype, 1.7320508f, 11);
      o.b = alloc_random((size_t)(B * N * K), dtype, wscale, 12);
      o.bias = alloc_random((size_t)N, dtype, 0.1f, 13);
      if (nres >= 1) o.d0 = alloc_random((size_t)(B * M * N), dtype, 1.0f, 14);
      if (nres >= 2) o.d1 = alloc_random((size_t)(B * M * N), dtype, 1.0f, 15);
    } else {
      o.a = alloc_copy_of(pool[0].a);
      o.b = alloc_copy_of(pool[0].b);
      o.bias = alloc_copy_of(pool[0].bias);
      o.d0 = alloc_copy_of(pool[0].d0);
      o.d1 = alloc_copy_of(pool[0].d1);
    }
    o.c.bytes = (size_t)(B * M * N) * 2;
    if (o.c.bytes) HIP_OK(hipMalloc(&o.c.p, o.c.bytes));
  }

  const int warmup = env_int("AITAMD_PROF_WARMUP", 3);
  const int iters = env_int("AITAMD_PROF_ITERS", 10);
  const char* only = getenv("AITAMD_PROF_ALGO");
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));

  // scratch memory of the instance being timed (the split-K ones; plain gemm_rcr ops only): zeroed once, the
  // launches leave its counters zero
  void* scratch = nullptr;
  size_t scratch_bytes = 0;
  auto launch = [&](int algo, const OperandSet& o) -> int {
    if (perm.layout && !batched && perm.operands == AITAMD_LAYOUT_RCR)
      return aitamd_gemm_rcr_permute(epi, dtype, algo, o.a.p, o.b.p, o.bias.p, o.c.p, M, N, K, K, K, perm.layout,
                                     perm.g[0], perm.g[1], perm.g[2], stream);
    if (batched && epi == AITAMD_EPI_ADD) {
      const int64_t lda = (perm.operands & 2) ? M : K, ldb = (perm.operands & 1) ? N : K;
      return aitamd_bmm_add(perm.operands, dtype, algo, o.a.p, o.b.p, o.d0.p, o.c.p, B, M, N, K, lda, ldb, N, N, M * K,
                            N * K, M * N, M * N, stream);
    }
    if (!batched && perm.layout && perm.operands != AITAMD_LAYOUT_RCR)
      return aitamd_gemm_permute(perm.operands, epi, dtype, algo, o.a.p, o.b.p, o.bias.p, o.c.p, M, N, K, K, N,
                                 perm.layout, perm.g[0], perm.g[1], perm.g[2], stream);
    if (batched && perm.operands != AITAMD_LAYOUT_RCR) {
      const int64_t lda = (perm.operands & 2) ? M : K, ldb = (perm.operands & 1) ? N : K;
      return aitamd_bmm(perm.operands, dtype, algo, o.a.p, o.b.p, o.c.p, B, M, N, K, lda, ldb, N, M * K, N * K, M * N,
                        perm.layout ? perm.g[0] : 0, stream);
    }
    if (batched && perm.layout)  // bmm_rcr_permute: perm.g[0] = d1
      return aitamd_bmm_rcr_permute(dtype, algo, o.a.p, o.b.p, o.c.p, B, M, N, K, K, K, M * K, N * K, perm.g[0], stream);
    if (batched)
      return aitamd_bmm_rcr(dtype, algo, o.a.p, o.b.p, o.c.p, B, M, N, K, K, K, N, M * K, N * K, M * N, stream);
    return aitamd_gemm_rcr_ws(epi, dtype, algo, o.a.p, o.b.p, o.bias.p, o.d0.p, o.d1.p, o.c.p, M, N, K, K, K, N, N,
                              scratch, (int64_t)scratch_bytes, stream);
  };

  int printed = 0;
  for (int algo = 0; algo < n_algos; ++algo) {
    const char* name = aitamd_gemm_algo_name(epi, dtype, algo);
    if (only && *only) {
      const bool numeric = only[0] >= '0' && only[0] <= '9';
      if (numeric ? atoi(only) != algo : strcmp(only, name) != 0) continue;
    }
    if (perm.operands != AITAMD_LAYOUT_RCR) {
      const int64_t lda = (perm.operands & 2) ? M : K, ldb = (perm.operands & 1) ? N : K;
      if (!aitamd_gemm_algo_supported_layout(epi, dtype, perm.operands, algo, M, N, K, lda, ldb, 16)) continue;
    } else if (!aitamd_gemm_algo_supported(epi, dtype, algo, M, N, K, K, K, 16)) {
      continue;
    }
    const bool plain = !batched && !perm.layout && perm.operands == AITAMD_LAYOUT_RCR;
    const int64_t ws = plain ? aitamd_gemm_workspace_bytes(epi, dtype, algo, 1, M, N, K) : 0;
    if (!plain && strstr(name, "_splitk")) continue;  // (the other entry points take no scratch memory)
    if (scratch) HIP_OK(hipFree(scratch));
    scratch = nullptr;
    scratch_bytes = (size_t)ws;
    if (ws > 0) {
      HIP_OK(hipMalloc(&scratch, scratch_bytes));
      HIP_OK(hipMemset(scratch, 0, scratch_bytes));
    } else if (strstr(name, "_splitk")) {
      continue;  // does not split on this problem: the same as the plain instance, which is timed anyway
    }
    bool ok = true;
    for (int i = 0; i < warmup && ok; ++i) ok = launch(algo, pool[i % sets]) == 0;
    if (!ok) {
      fprintf(stderr, "instance %s failed: %s\n", name, aitamd_last_error());
      continue;
    }
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipEventRecord(e0, stream));
    for (int i = 0; i < iters; ++i) launch(algo, pool[i % sets]);
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    printf("OP:%s,TIME:%.6f,WS:%lld\n", name, ms / (iters > 0 ? iters : 1), (long long)ws);
    fflush(stdout);
    ++printed;
  }
  if (scratch) HIP_OK(hipFree(scratch));
  HIP_OK(hipStreamDestroy(stream));
  return printed > 0 ? 0 : 3;
}

int profile_attention(int dtype, int64_t B, int64_t M, int64_t N, int64_t K, int64_t O, int64_t G, int causal) {
  const size_t set_bytes = 2 * (size_t)(B * (M * K + N * K + N * O + M * O));
  int sets = (int)(kPoolTargetBytes / (set_bytes ? set_bytes : 1)) + 1;
  if (sets > kMaxSets) sets = kMaxSets;
  std::vector<OperandSet> pool(sets);
  for (int s = 0; s < sets; ++s) {
    OperandSet& o = pool[s];
    if (s == 0) {
      o.a = alloc_random((size_t)(B * M * K), dtype, 1.7320508f, 21);
      o.b = alloc_random((size_t)(B * N * K), dtype, 1.7320508f, 22);
      o.d0 = alloc_random((size_t)(B * N * O), dtype, 1.7320508f, 23);
    } else {
      o.a = alloc_copy_of(pool[0].a);
      o.b = alloc_copy_of(pool[0].b);
      o.d0 = alloc_copy_of(pool[0].d0);
    }
    o.c.bytes = (size_t)(B * M * O) * 2;
    if (o.c.bytes) HIP_OK(hipMalloc(&o.c.p, o.c.bytes));
  }
  const int warmup = env_int("AITAMD_PROF_WARMUP", 3);
  const int iters = env_int("AITAMD_PROF_ITERS", 10);
  const float scale = K > 0 ? 1.0f / sqrtf((float)K) : 1.0f;
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  auto launch = [&](const OperandSet& o) {
    return aitamd_bmm_softmax_bmm_permute(dtype, o.a.p, o.b.p, o.d0.p, o.c.p, B, M, N, K, O, G, scale, causal, stream);
  };
  for (int i = 0; i < warmup; ++i) {
    if (launch(pool[i % sets]) != 0) {
      fprintf(stderr, "attention launch failed: %s\n", aitamd_last_error());
      return 3;
    }
  }
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipEventRecord(e0, stream));
  for (int i = 0; i < iters; ++i) launch(pool[i % sets]);
  HIP_OK(hipEventRecord(e1, stream));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  printf("OP:attention_q128,TIME:%.6f,WS:0\n", ms / (iters > 0 ? iters : 1));
  HIP_OK(hipStreamDestroy(stream));
  return 0;
}

// Element-wise kernel and row copy: one line each, operands rotating through the same kind of pool.
int profile_streaming(const std::string& kind, int func, int dtype, int64_t n0, int64_t n1, int64_t n2) {
  const bool ew = kind == "ew";
  const int64_t numel = ew ? n0 : 0, b_period = ew ? n1 : 0;
  const int64_t rows = ew ? 0 : n0, row_bytes = ew ? 0 : n1, pitch = ew ? 0 : n2;
  if (ew ? numel <= 0 : (rows <= 0 || row_bytes <= 0 || pitch < row_bytes)) {
    fprintf(stderr, "bad sizes\n");
    return 2;
  }
  const size_t in_bytes = ew ? (size_t)numel * 2 : (size_t)rows * pitch;
  const size_t out_bytes = ew ? (size_t)numel * 2 : (size_t)rows * row_bytes;
  int sets = (int)(kPoolTargetBytes / (in_bytes + out_bytes)) + 1;
  if (sets > kMaxSets) sets = kMaxSets;
  if (sets < 2) sets = 2;
  std::vector<DeviceBuf> in(sets), in2(sets), out(sets);
  for (int s = 0; s < sets; ++s) {
    in[s] = s == 0 ? alloc_random(in_bytes / 2, dtype, 1.0f, 31) : alloc_copy_of(in[0]);
    if (ew && b_period > 0) in2[s] = s == 0 ? alloc_random((size_t)b_period, dtype, 1.0f, 32) : alloc_copy_of(in2[0]);
    out[s].bytes = out_bytes;
    HIP_OK(hipMalloc(&out[s].p, out_bytes));
  }
  const int warmup = env_int("AITAMD_PROF_WARMUP", 3);
  const int iters = env_int("AITAMD_PROF_ITERS", 10);
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  auto launch = [&](int s) {
    return ew ? aitamd_elementwise(func, dtype, in[s].p, b_period > 0 ? in2[s].p : nullptr, out[s].p, numel,
                                   b_period > 0 ? b_period : 1, 0.5f, 0, stream)
              : aitamd_copy_rows(in[s].p, out[s].p, rows, row_bytes, pitch, row_bytes, stream);
  };
  for (int i = 0; i < warmup; ++i) {
    if (launch(i % sets) != 0) {
      fprintf(stderr, "launch failed: %s\n", aitamd_last_error());
      return 3;
    }
  }
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipEventRecord(e0, stream));
  for (int i = 0; i < iters; ++i) launch(i % sets);
  HIP_OK(hipEventRecord(e1, stream));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  printf("OP:%s,TIME:%.6f,WS:0\n", ew ? "elementwise" : "copy_rows", ms / (iters > 0 ? iters : 1));
  HIP_OK(hipStreamDestroy(stream));
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 4) {
    fprintf(stderr, "usage: %s gemm|gemm_permute|gemm_layout|bmm|bmm_permute|bmm_layout|attn|ew|copy <op> <dtype> dims...\n", argv[0]);
    return 2;
  }
  const std::string kind = argv[1];
  const std::string op = argv[2];
  const int dtype = atoi(argv[3]);
  std::vector<int64_t> d;
  for (int i = 4; i < argc; ++i) d.push_back(atoll(argv[i]));
  if (kind == "gemm") {
    if (d.size() < 3) return 2;
    return profile_gemm_like(op, dtype, 1, d[0], d[1], d[2], false);
  }
  if (kind == "gemm_permute") {  // M N K g1 g2 g3
    if (d.size() < 6) return 2;
    std::string base;
    PermuteSpec perm;
    if (!permute_op(op, &base, &perm.layout)) {
      fprintf(stderr, "%s is not a permuting op\n", op.c_str());
      return 2;
    }
    perm.g[0] = d[3];
    perm.g[1] = d[4];
    perm.g[2] = d[5];
    if (op == "gemm_rrr_bias_permute") perm.operands = AITAMD_LAYOUT_RRR;
    return profile_gemm_like(base, dtype, 1, d[0], d[1], d[2], false, perm);
  }
  if (kind == "bmm") {
    if (d.size() < 4) return 2;
    return profile_gemm_like(op, dtype, d[0], d[1], d[2], d[3], true);
  }
  if (kind == "bmm_permute") {  // B M N K d1
    if (d.size() < 5) return 2;
    PermuteSpec perm;
    perm.layout = 1;
    perm.g[0] = d[4];
    return profile_gemm_like("bmm_rcr", dtype, d[0], d[1], d[2], d[3], true, perm);
  }
  if (kind == "bmm_layout" || kind == "gemm_layout") {  // bmm_rrr[_permute] | bmm_ccr | bmm_crr: B M N K [d1]; gemm_rrr: M N K
    const bool batched = kind == "bmm_layout";
    const size_t need = batched ? 4 : 3;
    const size_t lay_at = op.find('_');
    if (d.size() < need || lay_at == std::string::npos || op.size() < lay_at + 4) return 2;
    PermuteSpec perm;
    perm.operands = (op[lay_at + 1] == 'c' ? 2 : 0) | (op[lay_at + 2] == 'r' ? 1 : 0);
    if (op.size() > 8 && op.compare(op.size() - 8, 8, "_permute") == 0) {
      if (d.size() < need + 1) return 2;
      perm.layout = 1;
      perm.g[0] = d[need];
    }
    const bool add = op.size() > 4 && op.compare(op.size() - 4, 4, "_add") == 0;
    if (batched) return profile_gemm_like(add ? "bmm_add" : "bmm_rcr", dtype, d[0], d[1], d[2], d[3], true, perm);
    return profile_gemm_like("bmm_rcr", dtype, 1, d[0], d[1], d[2], true, perm);
  }
  if (kind == "ew") {
    if (d.size() < 1) return 2;
    return profile_streaming(kind, atoi(op.c_str()), dtype, d[0], d.size() > 1 ? d[1] : 0, 0);
  }
  if (kind == "copy") {
    if (d.size() < 3) return 2;
    return profile_streaming(kind, 0, dtype, d[0], d[1], d[2]);
  }
  if (kind == "attn") {
    if (d.size() < 6) return 2;
    return profile_attention(dtype, d[0], d[1], d[2], d[3], d[4], d[5], d.size() > 6 ? (int)d[6] : 0);
  }
  fprintf(stderr, "unknown kind %s\n", kind.c_str());
  return 2;
}
