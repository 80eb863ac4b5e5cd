/*
 * TEST INFRASTRUCTURE ONLY.  Plain-C CPU restatement of the arithmetic of the
 * AITemplate ROCm GEMM family.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load this; the product never does.
 *
 * What is restated, and where the reference defines it:
 *  - gemm_rcr*      Y[m,n] = epi( sum_k X[m,k] W[n,k] )   fp32 accumulate, fp16/bf16 out
 *                   python/aitemplate/compiler/ops/gemm_universal/gemm_rcr.py:26-50 (docstring
 *                   equivalent), gemm_rcr_bias.py:27-44, gemm_rcr_bias_relu.py:24-43,
 *                   gemm_rcr_bias_gelu.py:24-43, gemm_rcr_bias_add.py:26-47,
 *                   gemm_rcr_bias_add_add.py:26-48; functor order
 *                   python/aitemplate/backend/rocm/gemm/common.py:269-309,
 *                   gemm_rcr_bias_add.py:36-45, gemm_rcr_bias_add_add.py:36-44.
 *  - bmm_rcr        python/aitemplate/compiler/ops/gemm_universal/bmm_xxx.py:261-278.
 *  - bmm_softmax_bmm_permute
 *                   python/aitemplate/compiler/ops/gemm_universal/bmm_softmax_bmm_permute.py:30-194,
 *                   scale / strides python/aitemplate/backend/rocm/gemm/bmm_softmax_bmm_permute.py:47-51,84-110.
 *
 * The arithmetic itself lives in Composable Kernel (un-vendored submodule, no
 * pinned commit, absent from the reference checkout), so this file restates the
 * published definitions.  `ref_rounding` != 0 reproduces the reference's
 * rounding points (accumulator rounded to the output type before the functor,
 * functor adds in the output type, scale rounded to fp16); 0 evaluates the
 * epilogue in fp32 and rounds once.
 *
 * Pins (tests/test_oracle.py): brute-force Python loops on tiny inputs,
 * W = I, X = 0, torch's F.linear / F.gelu(approximate="tanh") / softmax as
 * library routines, softmax row-sum and constant-V invariants, one-hot
 * permutation check.  The reference holds no golden vectors for this path.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- 16-bit float formats <-> fp32 (round to nearest even) ----------------- */
static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while ((man & 0x400u) == 0);
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0));
  }
  if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x33000001u) { /* below half of the smallest subnormal */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t man = (ax & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t base;
  if (e < -14) { /* subnormal half */
    shift = 13 + (-14 - e);
    base = 0;
  } else {
    shift = 13;
    base = ((uint32_t)(e + 15) << 10) - 0x400u; /* implicit bit adds 0x400 back */
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1))) q++;
  return (uint16_t)(sign | (base + q));
}

static float bf16_to_float(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t float_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

static float load16(const uint16_t* p, int64_t i, int dtype) {
  return dtype == 0 ? half_to_float(p[i]) : bf16_to_float(p[i]);
}
static uint16_t store16(float v, int dtype) { return dtype == 0 ? float_to_half(v) : float_to_bf16(v); }
static float round16(float v, int dtype) { return load16((uint16_t[]){store16(v, dtype)}, 0, dtype); }

/* ---- epilogues -------------------------------------------------------------- */
static float gelu_tanh_f(float x) {
  /* 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) */
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.0f + tanhf(u));
}
static float sigmoid_ff(float x) { return 1.0f / (1.0f + expf(-x)); }
static float hardswish_ff(float x) {
  float r = x + 3.0f;
  if (r < 0.0f) r = 0.0f;
  if (r > 6.0f) r = 6.0f;
  return x * r / 6.0f;
}

/* ids as in include/aitemplate_amd_kernels.h */
static float apply_epilogue(int epi, float acc, float b, float d0, float d1, int dtype, int ref_rounding) {
  float x = acc;
  if (ref_rounding) x = round16(x, dtype);
  if (epi == 0) return x;
  x = x + b;
  if (ref_rounding) x = round16(x, dtype);
  switch (epi) {
    case 1: return x;
    case 2: return x > 0.0f ? x : 0.0f;
    case 3: return gelu_tanh_f(x);
    case 4: return x + d0;
    case 5: {
      float y = x + d0;
      if (ref_rounding) y = round16(y, dtype);
      return y + d1;
    }
    case 6: { float y = x + d0; return y > 0.0f ? y : 0.0f; }
    case 7: {
      float y = x + d0;
      if (ref_rounding) y = round16(y, dtype);
      y = y + d1;
      return y > 0.0f ? y : 0.0f;
    }
    case 8: return sigmoid_ff(x);
    case 9: return tanhf(x);
    case 10: return x * sigmoid_ff(x);
    case 11: return hardswish_ff(x);
    case 12: return x * d0;
    case 13: return x * d0 + d1;
    case 14: return sigmoid_ff(x) * d0;
    case 15: return tanhf(sigmoid_ff(x) * d0);
    case 16: return tanhf(x * d0);
    default: return NAN;
  }
}

/* C[b][m][n] = epi(sum_k A[b][m][k] B[b][n][k]); stride 0 broadcasts. Returns 0. */
int oracle_bmm_rcr_epilogue(int epi, int dtype, int ref_rounding, const uint16_t* a, const uint16_t* b,
                            const uint16_t* bias, const uint16_t* d0, const uint16_t* d1, uint16_t* c,
                            int64_t batch, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                            int64_t ldd, int64_t sa, int64_t sb, int64_t sc, int64_t sd) {
  if (epi < 0 || epi > 16) return 1;
  for (int64_t bi = 0; bi < batch; ++bi) {
    /* widen the operands of this batch once */
    float* af = (float*)malloc(sizeof(float) * (size_t)(M * K > 0 ? M * K : 1));
    float* bf = (float*)malloc(sizeof(float) * (size_t)(N * K > 0 ? N * K : 1));
    if (!af || !bf) { free(af); free(bf); return 2; }
    for (int64_t m = 0; m < M; ++m)
      for (int64_t k = 0; k < K; ++k) af[m * K + k] = load16(a, bi * sa + m * lda + k, dtype);
    for (int64_t n = 0; n < N; ++n)
      for (int64_t k = 0; k < K; ++k) bf[n * K + k] = load16(b, bi * sb + n * ldb + k, dtype);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
      for (int64_t n = 0; n < N; ++n) {
        float acc = 0.0f;
        const float* ar = af + m * K;
        const float* br = bf + n * K;
        for (int64_t k = 0; k < K; ++k) acc += ar[k] * br[k];
        const float bv = (epi != 0 && bias) ? load16(bias, n, dtype) : 0.0f;
        const float d0v = d0 ? load16(d0, bi * sd + m * ldd + n, dtype) : 0.0f;
        const float d1v = d1 ? load16(d1, bi * sd + m * ldd + n, dtype) : 0.0f;
        c[bi * sc + m * ldc + n] = store16(apply_epilogue(epi, acc, bv, d0v, d1v, dtype, ref_rounding), dtype);
      }
    }
    free(af);
    free(bf);
  }
  return 0;
}

int oracle_gemm_rcr(int epi, int dtype, int ref_rounding, const uint16_t* a, const uint16_t* b, const uint16_t* bias,
                    const uint16_t* d0, const uint16_t* d1, uint16_t* c, int64_t M, int64_t N, int64_t K) {
  return oracle_bmm_rcr_epilogue(epi, dtype, ref_rounding, a, b, bias, d0, d1, c, 1, M, N, K, K, K, N, N, 0, 0, 0, 0);
}

/*
 * out[b / G][m][b % G][o] = sum_n softmax_n( scale * sum_k Q[b][m][k] K[b][n][k] ) V[b][n][o]
 * Q [B,M,K], K [B,N,K], V [B,N,O], out [B/G, M, G, O]; causal masks n > m.
 * ref_rounding: scale rounded to fp16 first (the reference casts alpha to the
 * kernel's fp16 element type).
 */
int oracle_bmm_softmax_bmm_permute(int dtype, int ref_rounding, const uint16_t* q, const uint16_t* k,
                                   const uint16_t* v, uint16_t* out, int64_t B, int64_t M, int64_t N, int64_t K,
                                   int64_t O, int64_t G, float scale, int causal) {
  if (G <= 0 || B % G != 0) return 1;
  if (ref_rounding) scale = round16(scale, dtype);
  int rc = 0;
#pragma omp parallel for schedule(dynamic, 16) collapse(2)
  for (int64_t b = 0; b < B; ++b) {
    for (int64_t m = 0; m < M; ++m) {
      float* s = (float*)malloc(sizeof(float) * (size_t)(N > 0 ? N : 1));
      if (!s) { rc = 2; continue; }
      float mx = -INFINITY;
      const int64_t n_end = causal ? ((m + 1) < N ? (m + 1) : N) : N;
      for (int64_t n = 0; n < n_end; ++n) {
        float acc = 0.0f;
        for (int64_t kk = 0; kk < K; ++kk)
          acc += load16(q, (b * M + m) * K + kk, dtype) * load16(k, (b * N + n) * K + kk, dtype);
        acc *= scale;
        if (acc != acc) acc = -INFINITY; /* NaN -> -inf, as the reference's acc0 functor */
        s[n] = acc;
        if (acc > mx) mx = acc;
      }
      float sum = 0.0f;
      for (int64_t n = 0; n < n_end; ++n) {
        s[n] = expf(s[n] - mx);
        sum += s[n];
      }
      for (int64_t o = 0; o < O; ++o) {
        float acc = 0.0f;
        for (int64_t n = 0; n < n_end; ++n) acc += s[n] * load16(v, (b * N + n) * O + o, dtype);
        const int64_t idx = (((b / G) * M + m) * G + (b % G)) * O + o;
        out[idx] = store16(n_end > 0 ? acc / sum : 0.0f, dtype);
      }
      free(s);
    }
  }
  return rc;
}
