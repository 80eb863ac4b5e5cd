// Register-level epilogues of the GEMM family.  Every functor sees the fp32
// accumulator plus (optionally) the bias element of its column and up to two
// residual elements of its (row, column), and returns the fp32 value that is
// rounded once to the output type.
//
// Formulas follow the element-wise functors the reference selects per op
// (python/aitemplate/backend/rocm/gemm/common.py:269-309 and the inline
// AddAdd / AddAddAdd functors in backend/rocm/gemm/gemm_rcr_bias_add.py:28-51,
// gemm_rcr_bias_add_add.py:28-52).  The reference rounds the accumulator to
// fp16 before the functor and adds in fp16; here the whole epilogue runs in
// fp32, which differs from it by at most a few fp16 ulps.
#pragma once

#include "common.hpp"

namespace aitamd {

// Stable ids: they are part of the C ABI (aitamd_gemm's `epilogue` argument).
enum EpilogueId : int {
  kEpiNone = 0,             // gemm_rcr, bmm_rcr
  kEpiBias = 1,             // gemm_rcr_bias
  kEpiBiasRelu = 2,         // gemm_rcr_bias_relu
  kEpiBiasGelu = 3,         // gemm_rcr_bias_gelu == gemm_rcr_bias_fast_gelu
  kEpiBiasAdd = 4,          // gemm_rcr_bias_add
  kEpiBiasAddAdd = 5,       // gemm_rcr_bias_add_add
  kEpiBiasAddRelu = 6,      // gemm_rcr_bias_add_relu
  kEpiBiasAddAddRelu = 7,   // gemm_rcr_bias_add_add_relu
  kEpiBiasSigmoid = 8,      // gemm_rcr_bias_sigmoid
  kEpiBiasTanh = 9,         // gemm_rcr_bias_tanh
  kEpiBiasSwish = 10,       // gemm_rcr_bias_swish
  kEpiBiasHardswish = 11,   // gemm_rcr_bias_hardswish
  kEpiBiasMul = 12,         // gemm_rcr_bias_mul
  kEpiBiasMulAdd = 13,      // gemm_rcr_bias_mul_add
  kEpiBiasSigmoidMul = 14,  // gemm_rcr_bias_sigmoid_mul
  kEpiBiasSigmoidMulTanh = 15,  // gemm_rcr_bias_sigmoid_mul_tanh
  kEpiBiasMulTanh = 16,     // gemm_rcr_bias_mul_tanh
  kEpiAdd = 17,             // bmm_rrr_add, bmm_ccr_add, bmm_crr_add: residual without bias
  kNumEpilogues = 18,
};

AITAMD_DEVICE float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// tanh-form GELU rewritten as x * sigmoid(2u), u = x*(0.797885 + 0.035677 x^2):
// 0.5 x (1 + tanh u) == x / (1 + exp(-2u)).  One v_exp + one v_rcp per element; the factor -2 log2(e) of
// the exponent is folded into the polynomial's coefficients (one multiply less per element).
AITAMD_DEVICE float gelu_tanh(float x) {
  constexpr float kScale = -2.0f * 1.4426950408889634f;
  constexpr float kC1 = kScale * 0.035677f, kC0 = kScale * 0.797885f;
  const float e = __builtin_amdgcn_exp2f(x * (kC1 * (x * x) + kC0));
  return x * fast_rcp(1.0f + e);
}

AITAMD_DEVICE float sigmoid_f(float x) {
  constexpr float kLog2e = 1.4426950408889634f;
  return fast_rcp(1.0f + __builtin_amdgcn_exp2f(-kLog2e * x));
}

AITAMD_DEVICE float tanh_f(float x) {
  // tanh x = 2 sigmoid(2x) - 1; saturates cleanly because exp2 -> 0 or inf.
  return 2.0f * sigmoid_f(2.0f * x) - 1.0f;
}

AITAMD_DEVICE float hardswish_f(float x) {
  float r = x + 3.0f;
  r = r < 0.0f ? 0.0f : (r > 6.0f ? 6.0f : r);
  return x * r * (1.0f / 6.0f);
}

template <int kId>
struct Epilogue;

// LEAD: how many of the residuals the expression adds, in order, right behind acc (+ b).  A caller may fold those
// adds into its conversion of the residuals (v_fma_mix: half -> float and add in one instruction, the same single
// rounding) and pass -0.0, which adds nothing, in their place.
#define AITAMD_DEF_EPI(ID, BIAS, ND, LEAD, EXPR)                                   \
  template <>                                                                  \
  struct Epilogue<ID> {                                                        \
    static constexpr int kId = ID;                                             \
    static constexpr bool kHasBias = BIAS;                                     \
    static constexpr int kNumD = ND;                                           \
    static constexpr int kLeadingAdds = LEAD;                                  \
    static AITAMD_DEVICE float apply(float acc, float b, float d0, float d1) { \
      (void)b; (void)d0; (void)d1;                                             \
      return EXPR;                                                             \
    }                                                                          \
  };

AITAMD_DEF_EPI(kEpiNone, false, 0, 0, acc)
AITAMD_DEF_EPI(kEpiBias, true, 0, 0, acc + b)
AITAMD_DEF_EPI(kEpiBiasRelu, true, 0, 0, fmaxf(acc + b, 0.0f))
AITAMD_DEF_EPI(kEpiBiasGelu, true, 0, 0, gelu_tanh(acc + b))
AITAMD_DEF_EPI(kEpiBiasAdd, true, 1, 1, (acc + b) + d0)
AITAMD_DEF_EPI(kEpiBiasAddAdd, true, 2, 2, ((acc + b) + d0) + d1)
AITAMD_DEF_EPI(kEpiBiasAddRelu, true, 1, 1, fmaxf((acc + b) + d0, 0.0f))
AITAMD_DEF_EPI(kEpiBiasAddAddRelu, true, 2, 2, fmaxf(((acc + b) + d0) + d1, 0.0f))
AITAMD_DEF_EPI(kEpiBiasSigmoid, true, 0, 0, sigmoid_f(acc + b))
AITAMD_DEF_EPI(kEpiBiasTanh, true, 0, 0, tanh_f(acc + b))
AITAMD_DEF_EPI(kEpiBiasSwish, true, 0, 0, (acc + b) * sigmoid_f(acc + b))
AITAMD_DEF_EPI(kEpiBiasHardswish, true, 0, 0, hardswish_f(acc + b))
AITAMD_DEF_EPI(kEpiBiasMul, true, 1, 0, (acc + b) * d0)
AITAMD_DEF_EPI(kEpiBiasMulAdd, true, 2, 0, (acc + b) * d0 + d1)
AITAMD_DEF_EPI(kEpiBiasSigmoidMul, true, 1, 0, sigmoid_f(acc + b) * d0)
AITAMD_DEF_EPI(kEpiBiasSigmoidMulTanh, true, 1, 0, tanh_f(sigmoid_f(acc + b) * d0))
AITAMD_DEF_EPI(kEpiBiasMulTanh, true, 1, 0, tanh_f((acc + b) * d0))
AITAMD_DEF_EPI(kEpiAdd, false, 1, 1, acc + d0)

#undef AITAMD_DEF_EPI

// Epi applied to xb = acc (+ bias, already added) and the residuals as stored, with the residual adds that lead
// the expression folded into the residuals' conversion (see LEAD above).
template <class Epi, class T>
AITAMD_DEVICE float apply_folded(float xb, T d0, T d1, float one) {
  using Tr = ElemTraits<T>;
  if constexpr (Epi::kLeadingAdds >= 1) xb = Tr::to_float_plus(d0, one, xb);
  if constexpr (Epi::kLeadingAdds >= 2) xb = Tr::to_float_plus(d1, one, xb);
  const float f0 = Epi::kLeadingAdds >= 1 ? -0.0f : (Epi::kNumD >= 1 ? Tr::to_float(d0) : 0.0f);
  const float f1 = Epi::kLeadingAdds >= 2 ? -0.0f : (Epi::kNumD >= 2 ? Tr::to_float(d1) : 0.0f);
  return Epi::apply(xb, -0.0f, f0, f1);
}

}  // namespace aitamd
