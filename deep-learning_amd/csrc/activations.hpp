// Device-side activation functions and the derivative forms the reference's
// backward pass uses (a function of the pre-activation x AND the stored output
// q).  Citations: /root/reference/lib/deep-learning/v1/ops/activations/functions.hpp.
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/dlmi.h"

namespace dlmi {

// functions.hpp:95-96, 108 — the reference's `_r` literals are floats in Release
constexpr float kSeluAlpha = 1.6732632423543772848170429916717f;
constexpr float kSeluScale = 1.0507009873554804934193349852946f;
constexpr float kLreluAlpha = 0.01f;

// exp(x) on the transcendental unit: v_exp_f32 computes 2^t to 1 ulp; the
// product x*log2(e) is formed in two pieces so that its rounding error (which
// would otherwise grow with |x|) is folded back in.  ~6 instructions instead of
// the ~40 of the branchy library routine, which made the fused normalization
// kernels VALU-bound instead of HBM-bound.  Max error ~2 ulp.
// Valid for x < 88.7 only: once 2^t overflows, the correction r*(e*ln 2) is
// +-inf and r + correction is NaN for about a third of the arguments.  The
// rectifier family calls it with x <= 0 (the positive side is discarded by a
// select, which does not propagate the NaN); anything that can see a large
// positive argument uses fast_exp_sat.
__device__ __forceinline__ float fast_exp(float x) {
  constexpr float kLog2eHi = 1.44269502162933349609375f;   // float(log2 e)
  constexpr float kLog2eLo = 1.925963033500011e-8f;        // log2 e - kLog2eHi
  constexpr float kLn2 = 0.693147182464599609375f;
  float const t = x * kLog2eHi;
  float const e = __builtin_fmaf(x, kLog2eHi, -t) + x * kLog2eLo;
  float const r = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(r, e * kLn2, r);
}
// The same, saturating to +inf like std::exp when the result overflows (the
// sigmoid and tanh take its reciprocal: 1/(1+inf) = 0, as in the reference).
__device__ __forceinline__ float fast_exp_sat(float x) {
  constexpr float kLog2eHi = 1.44269502162933349609375f;
  constexpr float kLog2eLo = 1.925963033500011e-8f;
  constexpr float kLn2 = 0.693147182464599609375f;
  float const t = x * kLog2eHi;
  float const e = __builtin_fmaf(x, kLog2eHi, -t) + x * kLog2eLo;
  float const r = __builtin_amdgcn_exp2f(t);
  return r == __builtin_inff() ? r : __builtin_fmaf(r, e * kLn2, r);
}
// 1/sqrt(v) and 1/v at hardware rate (1 ulp each).
__device__ __forceinline__ float fast_rsqrt(float v) { return __builtin_amdgcn_rsqf(v); }
__device__ __forceinline__ float fast_rcp(float v) { return __builtin_amdgcn_rcpf(v); }

template <int ACT>
__device__ __forceinline__ float act_fire(float x) {
  if constexpr (ACT == DLMI_ACT_ISRLU) {  // functions.hpp:86-87, slope 1
    return x < 0.0f ? x * fast_rsqrt(1.0f + x * x) : x;
  } else if constexpr (ACT == DLMI_ACT_ELU) {  // functions.hpp:91, slope 1: exp(x) - 1, not expm1
    return x < 0.0f ? (fast_exp(x) - 1.0f) : x;
  } else if constexpr (ACT == DLMI_ACT_SELU) {  // functions.hpp:97-98
    return kSeluScale * (x <= 0.0f ? kSeluAlpha * fast_exp(x) - kSeluAlpha : x);
  } else if constexpr (ACT == DLMI_ACT_RELU) {  // functions.hpp:102
    return x < 0.0f ? 0.0f : x;
  } else if constexpr (ACT == DLMI_ACT_LEAKY_RELU) {  // functions.hpp:106
    return x < 0.0f ? kLreluAlpha * x : x;
  } else if constexpr (ACT == DLMI_ACT_SIGMOID) {  // functions.hpp:40
    return fast_rcp(1.0f + fast_exp_sat(-x));
  } else if constexpr (ACT == DLMI_ACT_TANH) {  // functions.hpp:44
    return 2.0f * fast_rcp(1.0f + fast_exp_sat(-2.0f * x)) - 1.0f;
  } else {  // LINEAR
    return x;
  }
}

// functions.hpp:88 (ISRLU), :92 (ELU), :99 (SELU), :103 (ReLU), :107 (leaky), :41 (sigmoid), :45 (tanh)
template <int ACT>
__device__ __forceinline__ float act_derive(float x, float q) {
  if constexpr (ACT == DLMI_ACT_ISRLU) {
    float const t = q * fast_rcp(x);  // std::pow(q / x, 3)
    return x < 0.0f ? t * t * t : 1.0f;
  } else if constexpr (ACT == DLMI_ACT_ELU) {
    return x < 0.0f ? q : 1.0f;
  } else if constexpr (ACT == DLMI_ACT_SELU) {
    return kSeluScale * (x <= 0.0f ? (q + kSeluAlpha) : 1.0f);
  } else if constexpr (ACT == DLMI_ACT_RELU) {
    return x < 0.0f ? 0.0f : 1.0f;
  } else if constexpr (ACT == DLMI_ACT_LEAKY_RELU) {
    return x < 0.0f ? kLreluAlpha : 1.0f;
  } else if constexpr (ACT == DLMI_ACT_SIGMOID) {  // functions.hpp:41
    return q * (1.0f - q);
  } else if constexpr (ACT == DLMI_ACT_TANH) {  // functions.hpp:45
    return 1.0f - q * q;
  } else {
    return 1.0f;
  }
}

inline bool act_supported(int act) {
  switch (act) {
    case DLMI_ACT_ISRLU:
    case DLMI_ACT_ELU:
    case DLMI_ACT_SELU:
    case DLMI_ACT_RELU:
    case DLMI_ACT_LEAKY_RELU:
    case DLMI_ACT_LINEAR:
    case DLMI_ACT_SIGMOID:
    case DLMI_ACT_TANH:
      return true;
    default:
      return false;
  }
}

// Calls f.template operator()<ACT>() for the runtime activation code.
#define DLMI_DISPATCH_ACT(act, ...)                                        \
  switch (act) {                                                           \
    case DLMI_ACT_ISRLU: { constexpr int ACT = DLMI_ACT_ISRLU; __VA_ARGS__; } break;           \
    case DLMI_ACT_ELU: { constexpr int ACT = DLMI_ACT_ELU; __VA_ARGS__; } break;               \
    case DLMI_ACT_SELU: { constexpr int ACT = DLMI_ACT_SELU; __VA_ARGS__; } break;             \
    case DLMI_ACT_RELU: { constexpr int ACT = DLMI_ACT_RELU; __VA_ARGS__; } break;             \
    case DLMI_ACT_LEAKY_RELU: { constexpr int ACT = DLMI_ACT_LEAKY_RELU; __VA_ARGS__; } break; \
    case DLMI_ACT_SIGMOID: { constexpr int ACT = DLMI_ACT_SIGMOID; __VA_ARGS__; } break;       \
    case DLMI_ACT_TANH: { constexpr int ACT = DLMI_ACT_TANH; __VA_ARGS__; } break;             \
    default: { constexpr int ACT = DLMI_ACT_LINEAR; __VA_ARGS__; } break;                      \
  }

}  // namespace dlmi
