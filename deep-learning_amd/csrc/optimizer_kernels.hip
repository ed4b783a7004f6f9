// Optimizer steps over the packed parameter array for gfx950: plain gradient
// descent, momentum, the reference's Nesterov variant, Adam, AMSGrad, AdaBound and AMSBound, each
// with the optional masked weight decay, and iRPROP+; each zeroing the gradient it consumed.
//
// One pass, one thread per 4 parameters (float4), every array read once and
// written once: bound by HBM bandwidth (Adam: 32 bytes per parameter).  The
// arithmetic keeps the reference's expression order, with IEEE division and
// square root, so a trajectory of many steps stays on the reference's.
//
// Citations: /root/reference/lib/deep-learning/v1/optimizers/.
#include <initializer_list>

#include "dlmi_common.hpp"

namespace dlmi {

constexpr int kOptBlock = 256;
constexpr int kOptGd = 0, kOptMomentum = 1, kOptNesterov = 2, kOptAdam = 3, kOptAmsgrad = 4, kOptAdabound = 5,
              kOptAmsbound = 6, kOptIrpropPlus = 7;

struct OptArgs {
  float *p, *g;
  float *s0;          // momentum: previous delta; Adam: first moment
  float *s1;          // Adam: second moment
  float *s2;          // AMSGrad: running maximum of the second moment
  float const *mask;  // regularization mask, read only when WD
  size_t n;
  float lr;           // GD family: learning rate; Adam family: bias-corrected step size
  float mom, beta1, beta2, eps, wd;
  float rate_lo, rate_hi;  // AdaBound / AMSBound: the band the per-parameter step size is clipped into
  // iRPROP+: s0 previous gradient, s1 previous parameter move, s2 step size; factors and limits of the
  // step size; whether the loss got worse since the previous call
  float incr, decr, step_min, step_max;
  int loss_got_worse;
};

// One parameter.  gradient_descent.cpp:79-92, gradient_descent_momentum.cpp:44-63,
// nesterov_accelerated_gradient.cpp:44-63, adam.cpp:65-97, amsgrad.cpp:75-117, adabound.cpp:72-112,
// amsbound.cpp:80-124.
template <int KIND, bool WD>
__device__ __forceinline__ void opt_one(OptArgs const &a, float &p, float g, float &s0, float &s1, float &s2,
                                        float mask) {
  if constexpr (KIND == kOptIrpropPlus) {
    // irprop_plus.cpp:53-77: the step size of a parameter grows while its gradient keeps its sign and
    // shrinks when the sign flips; after a flip the last move is taken back if the loss got worse, and
    // the stored gradient is cleared so that the next call takes the plain-step branch.  Only signs and
    // one product per branch: bit-identical to the reference.
    float const prod = s0 * g;
    float const sgn = static_cast<float>((0.0f < g) - (g < 0.0f));  // ops/math.hpp:67-70
    if (prod > 0.0f) {
      float dt = s2 * a.incr;
      dt = a.step_max < dt ? a.step_max : dt;
      s2 = dt;
      s1 = -sgn * dt;
      p += s1;
      s0 = g;
    } else if (prod < 0.0f) {
      float const dt = s2 * a.decr;
      s2 = dt < a.step_min ? a.step_min : dt;
      if (a.loss_got_worse) p -= s1;
      s0 = 0.0f;
    } else {
      s1 = -sgn * s2;
      p += s1;
      s0 = g;
    }
    return;
  }
  float step;
  if constexpr (KIND == kOptGd) {
    step = a.lr * g;
  } else if constexpr (KIND == kOptMomentum) {
    s0 = a.lr * g + a.mom * s0;
    step = s0;
  } else if constexpr (KIND == kOptNesterov) {
    s0 = a.lr * g + a.mom * s0;
    step = a.mom * s0 - a.lr * g;  // the reference's sign
  } else {
    s0 = a.beta1 * s0 + (1.0f - a.beta1) * g;
    s1 = a.beta2 * s1 + (1.0f - a.beta2) * g * g;
    float v = s1;
    if constexpr (KIND == kOptAmsgrad || KIND == kOptAmsbound) {
      v = s2 > v ? s2 : v;
      s2 = v;
    }
    if constexpr (KIND == kOptAdabound || KIND == kOptAmsbound) {
      // the per-parameter step size, clipped into the band that closes on the final
      // learning rate (adabound.cpp:83-87, amsbound.cpp:94-99)
      float rate = a.lr / (sqrtf(v) + a.eps);
      rate = rate < a.rate_lo ? a.rate_lo : (rate > a.rate_hi ? a.rate_hi : rate);
      step = rate * s0;
    } else {
      step = a.lr * s0 / (sqrtf(v) + a.eps);
    }
  }
  if constexpr (WD) step += mask * a.wd * p;
  p -= step;
}

template <int KIND, bool WD>
__global__ __launch_bounds__(kOptBlock) void k_opt(OptArgs a, size_t n4) {
  constexpr bool kS0 = KIND != kOptGd, kS1 = KIND >= kOptAdam, kS2 = KIND == kOptAmsgrad || KIND == kOptAmsbound || KIND == kOptIrpropPlus;
  size_t const stride = static_cast<size_t>(gridDim.x) * kOptBlock;
  size_t i = static_cast<size_t>(blockIdx.x) * kOptBlock + threadIdx.x;
  for (; i < n4; i += stride) {
    float4 p = reinterpret_cast<float4 *>(a.p)[i];
    float4 const g = reinterpret_cast<float4 const *>(a.g)[i];
    float4 s0 = make_float4(0, 0, 0, 0), s1 = s0, s2 = s0, mk = s0;
    if constexpr (kS0) s0 = reinterpret_cast<float4 *>(a.s0)[i];
    if constexpr (kS1) s1 = reinterpret_cast<float4 *>(a.s1)[i];
    if constexpr (kS2) s2 = reinterpret_cast<float4 *>(a.s2)[i];
    if constexpr (WD) mk = reinterpret_cast<float4 const *>(a.mask)[i];
    opt_one<KIND, WD>(a, p.x, g.x, s0.x, s1.x, s2.x, mk.x);
    opt_one<KIND, WD>(a, p.y, g.y, s0.y, s1.y, s2.y, mk.y);
    opt_one<KIND, WD>(a, p.z, g.z, s0.z, s1.z, s2.z, mk.z);
    opt_one<KIND, WD>(a, p.w, g.w, s0.w, s1.w, s2.w, mk.w);
    reinterpret_cast<float4 *>(a.p)[i] = p;
    reinterpret_cast<float4 *>(a.g)[i] = make_float4(0, 0, 0, 0);
    if constexpr (kS0) reinterpret_cast<float4 *>(a.s0)[i] = s0;
    if constexpr (kS1) reinterpret_cast<float4 *>(a.s1)[i] = s1;
    if constexpr (kS2) reinterpret_cast<float4 *>(a.s2)[i] = s2;
  }
  for (i = n4 * 4 + static_cast<size_t>(blockIdx.x) * kOptBlock + threadIdx.x; i < a.n; i += stride) {
    float p = a.p[i], s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, mk = 0.0f;
    if constexpr (kS0) s0 = a.s0[i];
    if constexpr (kS1) s1 = a.s1[i];
    if constexpr (kS2) s2 = a.s2[i];
    if constexpr (WD) mk = a.mask[i];
    opt_one<KIND, WD>(a, p, a.g[i], s0, s1, s2, mk);
    a.p[i] = p;
    a.g[i] = 0.0f;
    if constexpr (kS0) a.s0[i] = s0;
    if constexpr (kS1) a.s1[i] = s1;
    if constexpr (kS2) a.s2[i] = s2;
  }
}

template <int KIND>
static int launch_opt(dlmi_ctx *ctx, OptArgs const &a, char const *what) {
  if (a.n == 0) return DLMI_OK;
  bool aligned = true;
  for (void const *q : {static_cast<void const *>(a.p), static_cast<void const *>(a.g),
                        static_cast<void const *>(a.s0), static_cast<void const *>(a.s1),
                        static_cast<void const *>(a.s2), static_cast<void const *>(a.mask)})
    if (q != nullptr && !dlmi_aligned16(q)) aligned = false;
  size_t const n4 = aligned ? a.n / 4 : 0;
  size_t blocks = dlmi_ceil_div(n4 ? n4 : a.n, kOptBlock);
  size_t const cap = static_cast<size_t>(ctx->num_cu) * 16;
  if (blocks > cap) blocks = cap;
  if (a.wd != 0.0f)
    hipLaunchKernelGGL((k_opt<KIND, true>), dim3(static_cast<unsigned>(blocks)), dim3(kOptBlock), 0, ctx->stream, a,
                       n4);
  else
    hipLaunchKernelGGL((k_opt<KIND, false>), dim3(static_cast<unsigned>(blocks)), dim3(kOptBlock), 0, ctx->stream, a,
                       n4);
  DLMI_LAUNCH_CHECK(ctx, what);
  return DLMI_OK;
}

}  // namespace dlmi

using namespace dlmi;

extern "C" {

int dlmi_opt_gd(dlmi_ctx *ctx, size_t n, float *params, float *grads, float const *mask, float lr, float wd) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, n == 0 || (params && grads), "null pointer");
  DLMI_REQUIRE(ctx, wd == 0.0f || mask != nullptr, "weight decay needs the regularization mask");
  OptArgs a{};
  a.p = params; a.g = grads; a.mask = mask; a.n = n; a.lr = lr; a.wd = wd;
  return launch_opt<kOptGd>(ctx, a, "k_opt<gd>");
}

int dlmi_opt_gd_momentum(dlmi_ctx *ctx, size_t n, float *params, float *grads, float *delta_prev, float const *mask,
                         float lr, float momentum, float wd, int nesterov) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, n == 0 || (params && grads && delta_prev), "null pointer");
  DLMI_REQUIRE(ctx, wd == 0.0f || mask != nullptr, "weight decay needs the regularization mask");
  OptArgs a{};
  a.p = params; a.g = grads; a.s0 = delta_prev; a.mask = mask; a.n = n; a.lr = lr; a.mom = momentum; a.wd = wd;
  return nesterov ? launch_opt<kOptNesterov>(ctx, a, "k_opt<nesterov>")
                  : launch_opt<kOptMomentum>(ctx, a, "k_opt<momentum>");
}

int dlmi_opt_adam(dlmi_ctx *ctx, size_t n, float *params, float *grads, float *m1, float *m2, float *m2_hat,
                  float const *mask, float lr_t, float beta1, float beta2, float eps, float wd) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, n == 0 || (params && grads && m1 && m2), "null pointer");
  DLMI_REQUIRE(ctx, wd == 0.0f || mask != nullptr, "weight decay needs the regularization mask");
  OptArgs a{};
  a.p = params; a.g = grads; a.s0 = m1; a.s1 = m2; a.s2 = m2_hat; a.mask = mask; a.n = n;
  a.lr = lr_t; a.beta1 = beta1; a.beta2 = beta2; a.eps = eps; a.wd = wd;
  return m2_hat != nullptr ? launch_opt<kOptAmsgrad>(ctx, a, "k_opt<amsgrad>")
                           : launch_opt<kOptAdam>(ctx, a, "k_opt<adam>");
}

int dlmi_opt_irprop_plus(dlmi_ctx *ctx, size_t n, float *params, float *grads, float *prev_grads, float *prev_moves,
                         float *step_sizes, float increase, float decrease, float step_min, float step_max,
                         int loss_got_worse) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, n == 0 || (params && grads && prev_grads && prev_moves && step_sizes), "null pointer");
  OptArgs a{};
  a.p = params; a.g = grads; a.s0 = prev_grads; a.s1 = prev_moves; a.s2 = step_sizes; a.n = n;
  a.incr = increase; a.decr = decrease; a.step_min = step_min; a.step_max = step_max;
  a.loss_got_worse = loss_got_worse != 0 ? 1 : 0;
  return launch_opt<kOptIrpropPlus>(ctx, a, "k_opt<irprop+>");
}

int dlmi_opt_adabound(dlmi_ctx *ctx, size_t n, float *params, float *grads, float *m1, float *m2, float *m2_hat,
                      float const *mask, float lr_t, float beta1, float beta2, float eps, float wd, float rate_lower,
                      float rate_upper) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, n == 0 || (params && grads && m1 && m2), "null pointer");
  DLMI_REQUIRE(ctx, wd == 0.0f || mask != nullptr, "weight decay needs the regularization mask");
  DLMI_REQUIRE(ctx, rate_lower <= rate_upper, "the lower bound of the step size exceeds the upper one");
  OptArgs a{};
  a.p = params; a.g = grads; a.s0 = m1; a.s1 = m2; a.s2 = m2_hat; a.mask = mask; a.n = n;
  a.lr = lr_t; a.beta1 = beta1; a.beta2 = beta2; a.eps = eps; a.wd = wd; a.rate_lo = rate_lower; a.rate_hi = rate_upper;
  return m2_hat != nullptr ? launch_opt<kOptAmsbound>(ctx, a, "k_opt<amsbound>")
                           : launch_opt<kOptAdabound>(ctx, a, "k_opt<adabound>");
}

}  // extern "C"
