// Element-wise leaves of the fully-connected path for gfx950: bias add,
// activation forward / derivative, dropout, identity add, inference-mode
// normalization (optionally fused with the activation), row softmax and the
// softmax + cross-entropy seed gradient.  One coalesced pass each; float4
// accesses whenever the row length and the pointers allow it.
//
// Citations: /root/reference/lib/deep-learning/v1/learner/.
#include <initializer_list>

#include "activations.hpp"
#include "block_pairs.hpp"
#include "dlmi_common.hpp"
#include "softmax_ce_row.hpp"

namespace dlmi {

constexpr int kEwBlock = 256;

static unsigned ew_grid(dlmi_ctx const *ctx, size_t work_items) {
  size_t const blocks = dlmi_ceil_div(work_items, kEwBlock);
  size_t const cap = static_cast<size_t>(ctx->num_cu) * 16;
  return static_cast<unsigned>(blocks < cap ? (blocks ? blocks : 1) : cap);
}

static bool all_aligned16(std::initializer_list<void const *> ptrs) {
  for (void const *p : ptrs)
    if (p != nullptr && !dlmi_aligned16(p)) return false;
  return true;
}

// ---- activation forward / backward (fwp_st.cpp:4768-4794, bwp_st.cpp:1177-1209)
template <int ACT>
__global__ __launch_bounds__(kEwBlock) void k_act_fwd(float const *__restrict__ x, float *__restrict__ y, size_t n4,
                                                       size_t n) {
  size_t const stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  size_t i = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x;
  for (; i < n4; i += stride) {
    float4 v = reinterpret_cast<float4 const *>(x)[i];
    v.x = act_fire<ACT>(v.x); v.y = act_fire<ACT>(v.y); v.z = act_fire<ACT>(v.z); v.w = act_fire<ACT>(v.w);
    reinterpret_cast<float4 *>(y)[i] = v;
  }
  for (i = n4 * 4 + static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < n; i += stride)
    y[i] = act_fire<ACT>(x[i]);
}

template <int ACT>
__global__ __launch_bounds__(kEwBlock) void k_act_bwd(float const *__restrict__ pre, float const *__restrict__ post,
                                                       float const *__restrict__ dY, float *__restrict__ dN,
                                                       size_t n4, size_t n) {
  size_t const stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  size_t i = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x;
  for (; i < n4; i += stride) {
    float4 const a = reinterpret_cast<float4 const *>(pre)[i];
    float4 const q = reinterpret_cast<float4 const *>(post)[i];
    float4 g = reinterpret_cast<float4 const *>(dY)[i];
    g.x *= act_derive<ACT>(a.x, q.x); g.y *= act_derive<ACT>(a.y, q.y);
    g.z *= act_derive<ACT>(a.z, q.z); g.w *= act_derive<ACT>(a.w, q.w);
    reinterpret_cast<float4 *>(dN)[i] = g;
  }
  for (i = n4 * 4 + static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < n; i += stride)
    dN[i] = dY[i] * act_derive<ACT>(pre[i], post[i]);
}

// ---- the same with one activation type per unit (fwp_st.cpp:4768-4794 takes an array of types, one per
// unit of the layer; a layer read from a .net file may mix them, load.cpp:4121).  Lanes of a wavefront sit on
// different units, so the switch diverges where neighbouring units differ; every unit still runs the code of
// the single-type kernels.
__device__ __forceinline__ float act_fire_of(int act, float x) {
  DLMI_DISPATCH_ACT(act, return act_fire<ACT>(x));
  return x;
}
__device__ __forceinline__ float act_derive_of(int act, float x, float q) {
  DLMI_DISPATCH_ACT(act, return act_derive<ACT>(x, q));
  return 1.0f;
}
__global__ __launch_bounds__(kEwBlock) void k_act_units_fwd(int const *__restrict__ types, float const *__restrict__ x,
                                                             float *__restrict__ y, size_t H, size_t n) {
  size_t const stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < n; i += stride)
    y[i] = act_fire_of(types[i % H], x[i]);
}
__global__ __launch_bounds__(kEwBlock) void k_act_units_bwd(int const *__restrict__ types, float const *__restrict__ pre,
                                                             float const *__restrict__ post, float const *__restrict__ dY,
                                                             float *__restrict__ dN, size_t H, size_t n) {
  size_t const stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < n; i += stride)
    dN[i] = dY[i] * act_derive_of(types[i % H], pre[i], post[i]);
}

// ---- out = a + b (fwp_st.cpp:5051-5112 with equal widths)
__global__ __launch_bounds__(kEwBlock) void k_add(float const *__restrict__ a, float const *__restrict__ b,
                                                   float *__restrict__ out, size_t n4, size_t n) {
  size_t const stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  size_t i = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x;
  for (; i < n4; i += stride) {
    float4 const u = reinterpret_cast<float4 const *>(a)[i];
    float4 const v = reinterpret_cast<float4 const *>(b)[i];
    reinterpret_cast<float4 *>(out)[i] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
  }
  for (i = n4 * 4 + static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < n; i += stride) out[i] = a[i] + b[i];
}

// ---- zero-padded identity shortcut (fwp_st.cpp:5051-5112, padding != 0):
// out [B, Hw] = wide [B, Hw], plus narrow [B, Hn] at column offset `pad`
__global__ __launch_bounds__(kEwBlock) void k_padded_add(float const *__restrict__ wide,
                                                          float const *__restrict__ narrow, float *__restrict__ out,
                                                          size_t B, size_t Hw, size_t Hn, size_t pad) {
  size_t const n = B * Hw, stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  for (size_t e = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; e < n; e += stride) {
    size_t const b = e / Hw, j = e - b * Hw;
    float v = wide[e];
    if (j >= pad && j - pad < Hn) v += narrow[b * Hn + (j - pad)];
    out[e] = v;
  }
}

// ---- shortcut gradient routing (bwp_st.cpp:1112-1175): over the Hc = min(Hi, Hd)
// shared columns, dd[b, j + od] += di[b, j + oi]
__global__ __launch_bounds__(kEwBlock) void k_residual_bwd(float const *__restrict__ di, float *__restrict__ dd,
                                                            size_t B, size_t Hi, size_t Hd, size_t Hc, size_t oi,
                                                            size_t od) {
  size_t const n = B * Hc, stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  for (size_t e = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; e < n; e += stride) {
    size_t const b = e / Hc, j = e - b * Hc;
    dd[b * Hd + j + od] += di[b * Hi + j + oi];
  }
}

// ---- clearing a buffer with a kernel (the reference's memset of the error arrays,
// bwp_st.cpp:115): unlike a memset node, this can be recorded into a HIP graph
__global__ __launch_bounds__(kEwBlock) void k_zero(float *__restrict__ p, size_t n) {
  size_t const stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  for (size_t e = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; e < n; e += stride) p[e] = 0.0f;
}

// ---- per-unit row kernels: element e = b*H + j, unit j = e % H ----------------
// mode 0: Z += bias                                     (fwp_st.cpp:4498-4516)
// mode 1: dropout, kind/per_element/scale in the args   (fwp_st.cpp:4830-4904)
// mode 2: y = f(gamma*((x-mov_mean)/mov_std)+beta) [* keep]  (fwp_st.cpp:4557-4584)
struct RowArgs {
  float const *x;
  float *y;
  float const *p0, *p1, *p2, *p3;  // per-unit vectors
  uint8_t const *mask;
  size_t B, H;
  int drop_kind, per_element;
  float scale;
};

template <int MODE, int ACT>
__device__ __forceinline__ float row_op(RowArgs const &a, float v, size_t e, size_t j) {
  if constexpr (MODE == 0) {
    return v + a.p0[j];
  } else if constexpr (MODE == 1) {
    if (a.drop_kind == 3) return v * a.scale;  // inference rescale
    uint8_t const m = a.per_element ? a.mask[e] : a.mask[j];
    return a.drop_kind == 1 ? (m ? v : 0.0f) : (m ? v * a.scale : 0.0f);
  } else {
    float const nn = a.p0[j] * ((v - a.p2[j]) / a.p3[j]) + a.p1[j];
    return act_fire<ACT>(nn) * a.scale;
  }
}

template <int MODE, int ACT, int VEC>
__global__ __launch_bounds__(kEwBlock) void k_row(RowArgs a) {
  size_t const n = a.B * a.H;
  size_t const stride = static_cast<size_t>(gridDim.x) * kEwBlock * VEC;
  for (size_t e = (static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x) * VEC; e < n; e += stride) {
    size_t const j = e % a.H;
    if constexpr (VEC == 4) {
      float4 v = *reinterpret_cast<float4 const *>(a.x + e);
      v.x = row_op<MODE, ACT>(a, v.x, e, j);
      v.y = row_op<MODE, ACT>(a, v.y, e + 1, j + 1);
      v.z = row_op<MODE, ACT>(a, v.z, e + 2, j + 2);
      v.w = row_op<MODE, ACT>(a, v.w, e + 3, j + 3);
      *reinterpret_cast<float4 *>(a.y + e) = v;
    } else {
      a.y[e] = row_op<MODE, ACT>(a, a.x[e], e, j);
    }
  }
}

template <int MODE, int ACT>
static int launch_row(dlmi_ctx *ctx, RowArgs const &a, char const *what) {
  bool const vec4 = a.H % 4 == 0 && all_aligned16({a.x, a.y});
  size_t const n = a.B * a.H;
  if (vec4)
    hipLaunchKernelGGL((k_row<MODE, ACT, 4>), dim3(ew_grid(ctx, n / 4)), dim3(kEwBlock), 0, ctx->stream, a);
  else
    hipLaunchKernelGGL((k_row<MODE, ACT, 1>), dim3(ew_grid(ctx, n)), dim3(kEwBlock), 0, ctx->stream, a);
  DLMI_LAUNCH_CHECK(ctx, what);
  return DLMI_OK;
}

// ---- softmax: one wavefront per row (fwp_st.cpp:4796-4828) -------------------
__global__ __launch_bounds__(kEwBlock) void k_softmax(float const *__restrict__ x, float *__restrict__ y, size_t B,
                                                       size_t H) {
  int const lane = threadIdx.x & 63;
  size_t const row = static_cast<size_t>(blockIdx.x) * (kEwBlock / 64) + threadIdx.x / 64;
  if (row >= B) return;
  float const *xi = x + row * H;
  float *yi = y + row * H;
  float mx = -3.402823466e+38f;
  for (size_t i = lane; i < H; i += 64) mx = fmaxf(mx, xi[i]);
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  float s = 0.0f;
  for (size_t i = lane; i < H; i += 64) {
    float const e = expf(xi[i] - mx);
    yi[i] = e;
    s += e;
  }
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  s = 1.0f / s;
  for (size_t i = lane; i < H; i += 64) yi[i] *= s;
}

// ---- softmax + cross-entropy seed gradient (compute_error_st.cpp:26-131,
// compute_loss.cpp:88-95, 101-138).  One wavefront per row; the double
// accumulators go out as one pair per block, added in a fixed order by the
// block that finishes last (block_pairs.hpp).
__global__ __launch_bounds__(kEwBlock) void k_softmax_ce_seed(float const *__restrict__ q, float const *__restrict__ y,
                                                               float *__restrict__ dZ, size_t B, size_t H,
                                                               double *__restrict__ pairs, double *__restrict__ acc,
                                                               unsigned *__restrict__ ticket) {
  int const lane = threadIdx.x & 63;
  size_t const row = static_cast<size_t>(blockIdx.x) * (kEwBlock / 64) + threadIdx.x / 64;
  double loss = 0.0, correct = 0.0;
  if (row < B) softmax_ce_seed_row(q + row * H, y + row * H, dZ + row * H, H, B, lane, loss, correct);
  if (acc != nullptr) {
    __shared__ double sh[2][kEwBlock / 64];
    if (lane == 0) {
      sh[0][threadIdx.x / 64] = loss;
      sh[1][threadIdx.x / 64] = correct;
    }
    __syncthreads();
    double l = 0.0, c = 0.0;
    if (threadIdx.x == 0)
      for (int w = 0; w < kEwBlock / 64; ++w) { l += sh[0][w]; c += sh[1][w]; }
    finish_block_pairs(l, c, pairs, acc, ticket);
  }
}

// ---- variance over a whole buffer (get_layer_variance, model.cpp:2824-2858) and a scaled range
// (scale_parameters_st, lsuv.cpp:101-104): what the LSUV loop needs between two forward passes.
// Block b owns elements [b * kMomentSpan, (b + 1) * kMomentSpan): the split, and with it the order of the
// double additions, depends on the buffer's length only, not on the device.
constexpr size_t kMomentSpan = size_t(kEwBlock) * 16;
__global__ __launch_bounds__(kEwBlock) void k_moment_pairs(float const *__restrict__ x, size_t n,
                                                            double *__restrict__ pairs) {
  __shared__ double sh[2][kEwBlock];
  size_t const first = static_cast<size_t>(blockIdx.x) * kMomentSpan;
  size_t const last = first + kMomentSpan < n ? first + kMomentSpan : n;
  double s = 0.0, q = 0.0;
  for (size_t e = first + threadIdx.x; e < last; e += kEwBlock) {
    double const v = static_cast<double>(x[e]);
    s += v;
    q += v * v;
  }
  sh[0][threadIdx.x] = s;
  sh[1][threadIdx.x] = q;
  __syncthreads();
  for (int half = kEwBlock / 2; half > 0; half >>= 1) {  // fixed pairing: lane i takes lane i + half
    if (static_cast<int>(threadIdx.x) < half) {
      sh[0][threadIdx.x] += sh[0][threadIdx.x + half];
      sh[1][threadIdx.x] += sh[1][threadIdx.x + half];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    pairs[2 * blockIdx.x] = sh[0][0];
    pairs[2 * blockIdx.x + 1] = sh[1][0];
  }
}

// variance = sum(x^2) / n - (sum(x) / n)^2 from the block pairs, added in block order by one thread per
// 256-block stride and then in lane order; written as one float
__global__ __launch_bounds__(kEwBlock) void k_variance_from_pairs(double const *__restrict__ pairs, unsigned nblocks,
                                                                   double inv_n, float *__restrict__ out) {
  __shared__ double sh[2][kEwBlock];
  double s = 0.0, q = 0.0;
  for (unsigned b = threadIdx.x; b < nblocks; b += kEwBlock) {
    s += pairs[2 * b];
    q += pairs[2 * b + 1];
  }
  sh[0][threadIdx.x] = s;
  sh[1][threadIdx.x] = q;
  __syncthreads();
  if (threadIdx.x == 0) {
    double ts = 0.0, tq = 0.0;
    for (int i = 0; i < kEwBlock; ++i) { ts += sh[0][i]; tq += sh[1][i]; }
    double const mean = ts * inv_n;
    out[0] = static_cast<float>(tq * inv_n - mean * mean);
  }
}

__global__ __launch_bounds__(kEwBlock) void k_scale(float *__restrict__ p, size_t n, float factor) {
  size_t const stride = static_cast<size_t>(gridDim.x) * kEwBlock;
  for (size_t e = static_cast<size_t>(blockIdx.x) * kEwBlock + threadIdx.x; e < n; e += stride) p[e] *= factor;
}

}  // namespace dlmi

using namespace dlmi;

extern "C" {

int dlmi_act_fwd(dlmi_ctx *ctx, dlmi_activation act, size_t B, size_t H, float const *x, float *y) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, act_supported(act), "unsupported activation");
  DLMI_REQUIRE(ctx, x && y, "null pointer");
  size_t const n = B * H;
  if (n == 0) return DLMI_OK;
  size_t const n4 = all_aligned16({x, y}) ? n / 4 : 0;
  unsigned const grid = ew_grid(ctx, n4 ? n4 : n);
  DLMI_DISPATCH_ACT(act, hipLaunchKernelGGL((k_act_fwd<ACT>), dim3(grid), dim3(kEwBlock), 0, ctx->stream, x, y, n4, n));
  DLMI_LAUNCH_CHECK(ctx, "k_act_fwd");
  return DLMI_OK;
}

int dlmi_act_bwd(dlmi_ctx *ctx, dlmi_activation act, size_t B, size_t H, float const *pre, float const *post,
                 float const *dY, float *dN) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, act_supported(act), "unsupported activation");
  DLMI_REQUIRE(ctx, pre && post && dY && dN, "null pointer");
  size_t const n = B * H;
  if (n == 0) return DLMI_OK;
  size_t const n4 = all_aligned16({pre, post, dY, dN}) ? n / 4 : 0;
  unsigned const grid = ew_grid(ctx, n4 ? n4 : n);
  DLMI_DISPATCH_ACT(act, hipLaunchKernelGGL((k_act_bwd<ACT>), dim3(grid), dim3(kEwBlock), 0, ctx->stream, pre, post,
                                            dY, dN, n4, n));
  DLMI_LAUNCH_CHECK(ctx, "k_act_bwd");
  return DLMI_OK;
}

// The caller's per-unit types, checked on the host and staged in the context's scratch for the kernel.
static int stage_unit_types(dlmi_ctx *ctx, size_t H, dlmi_activation const *types, int const **d_types) {
  for (size_t j = 0; j < H; ++j)
    if (!act_supported(types[j]))
      return dlmi_fail(ctx, DLMI_E_UNSUPPORTED, "unit %zu: unsupported activation %d", j, static_cast<int>(types[j]));
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(ctx->stream, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
    return dlmi_fail(ctx, DLMI_E_INVALID, "per-unit activation types are copied from the host: not while the stream is being recorded");
  int const rc = dlmi_scratch_reserve(ctx, H * sizeof(int));
  if (rc != DLMI_OK) return rc;
  static_assert(sizeof(dlmi_activation) == sizeof(int), "the enum travels as int");
  // ordered behind the stream's earlier work (the scratch may still be read), complete for the host on return
  DLMI_HIP(ctx, hipMemcpyWithStream(dlmi_scratch_data(ctx), types, H * sizeof(int), hipMemcpyHostToDevice, ctx->stream));
  *d_types = reinterpret_cast<int const *>(dlmi_scratch_data(ctx));
  return DLMI_OK;
}

int dlmi_act_fwd_units(dlmi_ctx *ctx, dlmi_activation const *types, size_t B, size_t H, float const *x, float *y) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, types && x && y, "null pointer");
  size_t const n = B * H;
  if (n == 0) return DLMI_OK;
  int const *d_types = nullptr;
  if (int const rc = stage_unit_types(ctx, H, types, &d_types); rc != DLMI_OK) return rc;
  hipLaunchKernelGGL(k_act_units_fwd, dim3(ew_grid(ctx, n)), dim3(kEwBlock), 0, ctx->stream, d_types, x, y, H, n);
  DLMI_LAUNCH_CHECK(ctx, "k_act_units_fwd");
  return DLMI_OK;
}

int dlmi_act_bwd_units(dlmi_ctx *ctx, dlmi_activation const *types, size_t B, size_t H, float const *pre,
                       float const *post, float const *dY, float *dN) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, types && pre && post && dY && dN, "null pointer");
  size_t const n = B * H;
  if (n == 0) return DLMI_OK;
  int const *d_types = nullptr;
  if (int const rc = stage_unit_types(ctx, H, types, &d_types); rc != DLMI_OK) return rc;
  hipLaunchKernelGGL(k_act_units_bwd, dim3(ew_grid(ctx, n)), dim3(kEwBlock), 0, ctx->stream, d_types, pre, post, dY,
                     dN, H, n);
  DLMI_LAUNCH_CHECK(ctx, "k_act_units_bwd");
  return DLMI_OK;
}

int dlmi_identity_add(dlmi_ctx *ctx, size_t n, float const *a, float const *b, float *out) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, a && b && out, "null pointer");
  if (n == 0) return DLMI_OK;
  size_t const n4 = all_aligned16({a, b, out}) ? n / 4 : 0;
  hipLaunchKernelGGL(k_add, dim3(ew_grid(ctx, n4 ? n4 : n)), dim3(kEwBlock), 0, ctx->stream, a, b, out, n4, n);
  DLMI_LAUNCH_CHECK(ctx, "k_add");
  return DLMI_OK;
}

int dlmi_zero_padded_identity_fwd(dlmi_ctx *ctx, size_t B, size_t HA, size_t HB, size_t padding, float const *a,
                                  float const *b, float *out) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, a && b && out, "null pointer");
  if (padding == 0) {
    DLMI_REQUIRE(ctx, HA == HB, "no padding needs equal widths");
    return dlmi_identity_add(ctx, B * HA, a, b, out);
  }
  DLMI_REQUIRE(ctx, HA != HB, "padding needs operands of different widths");
  bool const a_wide = HA > HB;
  size_t const Hw = a_wide ? HA : HB, Hn = a_wide ? HB : HA;
  DLMI_REQUIRE(ctx, padding + Hn <= Hw, "the padded operand does not fit the wider one");
  if (B * Hw == 0) return DLMI_OK;
  hipLaunchKernelGGL(k_padded_add, dim3(ew_grid(ctx, B * Hw)), dim3(kEwBlock), 0, ctx->stream, a_wide ? a : b,
                     a_wide ? b : a, out, B, Hw, Hn, padding);
  DLMI_LAUNCH_CHECK(ctx, "k_padded_add");
  return DLMI_OK;
}

int dlmi_residual_bwd(dlmi_ctx *ctx, size_t B, size_t input_size, size_t derivative_size, size_t padding,
                      float const *d_inputs, float *derivatives) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, d_inputs && derivatives, "null pointer");
  size_t const Hc = input_size < derivative_size ? input_size : derivative_size;
  size_t const Hwide = input_size < derivative_size ? derivative_size : input_size;
  size_t const pad = input_size == derivative_size ? 0 : padding;
  DLMI_REQUIRE(ctx, pad + Hc <= Hwide, "the padded operand does not fit the wider one");
  if (B * Hc == 0) return DLMI_OK;
  hipLaunchKernelGGL(k_residual_bwd, dim3(ew_grid(ctx, B * Hc)), dim3(kEwBlock), 0, ctx->stream, d_inputs, derivatives,
                     B, input_size, derivative_size, Hc, input_size > derivative_size ? pad : 0,
                     input_size < derivative_size ? pad : 0);
  DLMI_LAUNCH_CHECK(ctx, "k_residual_bwd");
  return DLMI_OK;
}

int dlmi_zero(dlmi_ctx *ctx, size_t n, float *p) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  if (n == 0) return DLMI_OK;
  DLMI_REQUIRE(ctx, p != nullptr, "null pointer");
  hipLaunchKernelGGL(k_zero, dim3(ew_grid(ctx, n)), dim3(kEwBlock), 0, ctx->stream, p, n);
  DLMI_LAUNCH_CHECK(ctx, "k_zero");
  return DLMI_OK;
}

int dlmi_layer_variance(dlmi_ctx *ctx, size_t B, size_t H, float const *y, float *variance) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, y != nullptr && variance != nullptr, "null pointer");
  size_t const n = B * H;
  DLMI_REQUIRE(ctx, n != 0, "dlmi_layer_variance: empty buffer");
  size_t const nblocks = dlmi_ceil_div(n, kMomentSpan);
  DLMI_REQUIRE(ctx, nblocks <= 0x7fffffffu, "dlmi_layer_variance: buffer too long");
  int rc = dlmi_scratch_reserve(ctx, nblocks * 2 * sizeof(double) + 256);
  if (rc != DLMI_OK) return rc;
  // the result sits in front of the pairs (256 bytes keep the doubles aligned)
  float *d_out = reinterpret_cast<float *>(dlmi_scratch_data(ctx));
  double *pairs = reinterpret_cast<double *>(reinterpret_cast<unsigned char *>(dlmi_scratch_data(ctx)) + 256);
  hipLaunchKernelGGL(k_moment_pairs, dim3(static_cast<unsigned>(nblocks)), dim3(kEwBlock), 0, ctx->stream, y, n, pairs);
  DLMI_LAUNCH_CHECK(ctx, "k_moment_pairs");
  hipLaunchKernelGGL(k_variance_from_pairs, dim3(1), dim3(kEwBlock), 0, ctx->stream, pairs,
                     static_cast<unsigned>(nblocks), 1.0 / static_cast<double>(n), d_out);
  DLMI_LAUNCH_CHECK(ctx, "k_variance_from_pairs");
  hipError_t const e = hipMemcpyAsync(variance, d_out, sizeof(float), hipMemcpyDeviceToHost, ctx->stream);
  if (e != hipSuccess) return dlmi_fail(ctx, DLMI_E_HIP, "dlmi_layer_variance: copy: %s", hipGetErrorString(e));
  return dlmi_ctx_synchronize(ctx);
}

int dlmi_scale(dlmi_ctx *ctx, size_t n, float *p, float factor) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  if (n == 0) return DLMI_OK;
  DLMI_REQUIRE(ctx, p != nullptr, "null pointer");
  hipLaunchKernelGGL(k_scale, dim3(ew_grid(ctx, n)), dim3(kEwBlock), 0, ctx->stream, p, n, factor);
  DLMI_LAUNCH_CHECK(ctx, "k_scale");
  return DLMI_OK;
}

int dlmi_bias_fwd(dlmi_ctx *ctx, size_t B, size_t H, float const *bias, float *Z) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, bias && Z, "null pointer");
  if (B * H == 0) return DLMI_OK;
  RowArgs a{};
  a.x = Z; a.y = Z; a.p0 = bias; a.B = B; a.H = H; a.scale = 1.0f;
  return launch_row<0, DLMI_ACT_LINEAR>(ctx, a, "k_row<bias>");
}

int dlmi_dropout_fwd(dlmi_ctx *ctx, dlmi_dropout kind, int training, int per_element, size_t B, size_t H,
                     uint8_t const *mask, float scale, float *v) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, v != nullptr, "null pointer");
  DLMI_REQUIRE(ctx, kind == DLMI_DROP_NONE || kind == DLMI_DROP_BERNOULLI || kind == DLMI_DROP_BERNOULLI_INVERTED,
               "unsupported dropout");
  if (B * H == 0 || kind == DLMI_DROP_NONE) return DLMI_OK;
  RowArgs a{};
  a.x = v; a.y = v; a.mask = mask; a.B = B; a.H = H; a.per_element = per_element; a.scale = scale;
  if (training) {
    DLMI_REQUIRE(ctx, mask != nullptr, "training-mode dropout needs a mask");
    a.drop_kind = kind == DLMI_DROP_BERNOULLI ? 1 : 2;
  } else {
    if (kind != DLMI_DROP_BERNOULLI) return DLMI_OK;  // inverted dropout is the identity at inference
    a.drop_kind = 3;
  }
  return launch_row<1, DLMI_ACT_LINEAR>(ctx, a, "k_row<dropout>");
}

int dlmi_norm_fwd_infer(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float const *gamma, float const *beta,
                        float const *mov_mean, float const *mov_std, float *out) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, x && gamma && beta && mov_mean && mov_std && out, "null pointer");
  if (B * H == 0) return DLMI_OK;
  RowArgs a{};
  a.x = x; a.y = out; a.p0 = gamma; a.p1 = beta; a.p2 = mov_mean; a.p3 = mov_std; a.B = B; a.H = H; a.scale = 1.0f;
  return launch_row<2, DLMI_ACT_LINEAR>(ctx, a, "k_row<norm_infer>");
}

int dlmi_fused_norm_act_infer(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                              float const *gamma, float const *beta, float const *mov_mean, float const *mov_std,
                              float *y) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, act_supported(desc->act), "unsupported activation");
  DLMI_REQUIRE(ctx, x && gamma && beta && mov_mean && mov_std && y, "null pointer");
  if (B * H == 0) return DLMI_OK;
  RowArgs a{};
  a.x = x; a.y = y; a.p0 = gamma; a.p1 = beta; a.p2 = mov_mean; a.p3 = mov_std; a.B = B; a.H = H;
  // plain Bernoulli rescales by the keep probability at inference (fwp_st.cpp:705-716)
  a.scale = desc->dropout == DLMI_DROP_BERNOULLI ? desc->drop_scale : 1.0f;
  int rc = DLMI_OK;
  DLMI_DISPATCH_ACT(desc->act, rc = (launch_row<2, ACT>(ctx, a, "k_row<norm_act_infer>")));
  return rc;
}

int dlmi_softmax_fwd(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float *y) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, x && y, "null pointer");
  if (B * H == 0) return DLMI_OK;
  hipLaunchKernelGGL(k_softmax, dim3(static_cast<unsigned>(dlmi_ceil_div(B, kEwBlock / 64))), dim3(kEwBlock), 0,
                     ctx->stream, x, y, B, H);
  DLMI_LAUNCH_CHECK(ctx, "k_softmax");
  return DLMI_OK;
}

int dlmi_softmax_ce_seed(dlmi_ctx *ctx, size_t B, size_t H, float const *q, float const *y, float *dZ,
                         double *stats) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, q && y && dZ, "null pointer");
  if (B * H == 0) return DLMI_OK;
  unsigned const nblocks = static_cast<unsigned>(dlmi_ceil_div(B, kEwBlock / 64));
  double *pairs = nullptr;
  if (stats != nullptr) {
    int rc = dlmi_scratch_reserve(ctx, static_cast<size_t>(nblocks) * 2 * sizeof(double));
    if (rc != DLMI_OK) return rc;
    pairs = reinterpret_cast<double *>(dlmi_scratch_data(ctx));
  }
  hipLaunchKernelGGL(k_softmax_ce_seed, dim3(nblocks), dim3(kEwBlock), 0, ctx->stream, q, y, dZ, B, H, pairs, stats,
                     ctx->pair_ticket);
  DLMI_LAUNCH_CHECK(ctx, "k_softmax_ce_seed");
  return DLMI_OK;
}

}  // extern "C"
