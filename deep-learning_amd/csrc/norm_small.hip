// Batch-(re)normalization + activation + dropout for SMALL batches (at most 256 rows, at most 2^20
// elements): one launch per direction.
//
// A mini-batch of the reference's own size (128 rows of a few hundred units) is a few hundred KB: the
// multi-launch path spends its time on the latency of three or four kernels, not on memory.  Here a
// workgroup owns 8 adjacent columns for ALL rows (256 threads = 32 row groups x 8 columns, every thread
// keeps its B / 32 rows in registers), so the column sums, the per-unit statistics and the apply step
// happen in one kernel with one LDS exchange in between.  The forward can also take the K slices of a
// split-K product as its input: it adds them in slice order (what k_splitk_reduce would have done),
// writes Z and carries on, which removes that launch as well.  Sums run in a fixed order (rows of a
// thread ascending, then row groups ascending): bit-reproducible, no float atomics.
// Citations: /root/reference/lib/deep-learning/v1/learner/ fwp_st.cpp:4586-4794, bwp_st.cpp:1177-1209,
// 1284-1366, 1447-1532.
#include <hip/hip_runtime.h>

#include "norm_shared.hpp"

namespace dlmi {
namespace {

constexpr int kSmallCols = 8;      // columns of a workgroup
constexpr int kSmallGroups = 32;   // row groups of a workgroup
constexpr int kSmallThreads = kSmallCols * kSmallGroups;
constexpr size_t kSmallMaxRows = 256;
constexpr size_t kSmallMaxElements = size_t(1) << 20;

struct SmallFwdArgs {
  float const *x;       // [B, H]; unused when slices are given
  float const *slices;  // [nslices][B][H] partial products whose sum is x, or nullptr
  float *z_out;         // where that sum is stored (slices only)
  unsigned nslices;
  float const *gamma, *beta, *residual;
  uint8_t const *mask;
  float *y;
  size_t B, H;
  FwdFinalize fin;
  int drop_mode;
  float drop_scale;
};

// RPT: rows per thread (B <= 32 * RPT).
template <int ACT, int RPT>
__global__ __launch_bounds__(kSmallThreads) void k_small_fwd(SmallFwdArgs a) {
  __shared__ float red[2][kSmallGroups][kSmallCols];
  int const c = threadIdx.x % kSmallCols, rg = threadIdx.x / kSmallCols;
  size_t const col = static_cast<size_t>(blockIdx.x) * kSmallCols + c;
  bool const live = col < a.H;
  float mm = 0.0f, ms = 1.0f, ga = 1.0f, be = 0.0f;
  uint8_t mk = 1;
  if (live) {
    mm = a.fin.mov_mean[col];
    ms = a.fin.mov_std[col];
    ga = a.gamma[col];
    be = a.beta[col];
    if (a.drop_mode == kDropUnit) mk = a.mask[col];
  }
  float v[RPT];
  bool ok[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    ok[i] = live && static_cast<size_t>(rg + kSmallGroups * i) < a.B;
    v[i] = 0.0f;
  }
  if (a.slices != nullptr) {
    size_t const plane = a.B * a.H;
    for (unsigned s = 0; s < a.nslices; ++s) {
      float t[RPT];
#pragma unroll
      for (int i = 0; i < RPT; ++i)
        t[i] = ok[i] ? a.slices[s * plane + static_cast<size_t>(rg + kSmallGroups * i) * a.H + col] : 0.0f;
#pragma unroll
      for (int i = 0; i < RPT; ++i) v[i] += t[i];
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i)
      if (ok[i]) a.z_out[static_cast<size_t>(rg + kSmallGroups * i) * a.H + col] = v[i];
  } else {
#pragma unroll
    for (int i = 0; i < RPT; ++i)
      if (ok[i]) v[i] = a.x[static_cast<size_t>(rg + kSmallGroups * i) * a.H + col];
  }
  float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
  for (int i = 0; i < RPT; ++i) {  // rows that do not exist hold 0
    s1 += v[i];
    s2 += v[i] * v[i];
  }
  red[0][rg][c] = s1;
  red[1][rg][c] = s2;
  __syncthreads();
  float t1 = 0.0f, t2 = 0.0f;
#pragma unroll
  for (int g = 0; g < kSmallGroups; ++g) {
    t1 += red[0][g][c];
    t2 += red[1][g][c];
  }
  // every thread of a column forms the same statistics; one stores them (the moving statistics were read
  // by all of them before the barrier above)
  UnitStats const u = fwd_unit_stats(a.fin, t1, t2, mm, ms);
  if (live && rg == 0) store_unit_stats(a.fin, col, u);
  float const inv = fast_rcp(u.stdv);
  float const rr = ga * (u.r * inv);   // gamma * r / std
  float const dd = ga * u.d + be;      // gamma * d + beta
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    if (!ok[i]) continue;
    size_t const off = static_cast<size_t>(rg + kSmallGroups * i) * a.H + col;
    float const nn = (v[i] - u.mean) * rr + dd;
    float q = act_fire<ACT>(nn);
    if (a.drop_mode != kDropNone) q = drop_apply(a.drop_mode == kDropElem ? a.mask[off] : mk, a.drop_scale, q);
    if (a.residual != nullptr) {
      asm volatile("" : "+v"(q));  // a rounding of its own, as the reference's add of two stored arrays
      q = a.residual[off] + q;
    }
    a.y[off] = q;
  }
}

struct SmallBwdArgs {
  float const *x, *dY, *gamma, *beta, *mean, *stdv, *r, *d;
  float const *dy_slices;  // [nslices][B][H] whose sum is dY, or nullptr
  unsigned nslices;
  float const *narrow_dz, *narrow_w;  // dY = narrow_dz [B][narrow_h] . narrow_w [narrow_h][H], or nullptr
  unsigned narrow_h;
  uint8_t const *mask;
  float *dgamma, *dbeta, *dX;
  size_t B, H;
  float batch_f, batch_scale, drop_scale;
  int drop_mode, drop_bwd_masked, accumulate;
};

template <int ACT, int RPT>
__global__ __launch_bounds__(kSmallThreads) void k_small_bwd(SmallBwdArgs a) {
  __shared__ float red[3][kSmallGroups][kSmallCols];
  __shared__ float ndz[kSmallMaxRows * kNarrowMaxUnits];  // the narrow layer's dZ, all rows
  int const c = threadIdx.x % kSmallCols, rg = threadIdx.x / kSmallCols;
  size_t const col = static_cast<size_t>(blockIdx.x) * kSmallCols + c;
  bool const live = col < a.H;
  // (all of a thread's loads are asked for before the first one is used: one memory latency, not one per piece)
  constexpr int kNdzPerThread = static_cast<int>(kSmallMaxRows * kNarrowMaxUnits / kSmallThreads);
  float ndz_in[kNdzPerThread];
  unsigned const ndz_count = a.narrow_dz != nullptr ? static_cast<unsigned>(a.B) * a.narrow_h : 0u;
  if (a.narrow_dz != nullptr) {
#pragma unroll
    for (int k = 0; k < kNdzPerThread; ++k) {
      unsigned const i = threadIdx.x + static_cast<unsigned>(k) * kSmallThreads;
      ndz_in[k] = i < ndz_count ? a.narrow_dz[i] : 0.0f;
    }
  }
  float mu = 0.0f, sd = 1.0f, rr = 1.0f, dd = 0.0f, ga = 1.0f, be = 0.0f;
  uint8_t mk = 1;
  if (live) {
    mu = a.mean[col];
    sd = a.stdv[col];
    if (a.r != nullptr) rr = a.r[col];
    if (a.d != nullptr) dd = a.d[col];
    ga = a.gamma[col];
    be = a.beta[col];
    if (a.drop_mode == kDropUnit) mk = a.mask[col];
  }
  float const rs = rr * fast_rcp(sd);
  // without dropout the masked form with m = 1 and scale = 1 is the plain one (q * 1 is exact)
  float const scale = a.drop_mode == kDropNone ? 1.0f : a.drop_scale;
  int const masked = a.drop_mode == kDropNone ? 0 : a.drop_bwd_masked;
  float xv[RPT], dn[RPT];
  bool ok[RPT];
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    ok[i] = live && static_cast<size_t>(rg + kSmallGroups * i) < a.B;
    xv[i] = mu;
    dn[i] = 0.0f;
  }
  float dy[RPT];
  uint8_t mv[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    size_t const off = static_cast<size_t>(rg + kSmallGroups * i) * a.H + col;
    dy[i] = 0.0f;
    mv[i] = mk;
    if (ok[i]) {
      xv[i] = a.x[off];
      if (a.dy_slices == nullptr && a.narrow_dz == nullptr) dy[i] = a.dY[off];
      if (a.drop_mode == kDropElem) mv[i] = a.mask[off];
    }
  }
  if (a.narrow_dz != nullptr) {
    // this column of the narrow layer's weights, then one chain of multiply-adds per row, units ascending
    float w[kNarrowMaxUnits];
#pragma unroll
    for (unsigned u = 0; u < kNarrowMaxUnits; ++u) w[u] = live && u < a.narrow_h ? a.narrow_w[u * a.H + col] : 0.0f;
#pragma unroll
    for (int k = 0; k < kNdzPerThread; ++k) {
      unsigned const i = threadIdx.x + static_cast<unsigned>(k) * kSmallThreads;
      if (i < ndz_count) ndz[i] = ndz_in[k];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      if (!ok[i]) continue;
      float const *z = ndz + static_cast<unsigned>(rg + kSmallGroups * i) * a.narrow_h;
      float t = 0.0f;
#pragma unroll
      for (unsigned u = 0; u < kNarrowMaxUnits; ++u)
        if (u < a.narrow_h) t = fmaf(z[u], w[u], t);
      dy[i] = t;
    }
  } else if (a.dy_slices != nullptr) {
    size_t const plane = a.B * a.H;
    for (unsigned s = 0; s < a.nslices; ++s) {
      float t[RPT];
#pragma unroll
      for (int i = 0; i < RPT; ++i)
        t[i] = ok[i] ? a.dy_slices[s * plane + static_cast<size_t>(rg + kSmallGroups * i) * a.H + col] : 0.0f;
#pragma unroll
      for (int i = 0; i < RPT; ++i) dy[i] += t[i];
    }
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    if (!ok[i]) continue;
    float xh = 0.0f;
    dn[i] = bwd_dn<ACT, kDropElem, false>(scale, masked, xv[i], dy[i], mv[i], mu, rs, dd, ga, be, xh);
    s0 += dn[i] * xh;
    s1 += dn[i];
    s2 += dn[i] * (xv[i] - mu);
  }
  red[0][rg][c] = s0;
  red[1][rg][c] = s1;
  red[2][rg][c] = s2;
  __syncthreads();
  float t0 = 0.0f, t1 = 0.0f, t2 = 0.0f;
#pragma unroll
  for (int g = 0; g < kSmallGroups; ++g) {
    t0 += red[0][g][c];
    t1 += red[1][g][c];
    t2 += red[2][g][c];
  }
  if (live && rg == 0) {  // accumulating like the reference's derivative array
    a.dgamma[col] += t0;
    a.dbeta[col] += t1;
  }
  // the per-unit coefficients of pass 2 (bwp_st.cpp:1508-1531), as the multi-launch finalize forms them
  float const dm = (ga * t1) * (-rr / sd);
  float const ds = (ga * t2) * (-rr / (sd * sd));
  float const c1 = ga * (rr / sd);
  float const c2 = ds / (a.batch_f * sd);
  float const c3 = dm * a.batch_scale;
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    if (!ok[i]) continue;
    size_t const off = static_cast<size_t>(rg + kSmallGroups * i) * a.H + col;
    float dx = dn[i] * c1 + (xv[i] - mu) * c2 + c3;
    if (a.accumulate) dx += a.dX[off];
    a.dX[off] = dx;
  }
}

// out[j] (+)= sum_b x[b, j]
template <int RPT>
__global__ __launch_bounds__(kSmallThreads) void k_small_colsum(float const *__restrict__ x, float *__restrict__ out,
                                                                 size_t B, size_t H, int accumulate) {
  __shared__ float red[kSmallGroups][kSmallCols];
  int const c = threadIdx.x % kSmallCols, rg = threadIdx.x / kSmallCols;
  size_t const col = static_cast<size_t>(blockIdx.x) * kSmallCols + c;
  bool const live = col < H;
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    size_t const b = static_cast<size_t>(rg + kSmallGroups * i);
    if (live && b < B) s += x[b * H + col];
  }
  red[rg][c] = s;
  __syncthreads();
  if (rg == 0 && live) {
    float t = 0.0f;
#pragma unroll
    for (int g = 0; g < kSmallGroups; ++g) t += red[g][c];
    out[col] = accumulate ? out[col] + t : t;
  }
}

int rows_per_thread(size_t B) {
  size_t const need = dlmi_ceil_div(B, static_cast<size_t>(kSmallGroups));
  return need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : 8;
}

#define DLMI_DISPATCH_RPT(rpt, ...)                          \
  switch (rpt) {                                             \
    case 1: { constexpr int RPT = 1; __VA_ARGS__; } break;   \
    case 2: { constexpr int RPT = 2; __VA_ARGS__; } break;   \
    case 4: { constexpr int RPT = 4; __VA_ARGS__; } break;   \
    default: { constexpr int RPT = 8; __VA_ARGS__; } break;  \
  }

}  // namespace

bool small_norm_eligible(dlmi_ctx const *ctx, size_t B, size_t H) {
  return ctx->tune.norm_small != 0 && B <= kSmallMaxRows && B * H <= kSmallMaxElements;
}

int small_fwd_try(dlmi_ctx *ctx, size_t B, size_t H, FwdTrainCall const &c) {
  bool const wanted = c.slices != nullptr;  // the producer already left its reduction to this kernel
  if (!small_norm_eligible(ctx, B, H) || c.xhat != nullptr || c.nrm != nullptr || c.y == nullptr) {
    if (wanted) return dlmi_fail(ctx, DLMI_E_INVALID, "small-batch forward: K slices given for a call it cannot take");
    return 0;
  }
  SmallFwdArgs a;
  a.x = c.x; a.slices = c.slices; a.z_out = c.z_out; a.nslices = c.nslices;
  a.gamma = c.gamma; a.beta = c.beta; a.residual = c.residual; a.mask = c.mask; a.y = c.y;
  a.B = B; a.H = H;
  a.fin.mean = c.mean; a.fin.stdv = c.stdv; a.fin.mov_mean = c.mov_mean; a.fin.mov_std = c.mov_std; a.fin.r = c.r; a.fin.d = c.d;
  a.fin.batch_scale = 1.0f / static_cast<float>(B);
  a.fin.momentum = c.momentum; a.fin.eps = c.eps; a.fin.r_max = c.r_max; a.fin.d_max = c.d_max;
  a.fin.renorm = c.norm == DLMI_NORM_BATCH_RENORM ? 1 : 0;
  a.drop_mode = c.drop_mode; a.drop_scale = c.drop_scale;
  dim3 const grid(static_cast<unsigned>(dlmi_ceil_div(H, static_cast<size_t>(kSmallCols))));
  int const rpt = rows_per_thread(B);
  DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_RPT(rpt, {
    hipLaunchKernelGGL((k_small_fwd<ACT, RPT>), grid, dim3(kSmallThreads), 0, ctx->stream, a);
  }));
  DLMI_LAUNCH_CHECK(ctx, "k_small_fwd");
  return 1;
}

int small_bwd_try(dlmi_ctx *ctx, size_t B, size_t H, BwdCall const &c) {
  if (!small_norm_eligible(ctx, B, H) || c.xhat_given || c.dmean != nullptr || c.dstd != nullptr) {
    if (c.dy_slices != nullptr || c.narrow_dz != nullptr)
      return dlmi_fail(ctx, DLMI_E_INVALID, "small-batch backward: a deferred product given for a call it cannot take");
    return 0;
  }
  if (c.narrow_dz != nullptr && (c.narrow_h == 0 || c.narrow_h > kNarrowMaxUnits || c.narrow_w == nullptr || c.dy_slices != nullptr))
    return dlmi_fail(ctx, DLMI_E_INVALID, "small-batch backward: bad narrow product");
  SmallBwdArgs a;
  a.dy_slices = c.dy_slices; a.nslices = c.nslices;
  a.narrow_dz = c.narrow_dz; a.narrow_w = c.narrow_w; a.narrow_h = c.narrow_h;
  a.x = c.x; a.dY = c.dY; a.gamma = c.gamma; a.beta = c.beta; a.mean = c.mean; a.stdv = c.stdv; a.r = c.r; a.d = c.d;
  a.mask = c.mask; a.dgamma = c.dgamma; a.dbeta = c.dbeta; a.dX = c.dX;
  a.B = B; a.H = H;
  a.batch_f = static_cast<float>(B); a.batch_scale = 1.0f / static_cast<float>(B); a.drop_scale = c.drop_scale;
  a.drop_mode = c.drop_mode; a.drop_bwd_masked = c.drop_bwd_masked; a.accumulate = c.accumulate ? 1 : 0;
  dim3 const grid(static_cast<unsigned>(dlmi_ceil_div(H, static_cast<size_t>(kSmallCols))));
  int const rpt = rows_per_thread(B);
  DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_RPT(rpt, {
    hipLaunchKernelGGL((k_small_bwd<ACT, RPT>), grid, dim3(kSmallThreads), 0, ctx->stream, a);
  }));
  DLMI_LAUNCH_CHECK(ctx, "k_small_bwd");
  return 1;
}

int small_colsum_try(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float *out, int accumulate) {
  if (!small_norm_eligible(ctx, B, H)) return 0;
  dim3 const grid(static_cast<unsigned>(dlmi_ceil_div(H, static_cast<size_t>(kSmallCols))));
  int const rpt = rows_per_thread(B);
  DLMI_DISPATCH_RPT(rpt, {
    hipLaunchKernelGGL((k_small_colsum<RPT>), grid, dim3(kSmallThreads), 0, ctx->stream, x, out, B, H, accumulate);
  });
  DLMI_LAUNCH_CHECK(ctx, "k_small_colsum");
  return 1;
}

}  // namespace dlmi
