// Batch normalization / batch renormalization kernels (training forward and
// backward, fused with the activation and the dropout mask) for gfx950.
//
// All of them are bound by HBM bandwidth, so the design goal is the minimum
// number of passes over the [B, H] tensors with fully coalesced 16-byte
// accesses and enough independent loads in flight per CU:
//
//   forward : stats (read x)            -> finalize [H] -> apply (read x, write y)
//   backward: reduce (read dY, x)       -> finalize [H] -> apply (read dY, x, write dX)
//
// x_hat, the pre-activation n = gamma*x_hat + beta and the activation output
// are recomputed in registers instead of being stored and re-read.
//
// Thread geometry of the column passes: a 256-thread block is TX x TY; a
// thread owns VEC (=4, one float4) adjacent units and walks the rows of its
// block's batch chunk with stride TY.  TX <= 64, so when H is small a
// wavefront spans several rows: those are combined with wavefront shuffles,
// the four wavefronts of the block with a small LDS tree, and the chunks of the
// batch by the finalize kernel in a fixed order (no float atomics: results are
// reproducible run to run).
//
// Citations: /root/reference/lib/deep-learning/v1/learner/.
#include "activations.hpp"
#include "dlmi_common.hpp"

namespace dlmi {

constexpr int kBlock = 256;
constexpr int kWave = 64;

struct ColGeom {
  int vec;        // 4 (float4 path) or 1 (any H, any alignment)
  int tx, tx_log2, ty;
  unsigned grid_x;
  unsigned nchunks;
  size_t rows_per_chunk;
};

static ColGeom col_geometry(dlmi_ctx const *ctx, size_t B, size_t H, bool vec4, int nacc) {
  ColGeom g;
  g.vec = vec4 ? 4 : 1;
  size_t const groups = dlmi_ceil_div(H, g.vec);
  g.tx = 64;
  g.tx_log2 = 6;
  while (g.tx > 1 && static_cast<size_t>(g.tx / 2) >= groups) {
    g.tx /= 2;
    --g.tx_log2;
  }
  g.ty = kBlock / g.tx;
  g.grid_x = static_cast<unsigned>(dlmi_ceil_div(groups, g.tx));
  // enough blocks to cover every CU a few times over, but each thread should
  // still stream >= 8 rows so the partials stay a small fraction of the traffic
  size_t want = dlmi_ceil_div(static_cast<size_t>(ctx->num_cu) * 8, g.grid_x);
  size_t const max_by_rows = B / (static_cast<size_t>(g.ty) * 8);
  if (want > max_by_rows) want = max_by_rows;
  // partial sums must fit the scratch block: nacc * nchunks * H floats (half of it)
  size_t const max_by_scratch = (ctx->scratch_bytes / 2) / (static_cast<size_t>(nacc) * H * sizeof(float));
  if (want > max_by_scratch) want = max_by_scratch;
  if (want < 1) want = 1;
  if (want > 65535) want = 65535;
  g.rows_per_chunk = dlmi_ceil_div(B, want);
  g.nchunks = static_cast<unsigned>(dlmi_ceil_div(B, g.rows_per_chunk));
  return g;
}

template <int VEC>
struct Vec;
template <>
struct Vec<4> {
  using f = float4;
  using u = uchar4;
};
template <>
struct Vec<1> {
  using f = float;
  using u = unsigned char;
};

template <int VEC>
__device__ __forceinline__ void load_f(float const *p, float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    float4 const t = *reinterpret_cast<float4 const *>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
    v[0] = *p;
  }
}
template <int VEC>
__device__ __forceinline__ void store_f(float *p, float const (&v)[VEC]) {
  if constexpr (VEC == 4) {
    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    *p = v[0];
  }
}
template <int VEC>
__device__ __forceinline__ void load_u8(uint8_t const *p, uint8_t (&v)[VEC]) {
  if constexpr (VEC == 4) {
    uchar4 const t = *reinterpret_cast<uchar4 const *>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
    v[0] = *p;
  }
}

// Sum NV per-thread values over the TY rows of the block.  On return the
// threads with threadIdx.x < TX hold the block totals for their column group.
template <int NV>
__device__ __forceinline__ void block_rows_reduce(float (&v)[NV], int tx, float *lds) {
  int const lane = threadIdx.x & (kWave - 1);
  int const wave = threadIdx.x / kWave;
  // rows that share a wavefront: lanes tx apart hold the same column group
  for (int off = tx; off < kWave; off <<= 1) {
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] += __shfl_xor(v[i], off, kWave);
  }
  int const cols_in_wave = tx < kWave ? tx : kWave;
  if (lane < cols_in_wave) {
#pragma unroll
    for (int i = 0; i < NV; ++i) lds[(wave * kWave + lane) * NV + i] = v[i];
  }
  __syncthreads();
  // LDS tree over the four wavefronts: (0+1) + (2+3), fixed order
  if (threadIdx.x < cols_in_wave) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      float const a = lds[(0 * kWave + lane) * NV + i] + lds[(1 * kWave + lane) * NV + i];
      float const b = lds[(2 * kWave + lane) * NV + i] + lds[(3 * kWave + lane) * NV + i];
      v[i] = a + b;
    }
  }
}

// ---------------------------------------------------------------- forward: statistics
// partial[(a * nchunks + chunk) * H + j], a = 0: sum x, 1: sum x^2
// (phase 1 of fwp_st.cpp:4692-4707 / fwp_mp.cpp:4640-4662)
template <int VEC>
__global__ __launch_bounds__(kBlock) void k_col_stats(float const *__restrict__ x, size_t B, size_t H,
                                                       int tx_log2, size_t rows_per_chunk,
                                                       float *__restrict__ partial) {
  __shared__ float lds[4 * kWave * 2 * VEC];
  int const TX = 1 << tx_log2, TY = kBlock >> tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  bool const live = col < H;
  size_t const b0 = blockIdx.y * rows_per_chunk;
  size_t const b1 = (b0 + rows_per_chunk < B) ? b0 + rows_per_chunk : B;
  float acc[2 * VEC];
#pragma unroll
  for (int i = 0; i < 2 * VEC; ++i) acc[i] = 0.0f;
  if (live) {
    size_t b = b0 + ty;
    for (; b + 3 * static_cast<size_t>(TY) < b1; b += 4 * static_cast<size_t>(TY)) {
      float v[4][VEC];
#pragma unroll
      for (int u = 0; u < 4; ++u) load_f<VEC>(x + (b + u * static_cast<size_t>(TY)) * H + col, v[u]);
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          acc[i] += v[u][i];
          acc[VEC + i] += v[u][i] * v[u][i];
        }
    }
    for (; b < b1; b += TY) {
      float v[VEC];
      load_f<VEC>(x + b * H + col, v);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        acc[i] += v[i];
        acc[VEC + i] += v[i] * v[i];
      }
    }
  }
  block_rows_reduce<2 * VEC>(acc, TX, lds);
  if (threadIdx.x < TX && live) {
    size_t const nch = gridDim.y;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      partial[(0 * nch + blockIdx.y) * H + col + i] = acc[i];
      partial[(1 * nch + blockIdx.y) * H + col + i] = acc[VEC + i];
    }
  }
}

// Sums NA partial-sum planes over the batch chunks for 64 adjacent units per
// block: wavefront w adds chunks w, w+4, w+8, ... (coalesced 256-byte rows, four
// independent accumulation chains per unit), then the four wavefront totals
// are combined through LDS in a fixed order.  On return the threads of
// wavefront 0 hold the totals of unit blockIdx.x*64 + lane.
constexpr int kFinCols = 64;
template <int NA>
__device__ __forceinline__ void chunk_totals(float const *__restrict__ partial, unsigned nchunks, size_t H,
                                             float (&tot)[NA], float *lds) {
  int const lane = threadIdx.x & (kWave - 1);
  int const wave = threadIdx.x / kWave;
  size_t const j = static_cast<size_t>(blockIdx.x) * kFinCols + lane;
#pragma unroll
  for (int a = 0; a < NA; ++a) tot[a] = 0.0f;
  if (j < H) {
    for (unsigned c = wave; c < nchunks; c += kBlock / kWave) {
#pragma unroll
      for (int a = 0; a < NA; ++a) tot[a] += partial[(a * static_cast<size_t>(nchunks) + c) * H + j];
    }
  }
#pragma unroll
  for (int a = 0; a < NA; ++a) lds[(wave * kWave + lane) * NA + a] = tot[a];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int a = 0; a < NA; ++a)
      tot[a] = (lds[(0 * kWave + lane) * NA + a] + lds[(1 * kWave + lane) * NA + a]) +
               (lds[(2 * kWave + lane) * NA + a] + lds[(3 * kWave + lane) * NA + a]);
  }
}

// Phase 2 of fwp_st.cpp:4709-4746: batch mean, moving mean, batch std, moving
// std, then r and d from the UPDATED moving statistics.  64 units per block.
__global__ __launch_bounds__(kBlock) void k_fwd_finalize(float const *__restrict__ partial, unsigned nchunks,
                                                          size_t B, size_t H, int renorm, float momentum,
                                                          float eps, float r_max, float d_max,
                                                          float *__restrict__ mean, float *__restrict__ stdv,
                                                          float *__restrict__ mov_mean,
                                                          float *__restrict__ mov_std, float *__restrict__ r,
                                                          float *__restrict__ d) {
  __shared__ float lds[kBlock * 2];
  float tot[2];
  chunk_totals<2>(partial, nchunks, H, tot, lds);
  size_t const j = static_cast<size_t>(blockIdx.x) * kFinCols + threadIdx.x;
  if (threadIdx.x >= kWave || j >= H) return;
  float const s1 = tot[0], s2 = tot[1];
  float const batch_scale = 1.0f / static_cast<float>(B);
  float const mu = s1 * batch_scale;
  float mm = mov_mean[j];
  mm += momentum * (mu - mm);
  float const sd = sqrtf(s2 * batch_scale - mu * mu + eps);
  float ms = mov_std[j];
  ms += momentum * (sd - ms);
  mean[j] = mu;
  stdv[j] = sd;
  mov_mean[j] = mm;
  mov_std[j] = ms;
  if (renorm) {
    float const g = sd / ms;
    float const lo = 1.0f / r_max;
    r[j] = g < lo ? lo : (g > r_max ? r_max : g);
    float const dd = (mu - mm) / ms;
    d[j] = dd < -d_max ? -d_max : (dd > d_max ? d_max : dd);
  } else {
    if (r != nullptr) r[j] = 1.0f;
    if (d != nullptr) d[j] = 0.0f;
  }
}

// Dropout as the forward applies it (fwp_st.cpp:4830-4883): kind 0 none,
// 1 plain Bernoulli (mask ? v : 0), 2 inverted (mask ? v*scale : 0).
__device__ __forceinline__ float drop_apply(int kind, uint8_t m, float scale, float v) {
  if (kind == 0) return v;
  if (kind == 1) return m ? v : 0.0f;
  return m ? v * scale : 0.0f;
}

struct FwdApplyArgs {
  float const *x, *gamma, *beta, *mean, *stdv, *r, *d;
  uint8_t const *mask;
  float *y;     // activation output after dropout (may be null)
  float *xhat;  // optional materialised x_hat
  float *nrm;   // optional materialised gamma*x_hat + beta
  size_t B, H, rows_per_chunk;
  int tx_log2, drop_kind, mask_per_element;
  float drop_scale;
};

// Phase 3 of fwp_st.cpp:4748-4765, then AF_FIRE (fwp_st.cpp:4768-4794), then the
// dropout leaf, in one pass.
template <int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void k_fwd_apply(FwdApplyArgs a) {
  int const TX = 1 << a.tx_log2, TY = kBlock >> a.tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> a.tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  if (col >= a.H) return;
  size_t const b0 = blockIdx.y * a.rows_per_chunk;
  size_t const b1 = (b0 + a.rows_per_chunk < a.B) ? b0 + a.rows_per_chunk : a.B;
  float mu[VEC], inv[VEC], rr[VEC], dd[VEC], ga[VEC], be[VEC];
  uint8_t mk[VEC];
  load_f<VEC>(a.mean + col, mu);
  load_f<VEC>(a.stdv + col, inv);
  load_f<VEC>(a.r + col, rr);
  load_f<VEC>(a.d + col, dd);
  load_f<VEC>(a.gamma + col, ga);
  load_f<VEC>(a.beta + col, be);
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    inv[i] = 1.0f / inv[i];
    mk[i] = 1;
  }
  if (a.drop_kind != 0 && !a.mask_per_element) load_u8<VEC>(a.mask + col, mk);
  constexpr int U = 4;
  size_t b = b0 + ty;
  auto body = [&](size_t row, float const (&xv)[VEC], uint8_t const (&mv)[VEC]) {
    float xh[VEC], nn[VEC], q[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      xh[i] = (xv[i] - mu[i]) * inv[i] * rr[i] + dd[i];
      nn[i] = ga[i] * xh[i] + be[i];
      q[i] = drop_apply(a.drop_kind, mv[i], a.drop_scale, act_fire<ACT>(nn[i]));
    }
    if (a.xhat != nullptr) store_f<VEC>(a.xhat + row * a.H + col, xh);
    if (a.nrm != nullptr) store_f<VEC>(a.nrm + row * a.H + col, nn);
    if (a.y != nullptr) store_f<VEC>(a.y + row * a.H + col, q);
  };
  for (; b + (U - 1) * static_cast<size_t>(TY) < b1; b += U * static_cast<size_t>(TY)) {
    float xv[U][VEC];
    uint8_t mv[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      size_t const row = b + u * static_cast<size_t>(TY);
      load_f<VEC>(a.x + row * a.H + col, xv[u]);
      if (a.drop_kind != 0 && a.mask_per_element) {
        load_u8<VEC>(a.mask + row * a.H + col, mv[u]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mv[u][i] = mk[i];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) body(b + u * static_cast<size_t>(TY), xv[u], mv[u]);
  }
  for (; b < b1; b += TY) {
    float xv[VEC];
    uint8_t mv[VEC];
    load_f<VEC>(a.x + b * a.H + col, xv);
    if (a.drop_kind != 0 && a.mask_per_element) {
      load_u8<VEC>(a.mask + b * a.H + col, mv);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) mv[i] = mk[i];
    }
    body(b, xv, mv);
  }
}

// ---------------------------------------------------------------- backward
struct BwdArgs {
  float const *x, *gamma, *beta, *mean, *stdv, *r, *d;
  float const *xhat;  // only when XHAT_GIVEN (un-fused leaf: dn = dY, x_hat stored)
  uint8_t const *mask;
  float const *dY;
  float *partial;     // reduce: [3][nchunks][H]
  float const *coef;  // apply: [3][H]  c1 = gamma*r/std, c2 = dstd/(B*std), c3 = dmean/B
  float *dX;
  size_t B, H, rows_per_chunk;
  int tx_log2, drop_kind, mask_per_element, drop_bwd_masked;
  float drop_scale;
};

// dn = dY * f'(n, q) for one element, recomputing x_hat, n and q from x.
// REFERENCE dropout mode: q is the post-dropout output and dY is untouched
// (bwp_st.cpp:1177-1209 reads the array the dropout leaf overwrote in place);
// MASKED mode: q is the pre-dropout activation and dY is masked and rescaled.
template <int ACT, bool XHAT_GIVEN>
__device__ __forceinline__ float bwd_dn(BwdArgs const &a, float xv, float dy, uint8_t m, float mu, float inv,
                                        float rr, float dd, float ga, float be, float &xh) {
  if constexpr (XHAT_GIVEN) {
    (void)xv; (void)m; (void)mu; (void)inv; (void)rr; (void)dd; (void)ga; (void)be;
    return dy;
  } else {
    xh = (xv - mu) * inv * rr + dd;
    float const nn = ga * xh + be;
    float q = act_fire<ACT>(nn);
    float g = dy;
    if (a.drop_kind != 0) {
      if (a.drop_bwd_masked) {
        g = drop_apply(a.drop_kind, m, a.drop_scale, dy);
      } else {
        q = drop_apply(a.drop_kind, m, a.drop_scale, q);
      }
    }
    return g * act_derive<ACT>(nn, q);
  }
}

// Pass 1 of bwp_st.cpp:1478-1506: column sums of dn*x_hat, dn and dn*(x-mean).
// (dmean and dstd follow from the last two in the finalize kernel:
//  sum e*(-r/std) = -(r/std)*gamma*sum dn, sum e*(x-mean)*(-r/std^2) likewise.)
template <int VEC, int ACT, bool XHAT_GIVEN>
__global__ __launch_bounds__(kBlock) void k_bwd_reduce(BwdArgs a) {
  __shared__ float lds[4 * kWave * 3 * VEC];
  int const TX = 1 << a.tx_log2, TY = kBlock >> a.tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> a.tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  bool const live = col < a.H;
  size_t const b0 = blockIdx.y * a.rows_per_chunk;
  size_t const b1 = (b0 + a.rows_per_chunk < a.B) ? b0 + a.rows_per_chunk : a.B;
  float acc[3 * VEC];
#pragma unroll
  for (int i = 0; i < 3 * VEC; ++i) acc[i] = 0.0f;
  if (live) {
    float mu[VEC], inv[VEC], rr[VEC], dd[VEC], ga[VEC], be[VEC];
    uint8_t mk[VEC];
    load_f<VEC>(a.mean + col, mu);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      inv[i] = 1.0f; rr[i] = 1.0f; dd[i] = 0.0f; ga[i] = 1.0f; be[i] = 0.0f; mk[i] = 1;
    }
    if constexpr (!XHAT_GIVEN) {
      load_f<VEC>(a.stdv + col, inv);
      load_f<VEC>(a.r + col, rr);
      load_f<VEC>(a.d + col, dd);
      load_f<VEC>(a.gamma + col, ga);
      load_f<VEC>(a.beta + col, be);
#pragma unroll
      for (int i = 0; i < VEC; ++i) inv[i] = 1.0f / inv[i];
      if (a.drop_kind != 0 && !a.mask_per_element) load_u8<VEC>(a.mask + col, mk);
    }
    constexpr int U = 2;
    auto body = [&](float const (&xv)[VEC], float const (&dy)[VEC], float const (&xg)[VEC],
                    uint8_t const (&mv)[VEC]) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float xh = xg[i];
        float const dn = bwd_dn<ACT, XHAT_GIVEN>(a, xv[i], dy[i], mv[i], mu[i], inv[i], rr[i], dd[i], ga[i],
                                                 be[i], xh);
        acc[i] += dn * xh;
        acc[VEC + i] += dn;
        acc[2 * VEC + i] += dn * (xv[i] - mu[i]);
      }
    };
    size_t b = b0 + ty;
    for (; b + (U - 1) * static_cast<size_t>(TY) < b1; b += U * static_cast<size_t>(TY)) {
      float xv[U][VEC], dy[U][VEC], xg[U][VEC];
      uint8_t mv[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        size_t const off = (b + u * static_cast<size_t>(TY)) * a.H + col;
        load_f<VEC>(a.x + off, xv[u]);
        load_f<VEC>(a.dY + off, dy[u]);
        if constexpr (XHAT_GIVEN) {
          load_f<VEC>(a.xhat + off, xg[u]);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) xg[u][i] = 0.0f;
        }
        if (!XHAT_GIVEN && a.drop_kind != 0 && a.mask_per_element) {
          load_u8<VEC>(a.mask + off, mv[u]);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) mv[u][i] = mk[i];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) body(xv[u], dy[u], xg[u], mv[u]);
    }
    for (; b < b1; b += TY) {
      float xv[VEC], dy[VEC], xg[VEC];
      uint8_t mv[VEC];
      size_t const off = b * a.H + col;
      load_f<VEC>(a.x + off, xv);
      load_f<VEC>(a.dY + off, dy);
      if constexpr (XHAT_GIVEN) {
        load_f<VEC>(a.xhat + off, xg);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) xg[i] = 0.0f;
      }
      if (!XHAT_GIVEN && a.drop_kind != 0 && a.mask_per_element) {
        load_u8<VEC>(a.mask + off, mv);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mv[i] = mk[i];
      }
      body(xv, dy, xg, mv);
    }
  }
  block_rows_reduce<3 * VEC>(acc, TX, lds);
  if (threadIdx.x < TX && live) {
    size_t const nch = gridDim.y;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      a.partial[(0 * nch + blockIdx.y) * a.H + col + i] = acc[i];
      a.partial[(1 * nch + blockIdx.y) * a.H + col + i] = acc[VEC + i];
      a.partial[(2 * nch + blockIdx.y) * a.H + col + i] = acc[2 * VEC + i];
    }
  }
}

// dgamma += S0, dbeta += S1 (accumulating like the reference's derivative
// array), dmean, dstd, and the three per-unit coefficients of pass 2
// (bwp_st.cpp:1508-1531):  dx = e*(r/std) + dstd*((x-mean)/(B*std)) + dmean*(1/B).
__global__ __launch_bounds__(kBlock) void k_bwd_finalize(float const *__restrict__ partial, unsigned nchunks,
                                                          size_t B, size_t H, float const *__restrict__ gamma,
                                                          float const *__restrict__ stdv,
                                                          float const *__restrict__ r,
                                                          float *__restrict__ dgamma, float *__restrict__ dbeta,
                                                          float *__restrict__ dmean, float *__restrict__ dstd,
                                                          float *__restrict__ coef) {
  __shared__ float lds[kBlock * 3];
  float tot[3];
  chunk_totals<3>(partial, nchunks, H, tot, lds);
  size_t const j = static_cast<size_t>(blockIdx.x) * kFinCols + threadIdx.x;
  if (threadIdx.x >= kWave || j >= H) return;
  float const s0 = tot[0], s1 = tot[1], s2 = tot[2];
  float const sd = stdv[j];
  float const rr = r != nullptr ? r[j] : 1.0f;
  float const ga = gamma[j];
  dgamma[j] += s0;
  dbeta[j] += s1;
  float const dm = (ga * s1) * (-rr / sd);
  float const ds = (ga * s2) * (-rr / (sd * sd));
  if (dmean != nullptr) dmean[j] = dm;
  if (dstd != nullptr) dstd[j] = ds;
  float const batch_scale = 1.0f / static_cast<float>(B);
  coef[0 * H + j] = ga * (rr / sd);
  coef[1 * H + j] = ds / (static_cast<float>(B) * sd);
  coef[2 * H + j] = dm * batch_scale;
}

template <int VEC, int ACT, bool XHAT_GIVEN>
__global__ __launch_bounds__(kBlock) void k_bwd_apply(BwdArgs a) {
  int const TX = 1 << a.tx_log2, TY = kBlock >> a.tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> a.tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  if (col >= a.H) return;
  size_t const b0 = blockIdx.y * a.rows_per_chunk;
  size_t const b1 = (b0 + a.rows_per_chunk < a.B) ? b0 + a.rows_per_chunk : a.B;
  float mu[VEC], inv[VEC], rr[VEC], dd[VEC], ga[VEC], be[VEC], c1[VEC], c2[VEC], c3[VEC];
  uint8_t mk[VEC];
  load_f<VEC>(a.mean + col, mu);
  load_f<VEC>(a.coef + 0 * a.H + col, c1);
  load_f<VEC>(a.coef + 1 * a.H + col, c2);
  load_f<VEC>(a.coef + 2 * a.H + col, c3);
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    inv[i] = 1.0f; rr[i] = 1.0f; dd[i] = 0.0f; ga[i] = 1.0f; be[i] = 0.0f; mk[i] = 1;
  }
  if constexpr (!XHAT_GIVEN) {
    load_f<VEC>(a.stdv + col, inv);
    load_f<VEC>(a.r + col, rr);
    load_f<VEC>(a.d + col, dd);
    load_f<VEC>(a.gamma + col, ga);
    load_f<VEC>(a.beta + col, be);
#pragma unroll
    for (int i = 0; i < VEC; ++i) inv[i] = 1.0f / inv[i];
    if (a.drop_kind != 0 && !a.mask_per_element) load_u8<VEC>(a.mask + col, mk);
  }
  constexpr int U = 2;
  auto body = [&](size_t off, float const (&xv)[VEC], float const (&dy)[VEC], uint8_t const (&mv)[VEC]) {
    float dx[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float xh = 0.0f;
      float const dn = bwd_dn<ACT, XHAT_GIVEN>(a, xv[i], dy[i], mv[i], mu[i], inv[i], rr[i], dd[i], ga[i],
                                               be[i], xh);
      dx[i] = dn * c1[i] + (xv[i] - mu[i]) * c2[i] + c3[i];
    }
    store_f<VEC>(a.dX + off, dx);
  };
  size_t b = b0 + ty;
  for (; b + (U - 1) * static_cast<size_t>(TY) < b1; b += U * static_cast<size_t>(TY)) {
    float xv[U][VEC], dy[U][VEC];
    uint8_t mv[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      size_t const off = (b + u * static_cast<size_t>(TY)) * a.H + col;
      load_f<VEC>(a.x + off, xv[u]);
      load_f<VEC>(a.dY + off, dy[u]);
      if (!XHAT_GIVEN && a.drop_kind != 0 && a.mask_per_element) {
        load_u8<VEC>(a.mask + off, mv[u]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mv[u][i] = mk[i];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) body((b + u * static_cast<size_t>(TY)) * a.H + col, xv[u], dy[u], mv[u]);
  }
  for (; b < b1; b += TY) {
    float xv[VEC], dy[VEC];
    uint8_t mv[VEC];
    size_t const off = b * a.H + col;
    load_f<VEC>(a.x + off, xv);
    load_f<VEC>(a.dY + off, dy);
    if (!XHAT_GIVEN && a.drop_kind != 0 && a.mask_per_element) {
      load_u8<VEC>(a.mask + off, mv);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) mv[i] = mk[i];
    }
    body(off, xv, dy, mv);
  }
}

// ---------------------------------------------------------------- host drivers
static int drop_kind_of(dlmi_dropout d) {
  return d == DLMI_DROP_BERNOULLI ? 1 : (d == DLMI_DROP_BERNOULLI_INVERTED ? 2 : 0);
}

static bool use_vec4(size_t H, std::initializer_list<void const *> ptrs) {
  if (H % 4 != 0) return false;
  for (void const *p : ptrs)
    if (p != nullptr && !dlmi_aligned16(p)) return false;
  return true;
}

struct FwdTrainCall {
  dlmi_norm norm;
  int act;
  int drop_kind, mask_per_element;
  float momentum, eps, r_max, d_max, drop_scale;
  float const *x, *gamma, *beta;
  uint8_t const *mask;
  float *mean, *stdv, *mov_mean, *mov_std, *r, *d, *y, *xhat, *nrm;
};

static int run_fwd_train(dlmi_ctx *ctx, size_t B, size_t H, FwdTrainCall const &c) {
  bool const vec4 = use_vec4(H, {c.x, c.gamma, c.beta, c.mean, c.stdv, c.r, c.d, c.y, c.xhat, c.nrm}) &&
                    (c.drop_kind == 0 || (reinterpret_cast<uintptr_t>(c.mask) & 3u) == 0);
  ColGeom const g = col_geometry(ctx, B, H, vec4, 2);
  float *partial = reinterpret_cast<float *>(ctx->scratch);
  dim3 const grid(g.grid_x, g.nchunks), block(kBlock);
  if (vec4)
    hipLaunchKernelGGL(k_col_stats<4>, grid, block, 0, ctx->stream, c.x, B, H, g.tx_log2, g.rows_per_chunk, partial);
  else
    hipLaunchKernelGGL(k_col_stats<1>, grid, block, 0, ctx->stream, c.x, B, H, g.tx_log2, g.rows_per_chunk, partial);
  DLMI_LAUNCH_CHECK(ctx, "k_col_stats");
  hipLaunchKernelGGL(k_fwd_finalize, dim3(static_cast<unsigned>(dlmi_ceil_div(H, kFinCols))), block, 0, ctx->stream,
                     partial, g.nchunks, B, H, c.norm == DLMI_NORM_BATCH_RENORM ? 1 : 0, c.momentum, c.eps,
                     c.r_max, c.d_max, c.mean, c.stdv, c.mov_mean, c.mov_std, c.r, c.d);
  DLMI_LAUNCH_CHECK(ctx, "k_fwd_finalize");
  FwdApplyArgs a;
  a.x = c.x; a.gamma = c.gamma; a.beta = c.beta; a.mean = c.mean; a.stdv = c.stdv; a.r = c.r; a.d = c.d;
  a.mask = c.mask; a.y = c.y; a.xhat = c.xhat; a.nrm = c.nrm;
  a.B = B; a.H = H; a.rows_per_chunk = g.rows_per_chunk; a.tx_log2 = g.tx_log2;
  a.drop_kind = c.drop_kind; a.mask_per_element = c.mask_per_element; a.drop_scale = c.drop_scale;
  DLMI_DISPATCH_ACT(c.act, {
    if (vec4)
      hipLaunchKernelGGL((k_fwd_apply<4, ACT>), grid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((k_fwd_apply<1, ACT>), grid, block, 0, ctx->stream, a);
  });
  DLMI_LAUNCH_CHECK(ctx, "k_fwd_apply");
  return DLMI_OK;
}

struct BwdCall {
  int act;
  bool xhat_given;
  int drop_kind, mask_per_element, drop_bwd_masked;
  float drop_scale;
  float const *x, *gamma, *beta, *mean, *stdv, *r, *d, *xhat, *dY;
  uint8_t const *mask;
  float *dgamma, *dbeta, *dmean, *dstd, *dX;
};

static int run_bwd(dlmi_ctx *ctx, size_t B, size_t H, BwdCall const &c) {
  bool const vec4 = use_vec4(H, {c.x, c.gamma, c.beta, c.mean, c.stdv, c.r, c.d, c.xhat, c.dY, c.dX}) &&
                    (c.drop_kind == 0 || (reinterpret_cast<uintptr_t>(c.mask) & 3u) == 0);
  ColGeom const g = col_geometry(ctx, B, H, vec4, 3);
  // scratch: first half partials [3][nchunks][H], second half coefficients [3][H]
  float *partial = reinterpret_cast<float *>(ctx->scratch);
  float *coef = reinterpret_cast<float *>(ctx->scratch + ctx->scratch_bytes / 2);
  BwdArgs a;
  a.x = c.x; a.gamma = c.gamma; a.beta = c.beta; a.mean = c.mean; a.stdv = c.stdv; a.r = c.r; a.d = c.d;
  a.xhat = c.xhat; a.mask = c.mask; a.dY = c.dY; a.partial = partial; a.coef = coef; a.dX = c.dX;
  a.B = B; a.H = H; a.rows_per_chunk = g.rows_per_chunk; a.tx_log2 = g.tx_log2;
  a.drop_kind = c.drop_kind; a.mask_per_element = c.mask_per_element; a.drop_bwd_masked = c.drop_bwd_masked;
  a.drop_scale = c.drop_scale;
  dim3 const grid(g.grid_x, g.nchunks), block(kBlock);
  if (c.xhat_given) {
    if (vec4)
      hipLaunchKernelGGL((k_bwd_reduce<4, DLMI_ACT_LINEAR, true>), grid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((k_bwd_reduce<1, DLMI_ACT_LINEAR, true>), grid, block, 0, ctx->stream, a);
  } else {
    DLMI_DISPATCH_ACT(c.act, {
      if (vec4)
        hipLaunchKernelGGL((k_bwd_reduce<4, ACT, false>), grid, block, 0, ctx->stream, a);
      else
        hipLaunchKernelGGL((k_bwd_reduce<1, ACT, false>), grid, block, 0, ctx->stream, a);
    });
  }
  DLMI_LAUNCH_CHECK(ctx, "k_bwd_reduce");
  hipLaunchKernelGGL(k_bwd_finalize, dim3(static_cast<unsigned>(dlmi_ceil_div(H, kFinCols))), block, 0, ctx->stream,
                     partial, g.nchunks, B, H, c.gamma, c.stdv, c.r, c.dgamma, c.dbeta, c.dmean, c.dstd, coef);
  DLMI_LAUNCH_CHECK(ctx, "k_bwd_finalize");
  if (c.xhat_given) {
    if (vec4)
      hipLaunchKernelGGL((k_bwd_apply<4, DLMI_ACT_LINEAR, true>), grid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((k_bwd_apply<1, DLMI_ACT_LINEAR, true>), grid, block, 0, ctx->stream, a);
  } else {
    DLMI_DISPATCH_ACT(c.act, {
      if (vec4)
        hipLaunchKernelGGL((k_bwd_apply<4, ACT, false>), grid, block, 0, ctx->stream, a);
      else
        hipLaunchKernelGGL((k_bwd_apply<1, ACT, false>), grid, block, 0, ctx->stream, a);
    });
  }
  DLMI_LAUNCH_CHECK(ctx, "k_bwd_apply");
  return DLMI_OK;
}

static int check_desc(dlmi_ctx *ctx, dlmi_fused_desc const *desc, uint8_t const *mask) {
  if (desc->norm != DLMI_NORM_BATCH && desc->norm != DLMI_NORM_BATCH_RENORM)
    return dlmi_fail(ctx, DLMI_E_INVALID, "fused path needs batch normalization or renormalization");
  if (!act_supported(desc->act)) return dlmi_fail(ctx, DLMI_E_INVALID, "unsupported activation %d", desc->act);
  if (desc->dropout != DLMI_DROP_NONE && desc->dropout != DLMI_DROP_BERNOULLI &&
      desc->dropout != DLMI_DROP_BERNOULLI_INVERTED)
    return dlmi_fail(ctx, DLMI_E_INVALID, "unsupported dropout %d", desc->dropout);
  if (desc->dropout != DLMI_DROP_NONE && mask == nullptr)
    return dlmi_fail(ctx, DLMI_E_INVALID, "dropout requested without a mask");
  return DLMI_OK;
}

}  // namespace dlmi

using namespace dlmi;

extern "C" {

int dlmi_norm_fwd_train(dlmi_ctx *ctx, dlmi_norm norm, size_t B, size_t H, float momentum, float eps,
                        float r_max, float d_max, float const *x, float const *gamma, float const *beta,
                        float *mean, float *stdv, float *mov_mean, float *mov_std, float *r, float *d,
                        float *xhat, float *out) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, norm == DLMI_NORM_BATCH || norm == DLMI_NORM_BATCH_RENORM, "norm must be BATCH or BATCH_RENORM");
  DLMI_REQUIRE(ctx, B > 0 && H > 0, "empty tensor");
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && mov_mean && mov_std && r && d, "null pointer");
  FwdTrainCall c;
  c.norm = norm; c.act = DLMI_ACT_LINEAR; c.drop_kind = 0; c.mask_per_element = 0;
  c.momentum = momentum; c.eps = eps; c.r_max = r_max; c.d_max = d_max; c.drop_scale = 1.0f;
  c.x = x; c.gamma = gamma; c.beta = beta; c.mask = nullptr;
  c.mean = mean; c.stdv = stdv; c.mov_mean = mov_mean; c.mov_std = mov_std; c.r = r; c.d = d;
  c.y = nullptr; c.xhat = xhat; c.nrm = out;
  return run_fwd_train(ctx, B, H, c);
}

int dlmi_fused_norm_act_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                            float const *gamma, float const *beta, uint8_t const *mask, float *mean,
                            float *stdv, float *mov_mean, float *mov_std, float *r, float *d, float *y) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, B > 0 && H > 0, "empty tensor");
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && mov_mean && mov_std && r && d && y, "null pointer");
  FwdTrainCall c;
  c.norm = desc->norm; c.act = desc->act; c.drop_kind = drop_kind_of(desc->dropout);
  c.mask_per_element = desc->mask_per_element;
  c.momentum = desc->momentum; c.eps = desc->eps; c.r_max = desc->r_max; c.d_max = desc->d_max;
  c.drop_scale = desc->drop_scale;
  c.x = x; c.gamma = gamma; c.beta = beta; c.mask = mask;
  c.mean = mean; c.stdv = stdv; c.mov_mean = mov_mean; c.mov_std = mov_std; c.r = r; c.d = d;
  c.y = y; c.xhat = nullptr; c.nrm = nullptr;
  return run_fwd_train(ctx, B, H, c);
}

int dlmi_norm_bwd(dlmi_ctx *ctx, dlmi_norm norm, size_t B, size_t H, float const *mean, float const *stdv,
                  float const *gamma, float const *r, float const *x, float const *xhat, float const *dN,
                  float *dgamma, float *dbeta, float *dmean, float *dstd, float *dx) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, norm == DLMI_NORM_BATCH || norm == DLMI_NORM_BATCH_RENORM, "norm must be BATCH or BATCH_RENORM");
  DLMI_REQUIRE(ctx, B > 0 && H > 0, "empty tensor");
  DLMI_REQUIRE(ctx, mean && stdv && gamma && x && xhat && dN && dgamma && dbeta && dx, "null pointer");
  DLMI_REQUIRE(ctx, norm == DLMI_NORM_BATCH || r != nullptr, "renormalization needs r");
  BwdCall c;
  c.act = DLMI_ACT_LINEAR; c.xhat_given = true; c.drop_kind = 0; c.mask_per_element = 0; c.drop_bwd_masked = 0;
  c.drop_scale = 1.0f;
  c.x = x; c.gamma = gamma; c.beta = nullptr; c.mean = mean; c.stdv = stdv;
  c.r = norm == DLMI_NORM_BATCH_RENORM ? r : nullptr; c.d = nullptr; c.xhat = xhat; c.dY = dN; c.mask = nullptr;
  c.dgamma = dgamma; c.dbeta = dbeta; c.dmean = dmean; c.dstd = dstd; c.dX = dx;
  return run_bwd(ctx, B, H, c);
}

int dlmi_fused_norm_act_bwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                            float const *gamma, float const *beta, uint8_t const *mask, float const *mean,
                            float const *stdv, float const *r, float const *d, float const *dY, float *dgamma,
                            float *dbeta, float *dX) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, B > 0 && H > 0, "empty tensor");
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && r && d && dY && dgamma && dbeta && dX, "null pointer");
  BwdCall c;
  c.act = desc->act; c.xhat_given = false; c.drop_kind = drop_kind_of(desc->dropout);
  c.mask_per_element = desc->mask_per_element;
  c.drop_bwd_masked = desc->dropout_bwd == DLMI_DROP_BWD_MASKED ? 1 : 0;
  c.drop_scale = desc->drop_scale;
  c.x = x; c.gamma = gamma; c.beta = beta; c.mean = mean; c.stdv = stdv; c.r = r; c.d = d; c.xhat = nullptr;
  c.dY = dY; c.mask = mask;
  c.dgamma = dgamma; c.dbeta = dbeta; c.dmean = nullptr; c.dstd = nullptr; c.dX = dX;
  return run_bwd(ctx, B, H, c);
}

}  // extern "C"
