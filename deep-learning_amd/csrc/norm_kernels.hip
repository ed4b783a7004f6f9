// Batch normalization / batch renormalization kernels (training forward and
// backward, fused with the activation and the dropout mask) for gfx950.
//
// All of them are bound by HBM bandwidth, so the design goal is the minimum
// number of passes over the [B, H] tensors with fully coalesced 16-byte
// accesses, enough independent loads in flight per CU and few enough ALU
// instructions per element that the vector units never become the limit:
//
//   forward : stats (read x)            -> finalize [H] -> apply (read x, write y)
//   backward: reduce (read dY, x)       -> finalize [H] -> apply (read dY, x, write dX)
//
// x_hat, the pre-activation n = gamma*x_hat + beta and the activation output
// are recomputed in registers instead of being stored and re-read.
//
// Thread geometry of the column passes: a 256-thread block is TX x TY; a
// thread owns VEC (=4, one float4) adjacent units and walks the rows of its
// block's batch chunk with stride TY.  In the reduction kernels TX <= 64, so
// when H is small a wavefront spans several rows: those are combined with
// wavefront shuffles, the four wavefronts of the block with a small LDS tree,
// and the chunks of the batch by the finalize kernel in a fixed order (no float
// atomics: results are reproducible run to run).  The apply kernels have
// nothing to reduce and use TX = 256 when H allows, so that every load / store
// instruction of a block covers 4 KiB of one row.
//
// Everything that is uniform over a launch and would put a branch between two
// loads (dropout mode, materialising x_hat) is a template parameter: a branch
// there makes the compiler wait for each load before issuing the next.
//
// Citations: /root/reference/lib/deep-learning/v1/learner/.
#include <cstdlib>
#include <initializer_list>

#include "activations.hpp"
#include "dlmi_common.hpp"

namespace dlmi {

constexpr int kBlock = 256;
constexpr int kWave = 64;

// rows in flight per thread in the reduction passes
#ifndef DLMI_STATS_U
#define DLMI_STATS_U 8
#endif
#ifndef DLMI_BWD_REDUCE_U
#define DLMI_BWD_REDUCE_U 4
#endif

// dropout as a template mode
constexpr int kDropNone = 0, kDropUnit = 1, kDropElem = 2;

struct ColGeom {
  int vec;  // 4 (float4 path) or 1 (any H, any alignment)
  int tx_log2;
  unsigned grid_x;
  unsigned nchunks;
  size_t rows_per_chunk;
};

// Tuning aids: DLMI_NORM_{STATS,BWD}_TX (64, 128 or 256), .._ROWS_PER_THREAD and
// .._BLOCKS_PER_CU override the geometry of the two reduction passes,
// DLMI_NORM_APPLY_ROWS_PER_THREAD that of the apply passes.
static int env_int(char const *name, int dflt) {
  char const *e = getenv(name);
  if (e == nullptr || *e == 0) return dflt;
  int const v = atoi(e);
  return v > 0 ? v : dflt;
}

// Geometry of a reduction pass.
static ColGeom reduce_geometry(dlmi_ctx const *ctx, size_t B, size_t H, bool vec4, int nacc) {
  static int const tx_caps[2] = {env_int("DLMI_NORM_STATS_TX", 64), env_int("DLMI_NORM_BWD_TX", 256)};
  static int const rpts[2] = {env_int("DLMI_NORM_STATS_ROWS_PER_THREAD", 16), env_int("DLMI_NORM_BWD_ROWS_PER_THREAD", 8)};
  static int const bpcs[2] = {env_int("DLMI_NORM_STATS_BLOCKS_PER_CU", 8), env_int("DLMI_NORM_BWD_BLOCKS_PER_CU", 1)};
  int const which = nacc == 2 ? 0 : 1;
  int const tx_cap = tx_caps[which], rows_per_thread = rpts[which], blocks_per_cu = bpcs[which];
  ColGeom g;
  g.vec = vec4 ? 4 : 1;
  size_t const groups = dlmi_ceil_div(H, g.vec);
  int tx = tx_cap >= 256 ? 256 : (tx_cap >= 128 ? 128 : 64);
  g.tx_log2 = tx == 256 ? 8 : (tx == 128 ? 7 : 6);
  while (tx > 1 && static_cast<size_t>(tx / 2) >= groups) {
    tx /= 2;
    --g.tx_log2;
  }
  int const ty = kBlock / tx;
  g.grid_x = static_cast<unsigned>(dlmi_ceil_div(groups, tx));
  // enough blocks to cover every CU several times over, but each thread still
  // streams rows_per_thread rows (16 in the statistics pass, 8 in the backward
  // reduction, where a batch of 1024 rows otherwise leaves half the CUs idle):
  // the partial sums stay a small fraction of the traffic and the fixed cost of
  // a block is amortised
  size_t want = dlmi_ceil_div(static_cast<size_t>(ctx->num_cu) * blocks_per_cu, g.grid_x);
  size_t const max_by_rows = B / (static_cast<size_t>(ty) * rows_per_thread);
  if (want > max_by_rows) want = max_by_rows;
  // partial sums must fit half of the scratch block: nacc * nchunks * H floats
  size_t const max_by_scratch = (ctx->scratch_bytes / 2) / (static_cast<size_t>(nacc) * H * sizeof(float));
  if (want > max_by_scratch) want = max_by_scratch;
  if (want < 1) want = 1;
  if (want > 65535) want = 65535;
  g.rows_per_chunk = dlmi_ceil_div(B, want);
  g.nchunks = static_cast<unsigned>(dlmi_ceil_div(B, g.rows_per_chunk));
  return g;
}

// Geometry of an apply pass: as wide as the row allows (TX up to 256), 8 rows
// per thread.
static ColGeom apply_geometry(size_t B, size_t H, bool vec4) {
  ColGeom g;
  g.vec = vec4 ? 4 : 1;
  size_t const groups = dlmi_ceil_div(H, g.vec);
  int tx = 256;
  g.tx_log2 = 8;
  while (tx > 1 && static_cast<size_t>(tx / 2) >= groups) {
    tx /= 2;
    --g.tx_log2;
  }
  int const ty = kBlock / tx;
  g.grid_x = static_cast<unsigned>(dlmi_ceil_div(groups, tx));
  static int const rows_per_thread = env_int("DLMI_NORM_APPLY_ROWS_PER_THREAD", 8);
  g.rows_per_chunk = static_cast<size_t>(ty) * rows_per_thread;
  size_t chunks = dlmi_ceil_div(B, g.rows_per_chunk);
  if (chunks > 65535) {
    chunks = 65535;
    g.rows_per_chunk = dlmi_ceil_div(B, chunks);
    chunks = dlmi_ceil_div(B, g.rows_per_chunk);
  }
  g.nchunks = static_cast<unsigned>(chunks);
  return g;
}

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
// TX < 64: rows that share a wavefront are combined with shuffles first, then
// the four wavefronts through LDS; TX >= 64: the 256/TX rows through LDS.
template <int NV>
__device__ __forceinline__ void block_rows_reduce(float (&v)[NV], int tx, float *lds) {
  int const lane = threadIdx.x & (kWave - 1);
  int const wave = threadIdx.x / kWave;
  // rows that share a wavefront: lanes tx apart hold the same column group
  for (int off = tx; off < kWave; off <<= 1) {
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] += __shfl_xor(v[i], off, kWave);
  }
  int const nrows = tx < kWave ? kBlock / kWave : kBlock / tx;
  if (nrows == 1) return;
  int const row = tx < kWave ? wave : static_cast<int>(threadIdx.x) / tx;
  int const cg = tx < kWave ? lane : static_cast<int>(threadIdx.x) & (tx - 1);
  if (tx >= kWave || lane < tx) {
#pragma unroll
    for (int i = 0; i < NV; ++i) lds[(row * tx + cg) * NV + i] = v[i];
  }
  __syncthreads();
  // fixed order: (0+1) + (2+3) for four rows, 0+1 for two
  if (static_cast<int>(threadIdx.x) < tx) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      float s = lds[(0 * tx + cg) * NV + i] + lds[(1 * tx + cg) * NV + i];
      if (nrows == 4) s += lds[(2 * tx + cg) * NV + i] + lds[(3 * tx + cg) * NV + i];
      v[i] = s;
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
    constexpr int U = DLMI_STATS_U;
    size_t b = b0 + ty;
    for (; b + (U - 1) * static_cast<size_t>(TY) < b1; b += U * static_cast<size_t>(TY)) {
      float v[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) load_f<VEC>(x + (b + u * static_cast<size_t>(TY)) * H + col, v[u]);
#pragma unroll
      for (int u = 0; u < U; ++u)
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

// Sums NA partial-sum planes over the batch chunks for 16 adjacent units per
// block: thread (lane c of 16, unit j of 16) adds chunks c, c+16, c+32, ... with
// independent loads, then the 16 lane totals of a unit are combined through
// LDS in a fixed order.  On return thread t < 16 holds the totals of unit
// blockIdx.x*16 + t.
constexpr int kFinCols = 16;
constexpr int kFinLanes = kBlock / kFinCols;
template <int NA>
__device__ __forceinline__ void chunk_totals(float const *__restrict__ partial, unsigned nchunks, size_t H,
                                             float (&tot)[NA], float *lds) {
  int const cj = threadIdx.x % kFinCols;
  int const cl = threadIdx.x / kFinCols;
  size_t const j = static_cast<size_t>(blockIdx.x) * kFinCols + cj;
#pragma unroll
  for (int a = 0; a < NA; ++a) tot[a] = 0.0f;
  if (j < H) {
#pragma unroll 4
    for (unsigned c = cl; c < nchunks; c += kFinLanes) {
#pragma unroll
      for (int a = 0; a < NA; ++a) tot[a] += partial[(a * static_cast<size_t>(nchunks) + c) * H + j];
    }
  }
#pragma unroll
  for (int a = 0; a < NA; ++a) lds[(cl * kFinCols + cj) * NA + a] = tot[a];
  __syncthreads();
  if (threadIdx.x < kFinCols) {
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      float s = 0.0f;
#pragma unroll
      for (int l = 0; l < kFinLanes; ++l) s += lds[(l * kFinCols + threadIdx.x) * NA + a];
      tot[a] = s;
    }
  }
}

// Phase 2 of fwp_st.cpp:4709-4746: batch mean, moving mean, batch std, moving
// std, then r and d from the UPDATED moving statistics.
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
  if (threadIdx.x >= kFinCols || j >= H) return;
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

// Dropout as the forward applies it (fwp_st.cpp:4830-4883): mask ? v*scale : 0
// with scale = 1 for plain Bernoulli, 1/keep for inverted Bernoulli.
__device__ __forceinline__ float drop_apply(uint8_t m, float scale, float v) { return m ? v * scale : 0.0f; }

struct FwdApplyArgs {
  float const *x, *gamma, *beta, *mean, *stdv, *r, *d;
  uint8_t const *mask;
  float *y;     // activation output after dropout
  float *xhat;  // optional materialised x_hat            (MAT only)
  float *nrm;   // optional materialised gamma*x_hat+beta (MAT only)
  size_t B, H, rows_per_chunk;
  int tx_log2;
  float drop_scale;
};

// Phase 3 of fwp_st.cpp:4748-4765, then AF_FIRE (fwp_st.cpp:4768-4794), then the
// dropout leaf, in one pass.
// MAT: materialise x_hat / the pre-activation (the un-fused leaf) with the
// reference's expression order.  Otherwise the per-unit constants are folded so
// that an element costs one subtraction and one fused multiply-add before the
// activation:  n = (x - mean) * (gamma*r/std) + (gamma*d + beta).
template <int VEC, int ACT, int DROPM, bool MAT>
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
    inv[i] = fast_rcp(inv[i]);
    mk[i] = 1;
    if constexpr (!MAT) {
      rr[i] = ga[i] * (rr[i] * inv[i]);  // gamma * r / std
      dd[i] = ga[i] * dd[i] + be[i];     // gamma * d + beta
    }
  }
  if constexpr (DROPM == kDropUnit) load_u8<VEC>(a.mask + col, mk);
  constexpr int U = 4;
  auto body = [&](size_t off, float const (&xv)[VEC], uint8_t const (&mv)[VEC]) {
    float xh[VEC], nn[VEC], q[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      if constexpr (MAT) {
        xh[i] = (xv[i] - mu[i]) * inv[i] * rr[i] + dd[i];
        nn[i] = ga[i] * xh[i] + be[i];
      } else {
        nn[i] = (xv[i] - mu[i]) * rr[i] + dd[i];
      }
      q[i] = act_fire<ACT>(nn[i]);
      if constexpr (DROPM != kDropNone) q[i] = drop_apply(mv[i], a.drop_scale, q[i]);
    }
    if constexpr (MAT) {
      if (a.xhat != nullptr) store_f<VEC>(a.xhat + off, xh);
      if (a.nrm != nullptr) store_f<VEC>(a.nrm + off, nn);
      if (a.y != nullptr) store_f<VEC>(a.y + off, q);
    } else {
      store_f<VEC>(a.y + off, q);
    }
  };
  size_t b = b0 + ty;
  for (; b + (U - 1) * static_cast<size_t>(TY) < b1; b += U * static_cast<size_t>(TY)) {
    float xv[U][VEC];
    uint8_t mv[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      size_t const off = (b + u * static_cast<size_t>(TY)) * a.H + col;
      load_f<VEC>(a.x + off, xv[u]);
      if constexpr (DROPM == kDropElem) {
        load_u8<VEC>(a.mask + off, mv[u]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mv[u][i] = mk[i];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) body((b + u * static_cast<size_t>(TY)) * a.H + col, xv[u], mv[u]);
  }
  for (; b < b1; b += TY) {
    float xv[VEC];
    uint8_t mv[VEC];
    size_t const off = b * a.H + col;
    load_f<VEC>(a.x + off, xv);
    if constexpr (DROPM == kDropElem) {
      load_u8<VEC>(a.mask + off, mv);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) mv[i] = mk[i];
    }
    body(off, xv, mv);
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
  int tx_log2, drop_bwd_masked;
  float drop_scale;
};

// Per-unit constants of the backward recompute, loaded once per thread.
template <int VEC>
struct UnitConsts {
  float mu[VEC], rs[VEC], dd[VEC], ga[VEC], be[VEC];  // rs = r / std
  uint8_t mk[VEC];
};

template <int VEC, int DROPM, bool XHAT_GIVEN>
__device__ __forceinline__ void load_unit_consts(BwdArgs const &a, size_t col, UnitConsts<VEC> &u) {
  load_f<VEC>(a.mean + col, u.mu);
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    u.rs[i] = 1.0f; u.dd[i] = 0.0f; u.ga[i] = 1.0f; u.be[i] = 0.0f; u.mk[i] = 1;
  }
  if constexpr (!XHAT_GIVEN) {
    float sd[VEC], rr[VEC];
    load_f<VEC>(a.stdv + col, sd);
    load_f<VEC>(a.r + col, rr);
    load_f<VEC>(a.d + col, u.dd);
    load_f<VEC>(a.gamma + col, u.ga);
    load_f<VEC>(a.beta + col, u.be);
#pragma unroll
    for (int i = 0; i < VEC; ++i) u.rs[i] = rr[i] * fast_rcp(sd[i]);
    if constexpr (DROPM == kDropUnit) load_u8<VEC>(a.mask + col, u.mk);
  }
}

// dn = dY * f'(n, q) for one element, recomputing x_hat, n and q from x.
// REFERENCE dropout mode: q is the post-dropout output and dY is untouched
// (bwp_st.cpp:1177-1209 reads the array the dropout leaf overwrote in place);
// MASKED mode: q is the pre-dropout activation and dY is masked and rescaled.
template <int ACT, int DROPM, bool XHAT_GIVEN>
__device__ __forceinline__ float bwd_dn(BwdArgs const &a, float xv, float dy, uint8_t m, float mu, float rs,
                                        float dd, float ga, float be, float &xh) {
  if constexpr (XHAT_GIVEN) {
    (void)a; (void)xv; (void)m; (void)mu; (void)rs; (void)dd; (void)ga; (void)be;
    return dy;
  } else {
    xh = (xv - mu) * rs + dd;
    float const nn = ga * xh + be;
    float q = act_fire<ACT>(nn);
    float g = dy;
    if constexpr (DROPM != kDropNone) {
      float const gm = drop_apply(m, a.drop_scale, dy);
      float const qm = drop_apply(m, a.drop_scale, q);
      g = a.drop_bwd_masked ? gm : dy;
      q = a.drop_bwd_masked ? q : qm;
    }
    return g * act_derive<ACT>(nn, q);
  }
}

// Pass 1 of bwp_st.cpp:1478-1506: column sums of dn*x_hat, dn and dn*(x-mean).
// (dmean and dstd follow from the last two in the finalize kernel:
//  sum e*(-r/std) = -(r/std)*gamma*sum dn, sum e*(x-mean)*(-r/std^2) likewise.)
template <int VEC, int ACT, int DROPM, bool XHAT_GIVEN>
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
    UnitConsts<VEC> uc;
    load_unit_consts<VEC, DROPM, XHAT_GIVEN>(a, col, uc);
    constexpr int U = DLMI_BWD_REDUCE_U;
    auto body = [&](float const (&xv)[VEC], float const (&dy)[VEC], float const (&xg)[VEC],
                    uint8_t const (&mv)[VEC]) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float xh = xg[i];
        float const dn = bwd_dn<ACT, DROPM, XHAT_GIVEN>(a, xv[i], dy[i], mv[i], uc.mu[i], uc.rs[i], uc.dd[i],
                                                        uc.ga[i], uc.be[i], xh);
        acc[i] += dn * xh;
        acc[VEC + i] += dn;
        acc[2 * VEC + i] += dn * (xv[i] - uc.mu[i]);
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
        if constexpr (DROPM == kDropElem) {
          load_u8<VEC>(a.mask + off, mv[u]);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) mv[u][i] = uc.mk[i];
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
      if constexpr (DROPM == kDropElem) {
        load_u8<VEC>(a.mask + off, mv);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mv[i] = uc.mk[i];
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
  if (threadIdx.x >= kFinCols || j >= H) return;
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

template <int VEC, int ACT, int DROPM, bool XHAT_GIVEN>
__global__ __launch_bounds__(kBlock) void k_bwd_apply(BwdArgs a) {
  int const TX = 1 << a.tx_log2, TY = kBlock >> a.tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> a.tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  if (col >= a.H) return;
  size_t const b0 = blockIdx.y * a.rows_per_chunk;
  size_t const b1 = (b0 + a.rows_per_chunk < a.B) ? b0 + a.rows_per_chunk : a.B;
  UnitConsts<VEC> uc;
  load_unit_consts<VEC, DROPM, XHAT_GIVEN>(a, col, uc);
  float c1[VEC], c2[VEC], c3[VEC];
  load_f<VEC>(a.coef + 0 * a.H + col, c1);
  load_f<VEC>(a.coef + 1 * a.H + col, c2);
  load_f<VEC>(a.coef + 2 * a.H + col, c3);
  constexpr int U = 4;
  auto body = [&](size_t off, float const (&xv)[VEC], float const (&dy)[VEC], uint8_t const (&mv)[VEC]) {
    float dx[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float xh = 0.0f;
      float const dn = bwd_dn<ACT, DROPM, XHAT_GIVEN>(a, xv[i], dy[i], mv[i], uc.mu[i], uc.rs[i], uc.dd[i], uc.ga[i],
                                                      uc.be[i], xh);
      dx[i] = dn * c1[i] + (xv[i] - uc.mu[i]) * c2[i] + c3[i];
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
      if constexpr (DROPM == kDropElem) {
        load_u8<VEC>(a.mask + off, mv[u]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mv[u][i] = uc.mk[i];
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
    if constexpr (DROPM == kDropElem) {
      load_u8<VEC>(a.mask + off, mv);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) mv[i] = uc.mk[i];
    }
    body(off, xv, dy, mv);
  }
}

// ---------------------------------------------------------------- host drivers
static bool use_vec4(size_t H, std::initializer_list<void const *> ptrs) {
  if (H % 4 != 0) return false;
  for (void const *p : ptrs)
    if (p != nullptr && !dlmi_aligned16(p)) return false;
  return true;
}

// Runs f.template operator()<DROPM>() for the runtime dropout mode.
#define DLMI_DISPATCH_DROP(mode, ...)                                         \
  switch (mode) {                                                             \
    case kDropUnit: { constexpr int DROPM = kDropUnit; __VA_ARGS__; } break;  \
    case kDropElem: { constexpr int DROPM = kDropElem; __VA_ARGS__; } break;  \
    default: { constexpr int DROPM = kDropNone; __VA_ARGS__; } break;         \
  }

struct FwdTrainCall {
  dlmi_norm norm;
  int act;
  int drop_mode;  // kDropNone / kDropUnit / kDropElem
  float momentum, eps, r_max, d_max, drop_scale;
  float const *x, *gamma, *beta;
  uint8_t const *mask;
  float *mean, *stdv, *mov_mean, *mov_std, *r, *d, *y, *xhat, *nrm;
  float const *partial_in = nullptr;  // column-sum partials already produced elsewhere ...
  unsigned partial_chunks = 0;        // ... [2][partial_chunks][H]; skips the statistics pass
};

static int run_fwd_train(dlmi_ctx *ctx, size_t B, size_t H, FwdTrainCall const &c) {
  int rc = dlmi_scratch_reserve(ctx, 2 * 16 * 2 * H * sizeof(float));
  if (rc != DLMI_OK) return rc;
  bool const vec4 = use_vec4(H, {c.x, c.gamma, c.beta, c.mean, c.stdv, c.r, c.d, c.y, c.xhat, c.nrm}) &&
                    (c.drop_mode == kDropNone || (reinterpret_cast<uintptr_t>(c.mask) & 3u) == 0);
  dim3 const block(kBlock);
  float const *partial = c.partial_in;
  unsigned nchunks = c.partial_chunks;
  if (partial == nullptr) {
    ColGeom const g = reduce_geometry(ctx, B, H, vec4, 2);
    float *pw = reinterpret_cast<float *>(ctx->scratch);
    dim3 const grid(g.grid_x, g.nchunks);
    if (vec4)
      hipLaunchKernelGGL(k_col_stats<4>, grid, block, 0, ctx->stream, c.x, B, H, g.tx_log2, g.rows_per_chunk, pw);
    else
      hipLaunchKernelGGL(k_col_stats<1>, grid, block, 0, ctx->stream, c.x, B, H, g.tx_log2, g.rows_per_chunk, pw);
    DLMI_LAUNCH_CHECK(ctx, "k_col_stats");
    partial = pw;
    nchunks = g.nchunks;
  }
  hipLaunchKernelGGL(k_fwd_finalize, dim3(static_cast<unsigned>(dlmi_ceil_div(H, kFinCols))), block, 0, ctx->stream,
                     partial, nchunks, B, H, c.norm == DLMI_NORM_BATCH_RENORM ? 1 : 0, c.momentum, c.eps,
                     c.r_max, c.d_max, c.mean, c.stdv, c.mov_mean, c.mov_std, c.r, c.d);
  DLMI_LAUNCH_CHECK(ctx, "k_fwd_finalize");
  ColGeom const ga = apply_geometry(B, H, vec4);
  FwdApplyArgs a;
  a.x = c.x; a.gamma = c.gamma; a.beta = c.beta; a.mean = c.mean; a.stdv = c.stdv; a.r = c.r; a.d = c.d;
  a.mask = c.mask; a.y = c.y; a.xhat = c.xhat; a.nrm = c.nrm;
  a.B = B; a.H = H; a.rows_per_chunk = ga.rows_per_chunk; a.tx_log2 = ga.tx_log2; a.drop_scale = c.drop_scale;
  dim3 const agrid(ga.grid_x, ga.nchunks);
  if (c.xhat != nullptr || c.nrm != nullptr) {  // un-fused leaf: LINEAR, no dropout by construction
    if (vec4)
      hipLaunchKernelGGL((k_fwd_apply<4, DLMI_ACT_LINEAR, kDropNone, true>), agrid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((k_fwd_apply<1, DLMI_ACT_LINEAR, kDropNone, true>), agrid, block, 0, ctx->stream, a);
  } else if (c.y != nullptr) {
    DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_DROP(c.drop_mode, {
      if (vec4)
        hipLaunchKernelGGL((k_fwd_apply<4, ACT, DROPM, false>), agrid, block, 0, ctx->stream, a);
      else
        hipLaunchKernelGGL((k_fwd_apply<1, ACT, DROPM, false>), agrid, block, 0, ctx->stream, a);
    }));
  }
  DLMI_LAUNCH_CHECK(ctx, "k_fwd_apply");
  return DLMI_OK;
}

struct BwdCall {
  int act;
  bool xhat_given;
  int drop_mode, drop_bwd_masked;
  float drop_scale;
  float const *x, *gamma, *beta, *mean, *stdv, *r, *d, *xhat, *dY;
  uint8_t const *mask;
  float *dgamma, *dbeta, *dmean, *dstd, *dX;
};

static int run_bwd(dlmi_ctx *ctx, size_t B, size_t H, BwdCall const &c) {
  int rc = dlmi_scratch_reserve(ctx, 2 * 16 * 3 * H * sizeof(float));
  if (rc != DLMI_OK) return rc;
  bool const vec4 = use_vec4(H, {c.x, c.gamma, c.beta, c.mean, c.stdv, c.r, c.d, c.xhat, c.dY, c.dX}) &&
                    (c.drop_mode == kDropNone || (reinterpret_cast<uintptr_t>(c.mask) & 3u) == 0);
  ColGeom const g = reduce_geometry(ctx, B, H, vec4, 3);
  // scratch: first half partials [3][nchunks][H], second half coefficients [3][H]
  float *partial = reinterpret_cast<float *>(ctx->scratch);
  float *coef = reinterpret_cast<float *>(ctx->scratch + ctx->scratch_bytes / 2);
  BwdArgs a;
  a.x = c.x; a.gamma = c.gamma; a.beta = c.beta; a.mean = c.mean; a.stdv = c.stdv; a.r = c.r; a.d = c.d;
  a.xhat = c.xhat; a.mask = c.mask; a.dY = c.dY; a.partial = partial; a.coef = coef; a.dX = c.dX;
  a.B = B; a.H = H; a.rows_per_chunk = g.rows_per_chunk; a.tx_log2 = g.tx_log2;
  a.drop_bwd_masked = c.drop_bwd_masked; a.drop_scale = c.drop_scale;
  dim3 const grid(g.grid_x, g.nchunks), block(kBlock);
  if (c.xhat_given) {
    if (vec4)
      hipLaunchKernelGGL((k_bwd_reduce<4, DLMI_ACT_LINEAR, kDropNone, true>), grid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((k_bwd_reduce<1, DLMI_ACT_LINEAR, kDropNone, true>), grid, block, 0, ctx->stream, a);
  } else {
    DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_DROP(c.drop_mode, {
      if (vec4)
        hipLaunchKernelGGL((k_bwd_reduce<4, ACT, DROPM, false>), grid, block, 0, ctx->stream, a);
      else
        hipLaunchKernelGGL((k_bwd_reduce<1, ACT, DROPM, false>), grid, block, 0, ctx->stream, a);
    }));
  }
  DLMI_LAUNCH_CHECK(ctx, "k_bwd_reduce");
  hipLaunchKernelGGL(k_bwd_finalize, dim3(static_cast<unsigned>(dlmi_ceil_div(H, kFinCols))), block, 0, ctx->stream,
                     partial, g.nchunks, B, H, c.gamma, c.stdv, c.r, c.dgamma, c.dbeta, c.dmean, c.dstd, coef);
  DLMI_LAUNCH_CHECK(ctx, "k_bwd_finalize");
  ColGeom const ga = apply_geometry(B, H, vec4);
  a.rows_per_chunk = ga.rows_per_chunk;
  a.tx_log2 = ga.tx_log2;
  dim3 const agrid(ga.grid_x, ga.nchunks);
  if (c.xhat_given) {
    if (vec4)
      hipLaunchKernelGGL((k_bwd_apply<4, DLMI_ACT_LINEAR, kDropNone, true>), agrid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((k_bwd_apply<1, DLMI_ACT_LINEAR, kDropNone, true>), agrid, block, 0, ctx->stream, a);
  } else {
    DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_DROP(c.drop_mode, {
      if (vec4)
        hipLaunchKernelGGL((k_bwd_apply<4, ACT, DROPM, false>), agrid, block, 0, ctx->stream, a);
      else
        hipLaunchKernelGGL((k_bwd_apply<1, ACT, DROPM, false>), agrid, block, 0, ctx->stream, a);
    }));
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

static int drop_mode_of(dlmi_fused_desc const *desc) {
  if (desc->dropout == DLMI_DROP_NONE) return kDropNone;
  return desc->mask_per_element ? kDropElem : kDropUnit;
}
// plain Bernoulli keeps the value as it is (scale 1); inverted rescales by 1/keep
static float drop_scale_of(dlmi_fused_desc const *desc) {
  return desc->dropout == DLMI_DROP_BERNOULLI_INVERTED ? desc->drop_scale : 1.0f;
}

int fused_fwd_from_partials(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                            float const *gamma, float const *beta, uint8_t const *mask, float *mean, float *stdv,
                            float *mov_mean, float *mov_std, float *r, float *d, float *y, float const *partial,
                            unsigned nchunks) {
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && mov_mean && mov_std && r && d && y, "null pointer");
  FwdTrainCall c;
  c.norm = desc->norm; c.act = desc->act; c.drop_mode = drop_mode_of(desc);
  c.momentum = desc->momentum; c.eps = desc->eps; c.r_max = desc->r_max; c.d_max = desc->d_max;
  c.drop_scale = drop_scale_of(desc);
  c.x = x; c.gamma = gamma; c.beta = beta; c.mask = mask;
  c.mean = mean; c.stdv = stdv; c.mov_mean = mov_mean; c.mov_std = mov_std; c.r = r; c.d = d;
  c.y = y; c.xhat = nullptr; c.nrm = nullptr;
  c.partial_in = partial; c.partial_chunks = nchunks;
  return run_fwd_train(ctx, B, H, c);
}

// out[j] (+)= column sum, from the first plane of the statistics partials.
__global__ __launch_bounds__(kBlock) void k_colsum_finalize(float const *__restrict__ partial, unsigned nchunks,
                                                             size_t H, float *__restrict__ out, int accumulate) {
  __shared__ float lds[kBlock];
  float tot[1];
  chunk_totals<1>(partial, nchunks, H, tot, lds);
  size_t const j = static_cast<size_t>(blockIdx.x) * kFinCols + threadIdx.x;
  if (threadIdx.x >= kFinCols || j >= H) return;
  out[j] = accumulate ? out[j] + tot[0] : tot[0];
}

int column_sums(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float *out, int accumulate) {
  int rc = dlmi_scratch_reserve(ctx, 2 * 16 * 2 * H * sizeof(float));
  if (rc != DLMI_OK) return rc;
  bool const vec4 = use_vec4(H, {x});
  ColGeom const g = reduce_geometry(ctx, B, H, vec4, 2);
  float *pw = reinterpret_cast<float *>(ctx->scratch);
  dim3 const grid(g.grid_x, g.nchunks), block(kBlock);
  if (vec4)
    hipLaunchKernelGGL(k_col_stats<4>, grid, block, 0, ctx->stream, x, B, H, g.tx_log2, g.rows_per_chunk, pw);
  else
    hipLaunchKernelGGL(k_col_stats<1>, grid, block, 0, ctx->stream, x, B, H, g.tx_log2, g.rows_per_chunk, pw);
  DLMI_LAUNCH_CHECK(ctx, "k_col_stats");
  hipLaunchKernelGGL(k_colsum_finalize, dim3(static_cast<unsigned>(dlmi_ceil_div(H, kFinCols))), block, 0, ctx->stream,
                     pw, g.nchunks, H, out, accumulate);
  DLMI_LAUNCH_CHECK(ctx, "k_colsum_finalize");
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
  c.norm = norm; c.act = DLMI_ACT_LINEAR; c.drop_mode = kDropNone;
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
  c.norm = desc->norm; c.act = desc->act; c.drop_mode = drop_mode_of(desc);
  c.momentum = desc->momentum; c.eps = desc->eps; c.r_max = desc->r_max; c.d_max = desc->d_max;
  c.drop_scale = drop_scale_of(desc);
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
  c.act = DLMI_ACT_LINEAR; c.xhat_given = true; c.drop_mode = kDropNone; c.drop_bwd_masked = 0;
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
  c.act = desc->act; c.xhat_given = false; c.drop_mode = drop_mode_of(desc);
  c.drop_bwd_masked = desc->dropout_bwd == DLMI_DROP_BWD_MASKED ? 1 : 0;
  c.drop_scale = drop_scale_of(desc);
  c.x = x; c.gamma = gamma; c.beta = beta; c.mean = mean; c.stdv = stdv; c.r = r; c.d = d; c.xhat = nullptr;
  c.dY = dY; c.mask = mask;
  c.dgamma = dgamma; c.dbeta = dbeta; c.dmean = nullptr; c.dstd = nullptr; c.dX = dX;
  return run_bwd(ctx, B, H, c);
}

}  // extern "C"
