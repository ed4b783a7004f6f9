// Fully-connected products of a NARROW layer on a mini-batch (at most 16 units: the 10-way output layer of
// the reference's own example network).  A 128 x 10 output is one sixth of one MFMA tile; the tiled GEMM
// needs a K split, a slice reduction and then separate softmax / bias-gradient launches around it, each
// of which costs more in launch latency than in work.  Here:
//   k_narrow_fc_fwd  Z = X W^T + b, optionally Q = softmax(Z), one wavefront per row
//                    (fwp_st.cpp:4498-4555, 4796-4828); optionally also the cross-entropy seed gradient of the row
//                    against its targets and the loss / accuracy sums (compute_error_st.cpp:26-131,
//                    compute_loss.cpp:88-95, 101-138): the output layer's forward pass and the start of the
//                    backward pass in one launch;
//   k_narrow_dw      dW (+)= dZ^T X and db (+)= column sums of dZ in one launch, a workgroup per 8 columns
//                    of X for all rows (update_derivative_fwp_st.cpp:246-302).
// and for a layer of ANY width on a mini-batch (at most 256 rows):
//   k_minibatch_dw   dW (+)= dZ^T X, a workgroup per 64 x 64 block of dW: its 64 columns of dZ and of X for all rows
//                    go into LDS once, the sum over the rows runs on the matrix pipe (v_mfma_f32_16x16x4_f32, the
//                    rows in ascending groups of four).  The reduction of this product is the batch: a hundred
//                    rows are eight K tiles of the tiled GEMM, which spends its time starting and draining its
//                    pipeline (784 x 512 on 128 rows: 12.4 us there, about half of it here).
// Sums run in a fixed order (no float atomics).  Citations: /root/reference/lib/deep-learning/v1/learner/.
#include <hip/hip_runtime.h>

#include "block_pairs.hpp"
#include "dlmi_common.hpp"
#include "softmax_ce_row.hpp"

namespace dlmi {
namespace {

constexpr int kNarrowMaxUnits = 16;
constexpr size_t kNarrowMaxRowsFwd = 1024;
constexpr size_t kNarrowMaxRowsDw = 256;
constexpr int kNarrowThreads = 256;
constexpr int kNarrowFwdThreads = 64;  // one row per workgroup: a mini-batch spreads over as many CUs as it has rows

typedef float nv4f __attribute__((ext_vector_type(4)));

// One wavefront per row.  Lane l takes k = 4l .. 4l+3, then + 256, ... (16-byte loads, coalesced over X's row
// and over each row of W; VEC = 1: k = l, l + 64, ... for rows that are not 16-byte aligned); all loads of a
// step are independent, so they are in flight together.  The 64 partial sums of an output are combined with the
// xor-shuffle tree; lane o then holds output o.  H is a template parameter so that the loops over the outputs
// unroll without predicates.
// What the seed-gradient variant takes besides: targets Y [B,H], the gradient dZ [B,H], and the loss / accuracy
// accumulators with their per-block pairs and ticket (block_pairs.hpp; acc == nullptr: no sums).
struct NarrowSeedArgs {
  float const *Y;
  float *dZ;
  double *pairs, *acc;
  unsigned *ticket;
};

template <int H, int VEC, bool SOFTMAX, bool SEED = false>
__global__ __launch_bounds__(kNarrowFwdThreads) void k_narrow_fc_fwd(float const *__restrict__ X, float const *__restrict__ W,
                                                                   float const *__restrict__ bias, float *__restrict__ Z,
                                                                   float *Q, size_t B, size_t K, NarrowSeedArgs sa) {
  static_assert(!SEED || (SOFTMAX && kNarrowFwdThreads == 64), "the seed variant is one wavefront per workgroup, grid = rows");
  int const lane = threadIdx.x & 63;
  size_t const row = static_cast<size_t>(blockIdx.x) * (kNarrowFwdThreads / 64) + threadIdx.x / 64;
  if (row >= B) return;
  float acc[H];
#pragma unroll
  for (int o = 0; o < H; ++o) acc[o] = 0.0f;
  float const *xr = X + row * K;
  if constexpr (VEC == 4) {
#pragma unroll 2
    for (size_t k = static_cast<size_t>(lane) * 4; k < K; k += 256) {
      nv4f const xv = *reinterpret_cast<nv4f const *>(xr + k);
      nv4f w[H];
#pragma unroll
      for (int o = 0; o < H; ++o) w[o] = *reinterpret_cast<nv4f const *>(W + static_cast<size_t>(o) * K + k);
#pragma unroll
      for (int o = 0; o < H; ++o) {
        acc[o] += xv[0] * w[o][0];
        acc[o] += xv[1] * w[o][1];
        acc[o] += xv[2] * w[o][2];
        acc[o] += xv[3] * w[o][3];
      }
    }
  } else {
#pragma unroll 4
    for (size_t k = lane; k < K; k += 64) {
      float const xv = xr[k];
      float w[H];
#pragma unroll
      for (int o = 0; o < H; ++o) w[o] = W[static_cast<size_t>(o) * K + k];
#pragma unroll
      for (int o = 0; o < H; ++o) acc[o] += xv * w[o];
    }
  }
  float z = 0.0f;
#pragma unroll
  for (int o = 0; o < H; ++o) {
    float s = acc[o];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == o) z = s;
  }
  bool const mine = lane < H;
  if (mine) {
    if (bias != nullptr) z += bias[lane];
    Z[row * H + lane] = z;
  }
  if constexpr (SOFTMAX) {
    // the arithmetic of the stand-alone softmax leaf: max, exp(x - max), sum over the same tree, times 1 / sum
    float mx = mine ? z : -3.402823466e+38f;
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float const e = mine ? expf(z - mx) : 0.0f;
    float s = e;
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    s = 1.0f / s;
    if (mine) Q[row * H + lane] = e * s;
  }
  if constexpr (SEED) {
    // (every workgroup of the launch holds a row: the grid is exactly B workgroups of one wavefront)
    double loss = 0.0, correct = 0.0;
    softmax_ce_seed_row(Q + row * H, sa.Y + row * H, sa.dZ + row * H, H, B, lane, loss, correct);
    if (sa.acc != nullptr) finish_block_pairs(loss, correct, sa.pairs, sa.acc, sa.ticket);
  }
}

constexpr int kDwCols = 8, kDwGroups = 32;

// dW[o][j] (+)= sum_b dZ[b][o] X[b][j], db[o] (+)= sum_b dZ[b][o].  B <= 256, H <= 16.  Workgroup `block` of
// ceil(K / 8) forms 8 columns of dW, workgroup 0 also db.  lds: kNarrowDwLds floats.
constexpr int kNarrowDwStride = kNarrowMaxUnits + 1;
constexpr int kNarrowDwLds = static_cast<int>(kNarrowMaxRowsDw) * kNarrowDwStride + kDwGroups * kNarrowMaxUnits * kDwCols;
__device__ __forceinline__ void narrow_dw_block(float const *__restrict__ X, float const *__restrict__ dZ,
                                                float *__restrict__ dW, float *__restrict__ db, size_t B, size_t K,
                                                int H, int accumulate, unsigned block, float *__restrict__ lds) {
  constexpr int kStride = kNarrowDwStride;
  float *const dz = lds;  // [B][kStride]
  float (*const red)[kNarrowMaxUnits][kDwCols] =
      reinterpret_cast<float (*)[kNarrowMaxUnits][kDwCols]>(lds + kNarrowMaxRowsDw * kStride);  // [kDwGroups]
  for (size_t i = threadIdx.x; i < B * static_cast<size_t>(H); i += kNarrowThreads)
    dz[(i / H) * kStride + (i % H)] = dZ[i];
  __syncthreads();
  int const c = threadIdx.x % kDwCols, rg = threadIdx.x / kDwCols;
  size_t const col = static_cast<size_t>(block) * kDwCols + c;
  float acc[kNarrowMaxUnits];
#pragma unroll
  for (int o = 0; o < kNarrowMaxUnits; ++o) acc[o] = 0.0f;
  if (col < K) {
    for (size_t b = rg; b < B; b += kDwGroups) {
      float const xv = X[b * K + col];
#pragma unroll
      for (int o = 0; o < kNarrowMaxUnits; ++o)
        if (o < H) acc[o] += dz[b * kStride + o] * xv;
    }
  }
#pragma unroll
  for (int o = 0; o < kNarrowMaxUnits; ++o) red[rg][o][c] = acc[o];
  __syncthreads();
  if (static_cast<int>(threadIdx.x) < H * kDwCols) {
    int const o = threadIdx.x / kDwCols, cc = threadIdx.x % kDwCols;
    size_t const j = static_cast<size_t>(block) * kDwCols + cc;
    if (j < K) {
      float t = 0.0f;
#pragma unroll
      for (int g = 0; g < kDwGroups; ++g) t += red[g][o][cc];
      float *dst = dW + static_cast<size_t>(o) * K + j;
      *dst = accumulate ? *dst + t : t;
    }
  }
  if (db != nullptr && block == 0 && static_cast<int>(threadIdx.x) >= kNarrowThreads - H) {
    int const o = kNarrowThreads - 1 - static_cast<int>(threadIdx.x);
    float t = 0.0f;
    for (size_t b = 0; b < B; ++b) t += dz[b * kStride + o];
    db[o] = accumulate ? db[o] + t : t;
  }
}

__global__ __launch_bounds__(kNarrowThreads) void k_narrow_dw(float const *__restrict__ X, float const *__restrict__ dZ,
                                                               float *__restrict__ dW, float *__restrict__ db, size_t B,
                                                               size_t K, int H, int accumulate) {
  __shared__ float lds[kNarrowDwLds];
  narrow_dw_block(X, dZ, dW, db, B, K, H, accumulate, blockIdx.x, lds);
}

}  // namespace

bool narrow_fc_fwd_eligible(dlmi_ctx const *ctx, size_t B, size_t H) {
  return ctx->tune.fc_narrow != 0 && H <= static_cast<size_t>(kNarrowMaxUnits) && B <= kNarrowMaxRowsFwd;
}

template <int H>
static void launch_narrow_fwd(dlmi_ctx *ctx, dim3 grid, bool vec, float const *X, float const *W, float const *bias, float *Z,
                              float *Q, size_t B, size_t K, NarrowSeedArgs const &sa) {
  dim3 const block(kNarrowFwdThreads);
  if (sa.Y != nullptr) {
    if (vec) hipLaunchKernelGGL((k_narrow_fc_fwd<H, 4, true, true>), grid, block, 0, ctx->stream, X, W, bias, Z, Q, B, K, sa);
    else hipLaunchKernelGGL((k_narrow_fc_fwd<H, 1, true, true>), grid, block, 0, ctx->stream, X, W, bias, Z, Q, B, K, sa);
  } else if (Q != nullptr) {
    if (vec) hipLaunchKernelGGL((k_narrow_fc_fwd<H, 4, true>), grid, block, 0, ctx->stream, X, W, bias, Z, Q, B, K, sa);
    else hipLaunchKernelGGL((k_narrow_fc_fwd<H, 1, true>), grid, block, 0, ctx->stream, X, W, bias, Z, Q, B, K, sa);
  } else {
    if (vec) hipLaunchKernelGGL((k_narrow_fc_fwd<H, 4, false>), grid, block, 0, ctx->stream, X, W, bias, Z, Q, B, K, sa);
    else hipLaunchKernelGGL((k_narrow_fc_fwd<H, 1, false>), grid, block, 0, ctx->stream, X, W, bias, Z, Q, B, K, sa);
  }
}

int narrow_fc_fwd(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *X, float const *W, float const *bias, float *Z,
                  float *Q, float const *Y, float *dZ, double *stats) {
  dim3 const grid(static_cast<unsigned>(dlmi_ceil_div(B, static_cast<size_t>(kNarrowFwdThreads / 64))));
  bool const vec = K % 4 == 0 && dlmi_aligned16(X) && dlmi_aligned16(W);
  NarrowSeedArgs sa{Y, dZ, nullptr, stats, ctx->pair_ticket};
  if (Y != nullptr) {
    if (Q == nullptr || dZ == nullptr) return dlmi_fail(ctx, DLMI_E_INVALID, "narrow_fc_fwd: the seed gradient needs Q and dZ");
    if (stats != nullptr) {
      int const rc = dlmi_scratch_reserve(ctx, static_cast<size_t>(grid.x) * 2 * sizeof(double));
      if (rc != DLMI_OK) return rc;
      sa.pairs = reinterpret_cast<double *>(dlmi_scratch_data(ctx));
    }
  }
  switch (H) {
#define DLMI_NARROW_CASE(n) case n: launch_narrow_fwd<n>(ctx, grid, vec, X, W, bias, Z, Q, B, K, sa); break;
    DLMI_NARROW_CASE(1) DLMI_NARROW_CASE(2) DLMI_NARROW_CASE(3) DLMI_NARROW_CASE(4) DLMI_NARROW_CASE(5)
    DLMI_NARROW_CASE(6) DLMI_NARROW_CASE(7) DLMI_NARROW_CASE(8) DLMI_NARROW_CASE(9) DLMI_NARROW_CASE(10)
    DLMI_NARROW_CASE(11) DLMI_NARROW_CASE(12) DLMI_NARROW_CASE(13) DLMI_NARROW_CASE(14) DLMI_NARROW_CASE(15)
    DLMI_NARROW_CASE(16)
#undef DLMI_NARROW_CASE
    default: return dlmi_fail(ctx, DLMI_E_INVALID, "narrow_fc_fwd: %zu units", H);
  }
  DLMI_LAUNCH_CHECK(ctx, "k_narrow_fc_fwd");
  return DLMI_OK;
}

namespace {

constexpr int kMbTile = 64;      // a workgroup's block of dW: 64 units x 64 inputs
constexpr int kMbRows = 64;      // batch rows staged at a time (2 x 64 x 80 floats = 40 KB of LDS)
constexpr int kMbStride = 80;    // floats between staged rows: 16 banks apart, so that the four rows a fragment
                                 // read touches (two per half wavefront) never share a bank
constexpr int kMbLds = 2 * kMbRows * kMbStride;  // floats of LDS a workgroup stages its rows in
constexpr size_t kMbMaxRows = 256;
constexpr size_t kMbMaxOutputs = size_t(1) << 20;  // H * K: larger layers go to the tiled GEMM

typedef float mv4f __attribute__((ext_vector_type(4)));

// dW[h][k] (+)= sum_b dZ[b][h] X[b][k].  Grid (ceil(K / 64), ceil(H / 64)), 256 threads = 4 wavefronts, each a
// 32 x 32 quarter of the block as 2 x 2 MFMA tiles of 16 x 16.  H, K multiples of 4, 16-byte aligned operands.
__device__ __forceinline__ void minibatch_dw_block(float const *__restrict__ X, float const *__restrict__ dZ,
                                                   float *__restrict__ dW, unsigned B, unsigned K, unsigned H,
                                                   int accumulate, unsigned block_k, unsigned block_h,
                                                   float *__restrict__ lds) {
  float *const zs = lds;                        // dZ[b][h0 .. h0 + 64)
  float *const xs = lds + kMbRows * kMbStride;  // X [b][k0 .. k0 + 64)
  unsigned const k0 = block_k * kMbTile, h0 = block_h * kMbTile;
  int const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int const wh = (wave >> 1) * 32, wk = (wave & 1) * 32;  // this wavefront's quarter
  int const li = lane & 15, lg = lane >> 4;               // position inside a 16 x 16 tile / group of rows
  mv4f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = mv4f{0.0f, 0.0f, 0.0f, 0.0f};
  int const c4 = (threadIdx.x & 15) * 4, r0 = threadIdx.x >> 4;  // staging: 16 threads per row, 16 rows per sweep
  // The rows go through LDS in passes of kMbRows; the loads of a pass are issued before the pass in front of it is
  // multiplied, and all of a pass's loads before its first LDS store: one memory latency in all, not one per pass.
  mv4f vz[kMbRows / 16], vx[kMbRows / 16];
  auto fetch = [&](unsigned b0) {
    unsigned const rows = B - b0 < static_cast<unsigned>(kMbRows) ? B - b0 : static_cast<unsigned>(kMbRows);
#pragma unroll
    for (int i = 0; i < kMbRows / 16; ++i) {
      unsigned const r = r0 + 16 * i;
      bool const row_ok = r < rows;
      vz[i] = row_ok && h0 + c4 < H ? *reinterpret_cast<mv4f const *>(dZ + static_cast<size_t>(b0 + r) * H + h0 + c4) : mv4f{0, 0, 0, 0};
      vx[i] = row_ok && k0 + c4 < K ? *reinterpret_cast<mv4f const *>(X + static_cast<size_t>(b0 + r) * K + k0 + c4) : mv4f{0, 0, 0, 0};
    }
  };
  fetch(0);
  // what is already in dW, asked for now: by the time the sums are formed it is there
  mv4f was[2][2];
#pragma unroll
  for (int ti = 0; ti < 2; ++ti)
#pragma unroll
    for (int tj = 0; tj < 2; ++tj)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        unsigned const h = h0 + wh + 16 * ti + 4 * lg + r, k = k0 + wk + 16 * tj + li;
        was[ti][tj][r] = accumulate && h < H && k < K ? dW[static_cast<size_t>(h) * K + k] : 0.0f;
      }
  for (unsigned b0 = 0; b0 < B; b0 += kMbRows) {
    unsigned const rows = B - b0 < static_cast<unsigned>(kMbRows) ? B - b0 : static_cast<unsigned>(kMbRows);
    unsigned const rows4 = (rows + 3u) & ~3u;  // the matrix pipe takes rows in fours: the tail is zeros
    if (b0 != 0) __syncthreads();              // everybody is done with the previous rows
#pragma unroll
    for (int i = 0; i < kMbRows / 16; ++i) {
      unsigned const r = r0 + 16 * i;
      if (r < rows4) {
        *reinterpret_cast<mv4f *>(zs + r * kMbStride + c4) = vz[i];
        *reinterpret_cast<mv4f *>(xs + r * kMbStride + c4) = vx[i];
      }
    }
    __syncthreads();
    if (b0 + kMbRows < B) fetch(b0 + kMbRows);
    // A[i][kk] = dZ[b + kk][h0 + wh + 16 ti + i], B[kk][j] = X[b + kk][k0 + wk + 16 tj + j]: lane (li, lg) holds
    // element (i = li, kk = lg) of A and (kk = lg, j = li) of B
    float const *zr = zs + lg * kMbStride + wh + li;
    float const *xr = xs + lg * kMbStride + wk + li;
    for (unsigned b = 0; b < rows4; b += 4) {
      float const a0 = zr[b * kMbStride], a1 = zr[b * kMbStride + 16], x0 = xr[b * kMbStride], x1 = xr[b * kMbStride + 16];
      acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, x0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, x1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, x0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, x1, acc[1][1], 0, 0, 0);
    }
  }
  // D[i = 4 lg + r][j = li] of every tile
#pragma unroll
  for (int ti = 0; ti < 2; ++ti)
#pragma unroll
    for (int tj = 0; tj < 2; ++tj)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        unsigned const h = h0 + wh + 16 * ti + 4 * lg + r, k = k0 + wk + 16 * tj + li;
        if (h < H && k < K) {
          // (was is 0 without accumulation; 0 + x is x bit for bit, up to the sign of a zero sum)
          dW[static_cast<size_t>(h) * K + k] = accumulate ? was[ti][tj][r] + acc[ti][tj][r] : acc[ti][tj][r];
        }
      }
}

__global__ __launch_bounds__(256) void k_minibatch_dw(float const *__restrict__ X, float const *__restrict__ dZ,
                                                       float *__restrict__ dW, unsigned B, unsigned K, unsigned H,
                                                       int accumulate) {
  __shared__ __attribute__((aligned(16))) float lds[kMbLds];
  minibatch_dw_block(X, dZ, dW, B, K, H, accumulate, blockIdx.x, blockIdx.y, lds);
}

// Several such products in one launch (the layers of a network after its backward pass): the workgroups walk the
// concatenated lists of blocks.  A block's arithmetic is that of the single launch.  The launch can also carry the
// weight and bias gradient of ONE narrow layer (at most 16 units: the output layer): the workgroups behind the
// last block run narrow_dw_block on it, as k_narrow_dw would.
struct MbDwGroupArgs {
  struct Problem {
    float const *X, *dZ;
    float *dW;
    unsigned B, K, H, blocks_k, block_end;  // block_end: this problem's blocks end before this linear workgroup id
  };
  Problem p[kMinibatchDwGroupMax];
  unsigned n;
  int accumulate;
  // the narrow layer: workgroups [p[n - 1].block_end, gridDim.x); narrow_dW == nullptr: none
  float const *narrow_X, *narrow_dZ;
  float *narrow_dW, *narrow_db;
  unsigned narrow_B, narrow_K, narrow_H;
};
constexpr int kMbGroupLds = kMbLds > kNarrowDwLds ? kMbLds : kNarrowDwLds;
static_assert(kNarrowThreads == 256, "both kinds of workgroup have 256 threads");
__global__ __launch_bounds__(256) void k_minibatch_dw_group(MbDwGroupArgs a) {
  __shared__ __attribute__((aligned(16))) float lds[kMbGroupLds];
  unsigned const mb_blocks = a.p[a.n - 1].block_end;
  if (blockIdx.x >= mb_blocks) {
    narrow_dw_block(a.narrow_X, a.narrow_dZ, a.narrow_dW, a.narrow_db, a.narrow_B, a.narrow_K,
                    static_cast<int>(a.narrow_H), a.accumulate, blockIdx.x - mb_blocks, lds);
    return;
  }
  unsigned i = 0;
  while (i + 1 < a.n && blockIdx.x >= a.p[i].block_end) ++i;
  MbDwGroupArgs::Problem const &q = a.p[i];
  unsigned const local = blockIdx.x - (i == 0 ? 0u : a.p[i - 1].block_end);
  minibatch_dw_block(q.X, q.dZ, q.dW, q.B, q.K, q.H, a.accumulate, local % q.blocks_k, local / q.blocks_k, lds);
}

}  // namespace

bool narrow_dw_eligible(dlmi_ctx const *ctx, size_t B, size_t H) {
  return ctx->tune.fc_narrow != 0 && H <= static_cast<size_t>(kNarrowMaxUnits) && B <= kNarrowMaxRowsDw;
}

int minibatch_dw_group(dlmi_ctx *ctx, size_t n, MinibatchDwProblem const *problems, int accumulate,
                       NarrowDwProblem const *narrow) {
  if (n == 0) return dlmi_fail(ctx, DLMI_E_INVALID, "minibatch_dw_group: no problem");
  if (narrow != nullptr && (!narrow_dw_eligible(ctx, narrow->B, narrow->H) || narrow->X == nullptr ||
                            narrow->dZ == nullptr || narrow->dW == nullptr || narrow->K == 0))
    return dlmi_fail(ctx, DLMI_E_INVALID, "minibatch_dw_group: the narrow layer does not qualify");
  for (size_t first = 0; first < n; first += kMinibatchDwGroupMax) {
    MbDwGroupArgs a;
    a.n = static_cast<unsigned>(n - first < static_cast<size_t>(kMinibatchDwGroupMax) ? n - first : kMinibatchDwGroupMax);
    a.accumulate = accumulate;
    unsigned total = 0;
    for (unsigned i = 0; i < a.n; ++i) {
      MinibatchDwProblem const &s = problems[first + i];
      if (!minibatch_dw_eligible(ctx, s.B, s.K, s.H, s.X, s.dZ, s.dW)) return dlmi_fail(ctx, DLMI_E_INVALID, "minibatch_dw_group: problem %u does not qualify", i);
      MbDwGroupArgs::Problem &q = a.p[i];
      q.X = s.X; q.dZ = s.dZ; q.dW = s.dW;
      q.B = static_cast<unsigned>(s.B); q.K = static_cast<unsigned>(s.K); q.H = static_cast<unsigned>(s.H);
      q.blocks_k = static_cast<unsigned>(dlmi_ceil_div(s.K, static_cast<size_t>(kMbTile)));
      total += q.blocks_k * static_cast<unsigned>(dlmi_ceil_div(s.H, static_cast<size_t>(kMbTile)));
      q.block_end = total;
    }
    for (unsigned i = a.n; i < static_cast<unsigned>(kMinibatchDwGroupMax); ++i) a.p[i] = a.p[a.n - 1];
    a.narrow_X = a.narrow_dZ = nullptr;
    a.narrow_dW = a.narrow_db = nullptr;
    a.narrow_B = a.narrow_K = a.narrow_H = 0;
    if (narrow != nullptr && first == 0) {  // with the first launch
      a.narrow_X = narrow->X; a.narrow_dZ = narrow->dZ; a.narrow_dW = narrow->dW; a.narrow_db = narrow->db;
      a.narrow_B = static_cast<unsigned>(narrow->B); a.narrow_K = static_cast<unsigned>(narrow->K);
      a.narrow_H = static_cast<unsigned>(narrow->H);
      total += static_cast<unsigned>(dlmi_ceil_div(narrow->K, static_cast<size_t>(kDwCols)));
    }
    hipLaunchKernelGGL(k_minibatch_dw_group, dim3(total), dim3(256), 0, ctx->stream, a);
    DLMI_LAUNCH_CHECK(ctx, "k_minibatch_dw_group");
  }
  return DLMI_OK;
}

bool minibatch_dw_eligible(dlmi_ctx const *ctx, size_t B, size_t K, size_t H, float const *Xin, float const *dZ, float const *dW) {
  return ctx->tune.minibatch_dw != 0 && B <= kMbMaxRows && H * K <= kMbMaxOutputs && H % 4 == 0 && K % 4 == 0 &&
         dlmi_aligned16(Xin) && dlmi_aligned16(dZ) && dW != nullptr;
}

int minibatch_dw_try(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *Xin, float const *dZ, float *dW, int accumulate) {
  if (!minibatch_dw_eligible(ctx, B, K, H, Xin, dZ, dW)) return 0;
  dim3 const grid(static_cast<unsigned>(dlmi_ceil_div(K, static_cast<size_t>(kMbTile))),
                  static_cast<unsigned>(dlmi_ceil_div(H, static_cast<size_t>(kMbTile))));
  hipLaunchKernelGGL(k_minibatch_dw, grid, dim3(256), 0, ctx->stream, Xin, dZ, dW, static_cast<unsigned>(B),
                     static_cast<unsigned>(K), static_cast<unsigned>(H), accumulate);
  DLMI_LAUNCH_CHECK(ctx, "k_minibatch_dw");
  return 1;
}

int narrow_dw_try(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *Xin, float const *dZ, float *dW, float *db,
                  int accumulate) {
  if (!narrow_dw_eligible(ctx, B, H)) return 0;
  dim3 const grid(static_cast<unsigned>(dlmi_ceil_div(K, static_cast<size_t>(kDwCols))));
  hipLaunchKernelGGL(k_narrow_dw, grid, dim3(kNarrowThreads), 0, ctx->stream, Xin, dZ, dW, db, B, K, static_cast<int>(H),
                     accumulate);
  DLMI_LAUNCH_CHECK(ctx, "k_narrow_dw");
  return 1;
}

}  // namespace dlmi

extern "C" int dlmi_fc_softmax_ce_fwd(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *X, float const *W,
                                      float const *bias, float const *Y, float *Z, float *Q, float *dZ, double *stats) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, X && W && Y && Z && Q && dZ, "null pointer");
  DLMI_REQUIRE(ctx, B > 0 && K > 0 && H > 0, "empty operand");
  if (dlmi::narrow_fc_fwd_eligible(ctx, B, H)) return dlmi::narrow_fc_fwd(ctx, B, K, H, X, W, bias, Z, Q, Y, dZ, stats);
  int const rc = dlmi_fc_softmax_fwd(ctx, B, K, H, X, W, bias, Z, Q);
  return rc != DLMI_OK ? rc : dlmi_softmax_ce_seed(ctx, B, H, Q, Y, dZ, stats);
}
