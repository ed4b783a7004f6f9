// Euclidean-norm constraints around the optimizer step for gfx950: the global
// gradient clip that precedes it and the per-unit max-norm constraint on the
// weights that follows it (Update_Parameter, v1/learner/model.cpp:4703-4866).
//
//   clip      g *= c / ||g||  when ||g|| >= c, over the whole gradient array
//             (Clip_Gradient__*, v1/ops/constraints/clip_gradient.cpp:75-83)
//   max-norm  w_h *= c / ||w_h||  when ||w_h|| >= c, for each unit's fan-in row
//             (Update_Weight_Regularization__Max_Norm_Constraints__Neurons__*,
//             v1/ops/constraints/max_norm.cpp:61-78)
// both through euclidean_norm_{st,mp} (v1/ops/constraints/euclidean.cpp:24-62).
//
// HBM-bound: the clip reads the gradient twice and writes it once (12 B per
// parameter; only 4 B when the norm is below the threshold, the scale pass then
// returns at once), max-norm likewise per row.  Sums are formed in a fixed
// order (per-thread strided sums, wavefront shuffles, LDS tree; block partials
// added in index order), so results repeat from run to run.
#include "dlmi_common.hpp"

namespace dlmi {

constexpr int kCBlock = 256;
constexpr int kCWave = 64;

// Sum over the block; every thread gets the total.
__device__ __forceinline__ float block_sum(float v, float *lds) {
#pragma unroll
  for (int off = kCWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kCWave);
  int const wave = threadIdx.x / kCWave, lane = threadIdx.x % kCWave;
  __syncthreads();  // lds may still be read from a previous call
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  return (lds[0] + lds[1]) + (lds[2] + lds[3]);
}

__global__ __launch_bounds__(kCBlock) void k_sumsq_partial(float const *__restrict__ g, size_t n, size_t n4,
                                                           float *__restrict__ partial) {
  __shared__ float lds[kCBlock / kCWave];
  size_t const stride = static_cast<size_t>(gridDim.x) * kCBlock;
  size_t i = static_cast<size_t>(blockIdx.x) * kCBlock + threadIdx.x;
  float s = 0.0f;
  for (; i < n4; i += stride) {
    float4 const v = reinterpret_cast<float4 const *>(g)[i];
    s += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
  }
  for (i = n4 * 4 + static_cast<size_t>(blockIdx.x) * kCBlock + threadIdx.x; i < n; i += stride) s += g[i] * g[i];
  s = block_sum(s, lds);
  if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

// One block: factor[0] = c / norm when norm >= c, else 1 (euclidean.cpp:33-38).
__global__ __launch_bounds__(kCBlock) void k_clip_factor(float const *__restrict__ partial, unsigned nparts,
                                                         float max_norm, float *__restrict__ factor) {
  __shared__ float lds[kCBlock / kCWave];
  float s = 0.0f;
  for (unsigned i = threadIdx.x; i < nparts; i += kCBlock) s += partial[i];
  s = block_sum(s, lds);
  if (threadIdx.x == 0) {
    float const norm = sqrtf(s);
    factor[0] = norm >= max_norm ? max_norm / norm : 1.0f;
  }
}

__global__ __launch_bounds__(kCBlock) void k_scale_by(float *__restrict__ g, size_t n, size_t n4,
                                                      float const *__restrict__ factor) {
  float const f = factor[0];
  if (f == 1.0f) return;  // below the threshold: nothing is rewritten
  size_t const stride = static_cast<size_t>(gridDim.x) * kCBlock;
  size_t i = static_cast<size_t>(blockIdx.x) * kCBlock + threadIdx.x;
  for (; i < n4; i += stride) {
    float4 v = reinterpret_cast<float4 *>(g)[i];
    v.x *= f; v.y *= f; v.z *= f; v.w *= f;
    reinterpret_cast<float4 *>(g)[i] = v;
  }
  for (i = n4 * 4 + static_cast<size_t>(blockIdx.x) * kCBlock + threadIdx.x; i < n; i += stride) g[i] *= f;
}

// One block per row of W [rows][cols].
__global__ __launch_bounds__(kCBlock) void k_max_norm_rows(float *__restrict__ W, size_t cols, float max_norm) {
  __shared__ float lds[kCBlock / kCWave];
  float *const row = W + static_cast<size_t>(blockIdx.x) * cols;
  float s = 0.0f;
  for (size_t k = threadIdx.x; k < cols; k += kCBlock) s += row[k] * row[k];
  s = block_sum(s, lds);
  float const norm = sqrtf(s);
  if (norm >= max_norm) {
    float const f = max_norm / norm;
    for (size_t k = threadIdx.x; k < cols; k += kCBlock) row[k] *= f;
  }
}

}  // namespace dlmi

using namespace dlmi;

extern "C" {

int dlmi_clip_gradient(dlmi_ctx *ctx, size_t n, float *grads, float max_norm) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, n == 0 || grads != nullptr, "null pointer");
  DLMI_REQUIRE(ctx, max_norm >= 0.0f, "negative threshold");
  if (n == 0) return DLMI_OK;
  size_t const n4 = dlmi_aligned16(grads) ? n / 4 : 0;
  size_t blocks = dlmi_ceil_div(n4 ? n4 : n, static_cast<size_t>(kCBlock) * 4);
  size_t const cap = static_cast<size_t>(ctx->num_cu) * 8;
  if (blocks > cap) blocks = cap;
  int rc = dlmi_scratch_reserve(ctx, (blocks + 1) * sizeof(float));
  if (rc != DLMI_OK) return rc;
  float *const partial = reinterpret_cast<float *>(dlmi_scratch_data(ctx));
  float *const factor = partial + blocks;
  hipLaunchKernelGGL(k_sumsq_partial, dim3(static_cast<unsigned>(blocks)), dim3(kCBlock), 0, ctx->stream, grads, n, n4,
                     partial);
  DLMI_LAUNCH_CHECK(ctx, "k_sumsq_partial");
  hipLaunchKernelGGL(k_clip_factor, dim3(1), dim3(kCBlock), 0, ctx->stream, partial, static_cast<unsigned>(blocks),
                     max_norm, factor);
  DLMI_LAUNCH_CHECK(ctx, "k_clip_factor");
  hipLaunchKernelGGL(k_scale_by, dim3(static_cast<unsigned>(blocks)), dim3(kCBlock), 0, ctx->stream, grads, n, n4,
                     factor);
  DLMI_LAUNCH_CHECK(ctx, "k_scale_by");
  return DLMI_OK;
}

int dlmi_max_norm_rows(dlmi_ctx *ctx, size_t rows, size_t cols, float *W, float max_norm) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, rows * cols == 0 || W != nullptr, "null pointer");
  DLMI_REQUIRE(ctx, max_norm >= 0.0f, "negative threshold");
  DLMI_REQUIRE(ctx, rows <= 0x7fffffffu, "too many rows for one launch");
  if (rows * cols == 0) return DLMI_OK;
  hipLaunchKernelGGL(k_max_norm_rows, dim3(static_cast<unsigned>(rows)), dim3(kCBlock), 0, ctx->stream, W, cols,
                     max_norm);
  DLMI_LAUNCH_CHECK(ctx, "k_max_norm_rows");
  return DLMI_OK;
}

}  // extern "C"
