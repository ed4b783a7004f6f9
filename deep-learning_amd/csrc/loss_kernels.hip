// Seed gradient, loss and accuracy of an output layer whose activation is
// element-wise (everything but softmax, which has its own kernel): the
// regression side of compute_error (v1/learner/compute_error_st.cpp:26-131,
// compute_loss.cpp:25-138) for gfx950.
//
// Per output (b, k), with q the layer's output, x its pre-activation and y the
// target:
//   loss term    loss_fn(q, y)                      compute_loss.cpp:52-99
//   accuracy     by the accuracy function           compute_error_st.cpp:56-100
//   dZ           f'(x, q) * loss_fn_derivative(q, y) compute_error_st.cpp:118-123,
//                                                   compute_loss.cpp:101-138
// One wavefront per row (the cross-entropy accuracy needs the row's arg-max);
// the reported sums are accumulated in double: one pair per block, added in a
// fixed order by the block that finishes last (block_pairs.hpp).  A tiny
// kernel next to the GEMMs: [batch, outputs] elements, 16 B each.
#include "activations.hpp"
#include "block_pairs.hpp"
#include "dlmi_common.hpp"

namespace dlmi {

constexpr int kLossBlock = 256;
constexpr float kLossEps = 0.0000001f;  // data/dtypes.hpp:113

__device__ __forceinline__ float sign_of(float v) { return static_cast<float>((0.0f < v) - (v < 0.0f)); }

template <int ACT>
__global__ __launch_bounds__(kLossBlock) void k_loss_seed(int loss, int accu, float accu_threshold,
                                                          float const *__restrict__ z, float const *__restrict__ q,
                                                          float const *__restrict__ y, float *__restrict__ dZ, size_t B,
                                                          size_t H, double *__restrict__ pairs, double *__restrict__ acc,
                                                          unsigned *__restrict__ ticket) {
  int const lane = threadIdx.x & 63;
  size_t const row = static_cast<size_t>(blockIdx.x) * (kLossBlock / 64) + threadIdx.x / 64;
  double lsum = 0.0, asum = 0.0;
  if (row < B) {
    float const *qi = q + row * H, *yi = y + row * H, *zi = z + row * H;
    bool const ce = loss == DLMI_LOSS_CROSS_ENTROPY;
    float const scale = ce ? static_cast<float>(B) : static_cast<float>(B * H);  // compute_loss.cpp:132-136
    float best = -3.402823466e+38f;
    long long best_k = -1, target_k = static_cast<long long>(H);
    for (size_t k = lane; k < H; k += 64) {
      float const qv = qi[k], yv = yi[k];
      float const diff = qv - yv;
      float const c = qv < kLossEps ? kLossEps : (qv > 1.0f - kLossEps ? 1.0f - kLossEps : qv);
      float l, dl;
      switch (loss) {
        case DLMI_LOSS_ME: case DLMI_LOSS_L1: l = diff; dl = -1.0f; break;
        case DLMI_LOSS_MAE: l = fabsf(diff); dl = qv > yv ? 1.0f : (qv < yv ? -1.0f : 0.0f); break;
        case DLMI_LOSS_CROSS_ENTROPY:
          l = yv == 1.0f ? -(yv * logf(c)) : 0.0f;
          dl = yv == 1.0f ? -1.0f / c : 0.0f;
          break;
        default: l = diff * diff; dl = 2.0f * diff; break;  // L2, MSE, RMSE
      }
      lsum += static_cast<double>(l);
      switch (accu) {
        case DLMI_ACCU_DISTANCE: if (fabsf(diff) <= accu_threshold) asum += 1.0; break;
        case DLMI_ACCU_DIRECTIONAL: asum += 1.0; break;
        case DLMI_ACCU_SIGN:
          if (sign_of(yv) == sign_of(qv) || (sign_of(yv) == 0.0f && qv >= -kLossEps && qv <= kLossEps)) asum += 1.0;
          break;
        default:  // cross-entropy accuracy: arg-max of the row against the target index
          if (qv >= best) { best = qv; best_k = static_cast<long long>(k); }
          if (yv == 1.0f) target_k = static_cast<long long>(k);
          break;
      }
      if (dZ != nullptr) dZ[row * H + k] = act_derive<ACT>(zi[k], qv) * (dl / scale);
    }
    for (int off = 32; off > 0; off >>= 1) {
      lsum += __shfl_xor(lsum, off, 64);
      asum += __shfl_xor(asum, off, 64);
      float const ob = __shfl_xor(best, off, 64);
      long long const ok = __shfl_xor(best_k, off, 64);
      if (ob > best || (ob == best && ok > best_k)) { best = ob; best_k = ok; }  // ">=" scan: the last maximum
      long long const ot = __shfl_xor(target_k, off, 64);
      long long const a = target_k == static_cast<long long>(H) ? -1 : target_k;
      long long const b = ot == static_cast<long long>(H) ? -1 : ot;
      long long const m = a > b ? a : b;
      target_k = m < 0 ? static_cast<long long>(H) : m;  // the last k with y == 1; H: none
    }
    if (accu == DLMI_ACCU_CROSS_ENTROPY) asum = (target_k == best_k) ? 1.0 : 0.0;
  }
  if (acc != nullptr) {
    __shared__ double sh[2][kLossBlock / 64];
    if (lane == 0) {
      sh[0][threadIdx.x / 64] = lsum;
      sh[1][threadIdx.x / 64] = asum;
    }
    __syncthreads();
    double l = 0.0, c = 0.0;
    if (threadIdx.x == 0)
      for (int w = 0; w < kLossBlock / 64; ++w) { l += sh[0][w]; c += sh[1][w]; }
    // no floating-point atomics: the sums, which iRPROP+ branches on, are the same from run to run
    finish_block_pairs(l, c, pairs, acc, ticket);
  }
}

}  // namespace dlmi

using namespace dlmi;

extern "C" {

int dlmi_loss_seed(dlmi_ctx *ctx, dlmi_loss loss, dlmi_accuracy accu, float accu_threshold, dlmi_activation act,
                   size_t B, size_t H, float const *z, float const *q, float const *y, float *dZ, double *stats) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  switch (loss) {
    case DLMI_LOSS_CROSS_ENTROPY: case DLMI_LOSS_L1: case DLMI_LOSS_L2: case DLMI_LOSS_MAE: case DLMI_LOSS_ME:
    case DLMI_LOSS_MSE: case DLMI_LOSS_RMSE: break;
    default: return dlmi_fail(ctx, DLMI_E_UNSUPPORTED, "dlmi_loss_seed: loss function %d has no derivative on this path", loss);
  }
  switch (accu) {
    case DLMI_ACCU_CROSS_ENTROPY: case DLMI_ACCU_DIRECTIONAL: case DLMI_ACCU_DISTANCE: case DLMI_ACCU_SIGN: break;
    default: return dlmi_fail(ctx, DLMI_E_UNSUPPORTED, "dlmi_loss_seed: accuracy function %d is not on this path", accu);
  }
  DLMI_REQUIRE(ctx, act_supported(act), "unsupported activation (softmax has dlmi_softmax_ce_seed)");
  if (B * H == 0) return DLMI_OK;
  DLMI_REQUIRE(ctx, q && y && (dZ == nullptr || z != nullptr), "null pointer");
  dim3 const grid(static_cast<unsigned>(dlmi_ceil_div(B, kLossBlock / 64))), block(kLossBlock);
  float const *zz = z != nullptr ? z : q;  // unused without dZ
  double *pairs = nullptr;
  if (stats != nullptr) {
    int rc = dlmi_scratch_reserve(ctx, static_cast<size_t>(grid.x) * 2 * sizeof(double));
    if (rc != DLMI_OK) return rc;
    pairs = reinterpret_cast<double *>(dlmi_scratch_data(ctx));
  }
  DLMI_DISPATCH_ACT(act, hipLaunchKernelGGL((k_loss_seed<ACT>), grid, block, 0, ctx->stream, static_cast<int>(loss),
                                            static_cast<int>(accu), accu_threshold, zz, q, y, dZ, B, H, pairs, stats,
                                            ctx->pair_ticket));
  DLMI_LAUNCH_CHECK(ctx, "k_loss_seed");
  return DLMI_OK;
}

}  // extern "C"
