// Softmax + cross-entropy seed gradient of ONE row by one wavefront (compute_error_st.cpp:26-131,
// compute_loss.cpp:88-95, 101-138), shared by the stand-alone seed kernel and by the narrow-layer forward kernel
// that forms the seed in the same launch: the same operations in the same order, so both give the same bits.
#pragma once
#include <hip/hip_runtime.h>

namespace dlmi {

// qi, yi, dzi: the row's softmax outputs, targets and gradient [H]; B: rows of the batch (the loss derivative is
// divided by it); lane: 0 .. 63.  Every lane of the wavefront calls it.  loss / correct: valid in lane 0.
// (qi may be memory the calling lane has just written itself.)
__device__ __forceinline__ void softmax_ce_seed_row(float const *qi, float const *yi, float *dzi, size_t H, size_t B,
                                                    int lane, double &loss, double &correct) {
  constexpr float kEps = 0.0000001f;  // data/dtypes.hpp:113
  float const inv_b = static_cast<float>(B);
  // S = sum_k q_k * dL_k  (dL_k != 0 only where y_k == 1)
  float s = 0.0f, lsum = 0.0f;
  float best = -3.402823466e+38f;
  long long best_k = -1, target_k = static_cast<long long>(H);
  for (size_t k = lane; k < H; k += 64) {
    float const qk = qi[k];
    float const c = qk < kEps ? kEps : (qk > 1.0f - kEps ? 1.0f - kEps : qk);
    if (yi[k] == 1.0f) {
      s += qk * ((-1.0f / c) / inv_b);
      lsum += -(yi[k] * logf(c));
      target_k = static_cast<long long>(k);  // last k with y == 1 wins below
    }
    if (qk >= best) { best = qk; best_k = static_cast<long long>(k); }
  }
  for (int off = 32; off > 0; off >>= 1) {
    s += __shfl_xor(s, off, 64);
    lsum += __shfl_xor(lsum, off, 64);
    float const ob = __shfl_xor(best, off, 64);
    long long const ok = __shfl_xor(best_k, off, 64);
    // ">=" scan keeps the LAST maximal index (compute_error_st.cpp:62-68)
    if (ob > best || (ob == best && ok > best_k)) { best = ob; best_k = ok; }
    long long const ot = __shfl_xor(target_k, off, 64);
    // the sequential scan keeps the last k with y_k == 1; H means "none"
    long long const a = target_k == static_cast<long long>(H) ? -1 : target_k;
    long long const b = ot == static_cast<long long>(H) ? -1 : ot;
    long long const m = a > b ? a : b;
    target_k = m < 0 ? static_cast<long long>(H) : m;
  }
  for (size_t i = lane; i < H; i += 64) {
    float const qv = qi[i];
    float const c = qv < kEps ? kEps : (qv > 1.0f - kEps ? 1.0f - kEps : qv);
    float const dl = yi[i] == 1.0f ? (-1.0f / c) / inv_b : 0.0f;
    // sum_k (q_i [i==k] - q_k q_i) dL_k = q_i dL_i - q_i S
    dzi[i] = qv * dl - qv * s;
  }
  loss = static_cast<double>(lsum);
  correct = (target_k == best_k) ? 1.0 : 0.0;
}

}  // namespace dlmi
