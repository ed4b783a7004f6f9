// Pieces of the batch-(re)normalization kernels that more than one translation unit uses: the per-unit
// forward statistics, the per-element backward recompute, the dropout modes and the host-side call
// descriptors.  Citations: /root/reference/lib/deep-learning/v1/learner/.
#ifndef DLMI_NORM_SHARED_HPP
#define DLMI_NORM_SHARED_HPP

#include <cstddef>
#include <cstdint>

#include "activations.hpp"
#include "dlmi_common.hpp"

namespace dlmi {

// dropout as a template mode
constexpr int kDropNone = 0, kDropUnit = 1, kDropElem = 2;

struct FwdFinalize {
  float *mean, *stdv, *mov_mean, *mov_std, *r, *d;
  float batch_scale;  // 1 / B as a float, multiplied like the reference's tmp_batch_scale
  float momentum, eps, r_max, d_max;
  int renorm;
};

// The six per-unit results of the forward step from the two column sums and the
// unit's moving mean / std as they were before the step.
struct UnitStats {
  float mean, stdv, mov_mean, mov_std, r, d;
};
__device__ __forceinline__ UnitStats fwd_unit_stats(FwdFinalize const &f, float s1, float s2, float mm, float ms) {
  UnitStats u;
  u.mean = s1 * f.batch_scale;
  mm += f.momentum * (u.mean - mm);
  u.stdv = sqrtf(s2 * f.batch_scale - u.mean * u.mean + f.eps);
  ms += f.momentum * (u.stdv - ms);
  u.mov_mean = mm;
  u.mov_std = ms;
  u.r = 1.0f;
  u.d = 0.0f;
  if (f.renorm) {
    float const g = u.stdv / ms;
    float const lo = 1.0f / f.r_max;
    u.r = g < lo ? lo : (g > f.r_max ? f.r_max : g);
    float const dd = (u.mean - mm) / ms;
    u.d = dd < -f.d_max ? -f.d_max : (dd > f.d_max ? f.d_max : dd);
  }
  return u;
}
__device__ __forceinline__ void store_unit_stats(FwdFinalize const &f, size_t j, UnitStats const &u) {
  f.mean[j] = u.mean;
  f.stdv[j] = u.stdv;
  f.mov_mean[j] = u.mov_mean;
  f.mov_std[j] = u.mov_std;
  if (f.r != nullptr) f.r[j] = u.r;
  if (f.d != nullptr) f.d[j] = u.d;
}
// mm, ms: the unit's moving mean and moving std as loaded before the sums were
// formed (so that their latency overlaps the partial-sum loads).
__device__ __forceinline__ void fwd_finalize_unit(FwdFinalize const &f, size_t j, float s1, float s2, float mm,
                                                  float ms) {
  store_unit_stats(f, j, fwd_unit_stats(f, s1, s2, mm, ms));
}

__device__ __forceinline__ float drop_apply(uint8_t m, float scale, float v) { return m ? v * scale : 0.0f; }


// dn = dY * f'(n, q) for one element, recomputing x_hat, n and q from x.
// REFERENCE dropout mode: q is the post-dropout output and dY is untouched
// (bwp_st.cpp:1177-1209 reads the array the dropout leaf overwrote in place);
// MASKED mode: q is the pre-dropout activation and dY is masked and rescaled.
template <int ACT, int DROPM, bool XHAT_GIVEN>
__device__ __forceinline__ float bwd_dn(float drop_scale, int drop_bwd_masked, float xv, float dy, uint8_t m,
                                        float mu, float rs, float dd, float ga, float be, float &xh) {
  if constexpr (XHAT_GIVEN) {
    (void)drop_scale; (void)drop_bwd_masked; (void)xv; (void)m; (void)mu; (void)rs; (void)dd; (void)ga; (void)be;
    return dy;
  } else {
    xh = (xv - mu) * rs + dd;
    float const nn = ga * xh + be;
    float q = act_fire<ACT>(nn);
    float g = dy;
    if constexpr (DROPM != kDropNone) {
      float const gm = drop_apply(m, drop_scale, dy);
      float const qm = drop_apply(m, drop_scale, q);
      g = drop_bwd_masked ? gm : dy;
      q = drop_bwd_masked ? q : qm;
    }
    return g * act_derive<ACT>(nn, q);
  }
}

// ---- host-side descriptors of one forward / backward call
struct FwdTrainCall {
  dlmi_norm norm;
  int act;
  int drop_mode;  // kDropNone / kDropUnit / kDropElem
  float momentum, eps, r_max, d_max, drop_scale;
  float const *x, *gamma, *beta;
  uint8_t const *mask;
  float const *residual = nullptr;
  float *mean, *stdv, *mov_mean, *mov_std, *r, *d, *y, *xhat, *nrm;
  float const *partial_in = nullptr;  // column-sum partials already produced elsewhere ...
  unsigned partial_chunks = 0;        // ... [2][partial_chunks][H]; skips the statistics pass
  float const *snapshot_in = nullptr;  // ... and the moving statistics before this step [2][H], copied by the same producer
  // x itself not formed yet: it is the sum of `nslices` partial products [nslices][B][H] (split-K slices), to
  // be added in slice order and stored to z_out (== x) by the small-batch kernel, the only one that takes them
  float const *slices = nullptr;
  unsigned nslices = 0;
  float *z_out = nullptr;
};

struct BwdCall {
  int act;
  bool xhat_given;
  int drop_mode, drop_bwd_masked;
  float drop_scale;
  float const *x, *gamma, *beta, *mean, *stdv, *r, *d, *xhat, *dY;
  uint8_t const *mask;
  float *dgamma, *dbeta, *dmean, *dstd, *dX;
  bool accumulate = false;  // dX += instead of dX =
  // optional: db[j] (+)= sum over the rows of the dX this call stores (the bias gradient of the layer,
  // update_derivative_fwp_st.cpp:283-302), formed while dX is written instead of by a pass of its own
  float *db = nullptr;
  bool db_accumulate = false;
  // dY not formed yet: it is the sum of `nslices` partial products [nslices][B][H], added in slice order by
  // the small-batch kernel (the only one that takes them); dY is unused then
  float const *dy_slices = nullptr;
  unsigned nslices = 0;
  // dY not formed yet: it is the product dZn . Wn of a NARROW layer above (narrow_h <= kNarrowMaxUnits units:
  // narrow_dz [B][narrow_h], narrow_w [narrow_h][H]), formed by the small-batch kernel itself, unit after unit
  // (Backward_Pass__FC__Loop, bwp_st.cpp:1009-1045: the sum over the layer's units, here in ascending order); dY is unused then
  float const *narrow_dz = nullptr, *narrow_w = nullptr;
  unsigned narrow_h = 0;
};
constexpr unsigned kNarrowMaxUnits = 16;

// The single-launch panel kernels (norm_panel_fwd.hip, norm_panel_bwd.hip).  Return 1 when the call was
// launched that way, 0 when the shape or the context does not qualify (the caller goes on with the
// multi-launch path), a negative DLMI_E_* code on failure.
int panel_fwd_try(dlmi_ctx *ctx, size_t B, size_t H, FwdTrainCall const &c, bool vec4, void *scratch, size_t scratch_bytes);
// db_partials / db_rows (optional): receive the [db_rows][H] partial column sums of dX the kernel left for c.db, or
// nullptr when it left none
int panel_bwd_try(dlmi_ctx *ctx, size_t B, size_t H, BwdCall const &c, bool vec4, void *scratch, size_t scratch_bytes,
                  float **db_partials = nullptr, unsigned *db_rows = nullptr);


// The small-batch kernels (norm_small.hip): one launch per direction for at most 256 rows and 2^20 elements.
// Same return convention (small_norm_eligible, the shape test alone, is declared in dlmi_common.hpp).
int small_fwd_try(dlmi_ctx *ctx, size_t B, size_t H, FwdTrainCall const &c);
int small_bwd_try(dlmi_ctx *ctx, size_t B, size_t H, BwdCall const &c);
int small_colsum_try(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float *out, int accumulate);

}  // namespace dlmi

#endif  // DLMI_NORM_SHARED_HPP
