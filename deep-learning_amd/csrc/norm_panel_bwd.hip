// Backward of batch-(re)normalization + activation + dropout in ONE launch that reads dY and x once: the
// column panel scheme of norm_panel_common.hpp.  Per element the same arithmetic as the multi-launch path
// (bwd_dn; sums of bwp_st.cpp:1478-1506, coefficients and dx of bwp_st.cpp:1508-1531); dn is formed once and
// kept in registers between the reduction and the apply step instead of being recomputed.
//
// Geometry: 512 threads = P/4 column groups of 4 units x 2048/P rows; a workgroup owns B/32 = RPT * 2048/P rows
// and walks panels of P columns: P = 64 (256 B per row) while four panels of x and dn fit the registers, P = 32
// for 4096 rows with a per-element mask.  B in {2048, 4096}, H a multiple of 512.  (Wider panels stream
// faster - the forward kernel's 128 columns reach 5.1 TB/s of actual traffic, 64 columns 3.7 TB/s - but the
// backward pass holds two values per element; the kernel still beats the multi-launch pair because it moves
// 12 instead of 20 bytes per element.)
#include "norm_panel_common.hpp"

namespace dlmi {
namespace {


struct PanelBwdArgs {
  float const *x, *dY, *gamma, *beta, *mean, *stdv, *r, *d;
  uint8_t const *mask;
  float *dX, *dgamma, *dbeta;
  size_t B, H;
  float batch_f, batch_scale, drop_scale;
  int drop_mode, drop_bwd_masked, accumulate;
  PanelSync sync;
  float *part;  // [xcd][panel][rank][3][kP]
};

// dn of one element, dropout mode at run time (bwd_dn of the multi-launch path, same operations)
template <int ACT>
__device__ __forceinline__ float panel_dn(int drop_mode, int drop_bwd_masked, float drop_scale, float xv, float dy,
                                          unsigned char m, float mu, float rs, float dd, float ga, float be, float &xh) {
  xh = (xv - mu) * rs + dd;
  float const nn = ga * xh + be;
  float q = act_fire<ACT>(nn);
  float g = dy;
  if (drop_mode != kDropNone) {
    float const gm = drop_apply(m, drop_scale, dy);
    float const qm = drop_apply(m, drop_scale, q);
    g = drop_bwd_masked ? gm : dy;
    q = drop_bwd_masked ? q : qm;
  }
  return g * act_derive<ACT>(nn, q);
}

// EXTRA: a per-element mask is read and / or dX accumulates (more registers per thread)
template <int ACT, int kP, int RPT, bool EXTRA>
__global__ __launch_bounds__(kPanelThreads) void k_bwd_panel(PanelBwdArgs a) {
  constexpr int kCG = kP / 4;                // column groups per panel row
  constexpr int kTY = kPanelThreads / kCG;   // rows per sweep
  constexpr int kVals = 3 * kP;              // sums per panel: dn*xhat, dn, dn*(x-mean) for every column
  constexpr int kRSplit = kP == 64 ? 2 : 4;  // threads per sum in the rank sum (384 of the 512 threads)
  constexpr int kRPer = kPanelRanks / kRSplit;
  __shared__ float sh[3][kTY][kP];       // per-sweep-row sums of the panel being published
  __shared__ float sh2[kRSplit][kVals];  // halves of the rank sum
  __shared__ float cst[4][7][kP];        // per panel in flight: mean, r/std, d, gamma, beta, std, r
  __shared__ float coef[3][kP];
  __shared__ unsigned s_rank, s_ok;
  PanelWho who;
  if (threadIdx.x == 0) s_ok = 1;
  if (!panel_enter(a.sync, who, &s_rank)) return;
  int const tx = threadIdx.x % kCG, ty = threadIdx.x / kCG;
  size_t const Hx = a.H / kPanelXcds;
  int const npanels = static_cast<int>(Hx / kP);
  size_t const row0 = static_cast<size_t>(who.rank) * (RPT * kTY);
  size_t const col_base = static_cast<size_t>(who.xcd) * Hx;

  struct Stage {
    pv4f x[RPT], g[RPT];          // x, and dY until publish() turns it into dn
    uchar4 m[EXTRA ? RPT : 1];    // per-element keep mask
  };
  auto load = [&](Stage &s, int p) {
    size_t const off0 = (row0 + ty) * a.H + col_base + static_cast<size_t>(p) * kP + tx * 4;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      size_t const off = off0 + static_cast<size_t>(i) * kTY * a.H;
      s.x[i] = __builtin_nontemporal_load(reinterpret_cast<pv4f const *>(a.x + off));
      s.g[i] = __builtin_nontemporal_load(reinterpret_cast<pv4f const *>(a.dY + off));
      if constexpr (EXTRA) {
        if (a.drop_mode == kDropElem) s.m[i] = *reinterpret_cast<uchar4 const *>(a.mask + off);
      }
    }
  };
  auto publish = [&](Stage &s, int p) {
    size_t const col = col_base + static_cast<size_t>(p) * kP;
    // per-unit constants of this thread's 4 columns (the forward's results)
    pv4f mu = *reinterpret_cast<pv4f const *>(a.mean + col + tx * 4);
    pv4f sd = *reinterpret_cast<pv4f const *>(a.stdv + col + tx * 4);
    pv4f rr = *reinterpret_cast<pv4f const *>(a.r + col + tx * 4);
    pv4f dd = *reinterpret_cast<pv4f const *>(a.d + col + tx * 4);
    pv4f ga = *reinterpret_cast<pv4f const *>(a.gamma + col + tx * 4);
    pv4f be = *reinterpret_cast<pv4f const *>(a.beta + col + tx * 4);
    uchar4 um = make_uchar4(1, 1, 1, 1);
    if (a.drop_mode == kDropUnit) um = *reinterpret_cast<uchar4 const *>(a.mask + col + tx * 4);
    pv4f rs;
#pragma unroll
    for (int e = 0; e < 4; ++e) rs[e] = rr[e] * fast_rcp(sd[e]);
    unsigned char const umv[4] = {um.x, um.y, um.z, um.w};
    pv4f s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0}, s2 = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      unsigned char mv[4] = {umv[0], umv[1], umv[2], umv[3]};
      if constexpr (EXTRA) {
        if (a.drop_mode == kDropElem) { mv[0] = s.m[i].x; mv[1] = s.m[i].y; mv[2] = s.m[i].z; mv[3] = s.m[i].w; }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float xh;
        float const dn = panel_dn<ACT>(a.drop_mode, a.drop_bwd_masked, a.drop_scale, s.x[i][e], s.g[i][e], mv[e], mu[e], rs[e],
                                       dd[e], ga[e], be[e], xh);
        s0[e] += dn * xh;
        s1[e] += dn;
        s2[e] += dn * (s.x[i][e] - mu[e]);
        s.g[i][e] = dn;
      }
    }
    __syncthreads();  // the previous publish's readers are done with sh
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      sh[0][ty][tx * 4 + e] = s0[e];
      sh[1][ty][tx * 4 + e] = s1[e];
      sh[2][ty][tx * 4 + e] = s2[e];
    }
    if (ty == 0) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int const c = tx * 4 + e;
        cst[p & 3][0][c] = mu[e]; cst[p & 3][1][c] = rs[e]; cst[p & 3][2][c] = dd[e]; cst[p & 3][3][c] = ga[e];
        cst[p & 3][4][c] = be[e]; cst[p & 3][5][c] = sd[e]; cst[p & 3][6][c] = rr[e];
      }
    }
    __syncthreads();
    if (threadIdx.x < kVals) {
      int const w = threadIdx.x / kP, c = threadIdx.x % kP;
      float t = 0.0f;
#pragma unroll
      for (int j = 0; j < kTY; ++j) t += sh[w][j][c];
      a.part[((static_cast<size_t>(who.xcd) * npanels + p) * kPanelRanks + who.rank) * kVals + w * kP + c] = t;
    }
  };
  auto arrive = [&](int p) {
    __syncthreads();
    if (threadIdx.x == 0) panel_count(panel_arrivals(who, p));
  };
  auto finish = [&](Stage const &s, int p) -> bool {
    size_t const col = col_base + static_cast<size_t>(p) * kP;
    size_t const off0 = (row0 + ty) * a.H + col + tx * 4;
    pv4f old[EXTRA ? RPT : 1];
    if constexpr (EXTRA) {
      if (a.accumulate) {
#pragma unroll
        for (int i = 0; i < RPT; ++i)
          old[i] = __builtin_nontemporal_load(reinterpret_cast<pv4f const *>(a.dX + off0 + static_cast<size_t>(i) * kTY * a.H));
      }
    }
    if (threadIdx.x == 0 && !panel_wait(who, p)) s_ok = 0;
    __syncthreads();
    if (!s_ok) return false;
    if (threadIdx.x < kRSplit * kVals) {
      int const vc = threadIdx.x % kVals, rs = threadIdx.x / kVals;
      float const *pp = a.part + (static_cast<size_t>(who.xcd) * npanels + p) * kPanelRanks * kVals + vc;
      float v[kRPer];
#pragma unroll
      for (int r = 0; r < kRPer; ++r) v[r] = __builtin_nontemporal_load(pp + static_cast<size_t>(rs * kRPer + r) * kVals);
      float t = 0.0f;
#pragma unroll
      for (int r = 0; r < kRPer; ++r) t += v[r];
      sh2[rs][vc] = t;
    }
    __syncthreads();
    if (threadIdx.x < kP) {
      int const c = threadIdx.x;
      float t0 = 0.0f, t1 = 0.0f, t2 = 0.0f;
#pragma unroll
      for (int j = 0; j < kRSplit; ++j) {
        t0 += sh2[j][c];
        t1 += sh2[j][kP + c];
        t2 += sh2[j][2 * kP + c];
      }
      float const ga = cst[p & 3][3][c], sd = cst[p & 3][5][c], rr = cst[p & 3][6][c];
      if (who.rank == 0) {  // accumulating like the reference's derivative array
        a.dgamma[col + c] += t0;
        a.dbeta[col + c] += t1;
      }
      float const dm = (ga * t1) * (-rr / sd);
      float const ds = (ga * t2) * (-rr / (sd * sd));
      coef[0][c] = ga * (rr / sd);
      coef[1][c] = ds / (a.batch_f * sd);
      coef[2][c] = dm * a.batch_scale;
    }
    __syncthreads();
    pv4f mu, c1, c2, c3;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mu[e] = cst[p & 3][0][tx * 4 + e];
      c1[e] = coef[0][tx * 4 + e];
      c2[e] = coef[1][tx * 4 + e];
      c3[e] = coef[2][tx * 4 + e];
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      pv4f out;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float dx = s.g[i][e] * c1[e] + (s.x[i][e] - mu[e]) * c2[e] + c3[e];
        if constexpr (EXTRA) {
          if (a.accumulate) dx += old[i][e];
        }
        out[e] = dx;
      }
      __builtin_nontemporal_store(out, reinterpret_cast<pv4f *>(a.dX + off0 + static_cast<size_t>(i) * kTY * a.H));
    }
    return true;
  };

  // Four panels in flight, one step apart (see norm_panel_fwd.hip): loading p+3, sums of p+2 stored,
  // p+1 counted in at the barrier word, p finished.
  Stage b0, b1, b2, b3;
  load(b0, 0);
  if (npanels > 1) load(b1, 1);
  if (npanels > 2) load(b2, 2);
  publish(b0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  arrive(0);
  if (npanels > 1) publish(b1, 1);
  bool const elem = EXTRA && a.drop_mode == kDropElem;
  auto step = [&](Stage &cur, Stage &s1, Stage &s2, Stage &s3, int p) -> bool {
    (void)s1;
    // loads of panel p+3 first; then the partial of p+1 (stored a step ago) must have reached the L2: it is
    // older than the RPT stores of dX that ended the last step and than the loads just issued
    if (p + 3 < npanels) {
      load(s3, p + 3);
      if (p + 1 < npanels) {
        if (elem) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * RPT) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * RPT) : "memory");
      }
    } else if (p + 1 < npanels) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(RPT) : "memory");
    }
    if (p + 1 < npanels) arrive(p + 1);
    if (p + 2 < npanels) publish(s2, p + 2);
    return finish(cur, p);
  };
  bool ok = true;
  for (int p = 0; p < npanels && ok; p += 4) {
    ok = step(b0, b1, b2, b3, p);
    if (ok && p + 1 < npanels) ok = step(b1, b2, b3, b0, p + 1);
    if (ok && p + 2 < npanels) ok = step(b2, b3, b0, b1, p + 2);
    if (ok && p + 3 < npanels) ok = step(b3, b0, b1, b2, p + 3);
  }
  if (ok) panel_leave(who);
}

template <int ACT, int P, int RPT, bool EXTRA>
void launch_bwd(dlmi_ctx *ctx, PanelBwdArgs const &a) {
  hipLaunchKernelGGL((k_bwd_panel<ACT, P, RPT, EXTRA>), dim3(kPanelXcds * kPanelRanks), dim3(kPanelThreads), 0, ctx->stream, a);
}

}  // namespace

int panel_bwd_try(dlmi_ctx *ctx, size_t B, size_t H, BwdCall const &c, bool vec4, void *scratch, size_t scratch_bytes) {
  if (!ctx->panel_ok || !vec4 || c.xhat_given || c.dmean != nullptr || c.dstd != nullptr) return 0;
  if (H % 512 != 0) return 0;
  // 8192 rows: four panels of x and dn only fit the registers at 32 columns per panel, and rows cut into
  // 128-byte pieces stream slower than the multi-launch kernels (measured 113 us against 108 us at 8192 x 4096)
  // 1024 rows: no faster than the multi-launch pair in isolation (15 us both) and slower inside a step, where a
  // launch that needs every CU at once cannot start into the tail of the kernel before it
  if (B != 2048 && B != 4096) return 0;
  bool const extra = c.accumulate || c.drop_mode == kDropElem;
  if (c.drop_mode == kDropElem && (reinterpret_cast<uintptr_t>(c.mask) & 3u) != 0) return 0;
  // the caller's scratch (the context's block, already reserved, or the fixed array of the entry point that
  // allocates nothing): too small for the chunk partials means the multi-launch kernels
  if (scratch == nullptr || scratch_bytes < panel_scratch_bytes(H)) return 0;
  int rc;
  PanelBwdArgs a;
  a.x = c.x; a.dY = c.dY; a.gamma = c.gamma; a.beta = c.beta; a.mean = c.mean; a.stdv = c.stdv; a.r = c.r; a.d = c.d;
  a.mask = c.mask; a.dX = c.dX; a.dgamma = c.dgamma; a.dbeta = c.dbeta;
  a.B = B; a.H = H;
  a.batch_f = static_cast<float>(B); a.batch_scale = 1.0f / static_cast<float>(B); a.drop_scale = c.drop_scale;
  a.drop_mode = c.drop_mode; a.drop_bwd_masked = c.drop_bwd_masked; a.accumulate = c.accumulate ? 1 : 0;
  a.sync = panel_sync_of(ctx);
  a.part = static_cast<float *>(scratch);
  rc = panel_admit(ctx);
  if (rc <= 0) return rc;
  // rows per workgroup = B / 32 = RPT * 2048 / P
  DLMI_DISPATCH_ACT(c.act, {
    if (extra) {
      switch (B) {
        case 2048: launch_bwd<ACT, 64, 2, true>(ctx, a); break;
        default: launch_bwd<ACT, 32, 2, true>(ctx, a); break;  // 4096 rows
      }
    } else {
      switch (B) {
        case 2048: launch_bwd<ACT, 64, 2, false>(ctx, a); break;
        default: launch_bwd<ACT, 64, 4, false>(ctx, a); break;  // 4096 rows
      }
    }
  });
  DLMI_LAUNCH_CHECK(ctx, "k_bwd_panel");
  panel_launched(ctx);
  return 1;
}

}  // namespace dlmi
