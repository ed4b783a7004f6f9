// Backward of batch-(re)normalization + activation + dropout in ONE launch that reads dY and x once: the
// column panel scheme of norm_panel_common.hpp.  Per element the same arithmetic as the multi-launch path
// (bwd_dn; sums of bwp_st.cpp:1478-1506, coefficients and dx of bwp_st.cpp:1508-1531); dn is formed once and
// kept in registers between the reduction and the apply step instead of being recomputed.
//
// Geometry: 512 threads = P/4 column groups of 4 units x 2048/P rows; a workgroup owns B/32 = RPT * 2048/P rows
// and walks panels of P columns: P = 64 (256 B per row) while five panels of x and dn fit the registers, P = 32
// for 4096 rows with a per-element mask or an accumulating dX and for 8192 rows.  B in {2048, 4096, 8192}, H a
// multiple of 512 and at most 8 * kPanelMaxCols.  (32-, 64- and 128-column panels stream alike; the backward pass
// holds two values per element, so narrower panels buy more of them in flight.  The kernel beats the multi-launch
// pair because it moves 12 instead of 20 bytes per element.)
// On request the kernel also leaves the column sums of the dX rows each workgroup stored (the bias gradient of the
// layer below the normalization, update_derivative_fwp_st.cpp:283-302, as 32 partial rows for a small second launch).
#include <type_traits>

#include "norm_panel_common.hpp"

namespace dlmi {
namespace {


constexpr int kPanelMaxCols = 1024;  // columns of one XCD whose per-unit constants fit the workgroup's LDS (H <= 8192)

struct PanelBwdArgs {
  float const *x, *dY, *gamma, *beta, *mean, *stdv, *r, *d;
  uint8_t const *mask;
  float *dX, *dgamma, *dbeta;
  size_t B, H;
  float batch_f, batch_scale, drop_scale;
  int drop_mode, drop_bwd_masked, accumulate;
  PanelSync sync;
  float *part;  // [xcd][panel][rank][3][kP]
  float *db_part;  // optional [rank][H]: column sums of the dX rows each workgroup stores (the bias gradient's partials)
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
  // per-unit constants of ALL columns of this XCD (the forward's results), fetched once before the first panel:
  // mean, r/std, d, gamma, beta, std, r, per-unit keep mask.  A load of them inside a step would return behind
  // that step's bulk loads (a wavefront's loads return in issue order) and stall the arithmetic on them.
  __shared__ float cst[8][kPanelMaxCols];
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

  // The constants are asked for BEFORE the first panels (they arrive first: a wavefront's loads return in issue
  // order) and put into LDS once they are there, with the panels' loads still in flight.  A thread fetches the
  // constants of up to kCstPer columns; a column beyond the XCD's range, or a mask that does not exist, is fetched
  // from a valid address all the same (no conditional issue, see issue_load) and not used.
  constexpr int kCstPer = kPanelMaxCols / kPanelThreads;
  float cin[kCstPer][6];
  unsigned cmask[kCstPer];
  auto request_constants = [&] {
#pragma unroll
    for (int k = 0; k < kCstPer; ++k) {
      size_t const c = threadIdx.x + static_cast<size_t>(k) * kPanelThreads;
      size_t const at = col_base + (c < Hx ? c : 0);
      issue_load(cin[k][0], a.mean + at);
      issue_load(cin[k][1], a.stdv + at);
      issue_load(cin[k][2], a.r + at);
      issue_load(cin[k][3], a.d + at);
      issue_load(cin[k][4], a.gamma + at);
      issue_load(cin[k][5], a.beta + at);
      // (four mask bytes from the aligned word that holds this column's; without a per-unit mask: any valid word)
      issue_load(cmask[k], a.drop_mode == kDropUnit ? a.mask + (at & ~static_cast<size_t>(3)) : reinterpret_cast<uint8_t const *>(a.gamma));
    }
  };
  auto store_constants = [&](int younger) {
    wait_younger_n(younger);
#pragma unroll
    for (int k = 0; k < kCstPer; ++k) {
#pragma unroll
      for (int j = 0; j < 6; ++j) asm volatile("" : "+v"(cin[k][j]));
      asm volatile("" : "+v"(cmask[k]));
      size_t const c = threadIdx.x + static_cast<size_t>(k) * kPanelThreads;
      if (c < Hx) {
        float const sd = cin[k][1], rr = cin[k][2];
        cst[0][c] = cin[k][0];
        cst[1][c] = rr * fast_rcp(sd);
        cst[2][c] = cin[k][3];
        cst[3][c] = cin[k][4];
        cst[4][c] = cin[k][5];
        cst[5][c] = sd;
        cst[6][c] = rr;
        unsigned const byte = (cmask[k] >> (8u * static_cast<unsigned>((col_base + c) & 3u))) & 0xffu;
        cst[7][c] = a.drop_mode == kDropUnit ? (byte ? 1.0f : 0.0f) : 1.0f;
      }
    }
    __syncthreads();
  };

  struct Stage {
    pv4f x[RPT], g[RPT];          // x, and dY until publish() turns it into dn
    unsigned m[EXTRA ? RPT : 1];  // per-element keep mask, four bytes
  };
  bool const elem = EXTRA && a.drop_mode == kDropElem;
  auto load = [&](Stage &s, int p) {
    size_t const off0 = (row0 + ty) * a.H + col_base + static_cast<size_t>(p) * kP + tx * 4;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      size_t const off = off0 + static_cast<size_t>(i) * kTY * a.H;
      issue_load(s.x[i], a.x + off);
      issue_load(s.g[i], a.dY + off);
      if constexpr (EXTRA) {  // (always asked for, from a fixed valid address when there is no such mask)
        issue_load(s.m[i], elem ? a.mask + off : reinterpret_cast<uint8_t const *>(a.gamma));
      }
    }
  };
  // Before the first use of a stage: at most `younger` memory operations of this wavefront that were issued after
  // the stage's loads may still be outstanding.
  auto wait_stage = [&](Stage &s, int younger) {
    wait_younger_n(younger);
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      asm volatile("" : "+v"(s.x[i]), "+v"(s.g[i]));
      if constexpr (EXTRA) asm volatile("" : "+v"(s.m[i]));
    }
  };
  auto publish = [&](Stage &s, int p) {
    // per-unit constants of this thread's 4 columns
    int const lc = p * kP + tx * 4;  // column inside this XCD's range
    pv4f mu, rs, dd, ga, be;
    unsigned char umv[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mu[e] = cst[0][lc + e]; rs[e] = cst[1][lc + e]; dd[e] = cst[2][lc + e]; ga[e] = cst[3][lc + e];
      be[e] = cst[4][lc + e];
      umv[e] = cst[7][lc + e] != 0.0f ? 1 : 0;
    }
    pv4f s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0}, s2 = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      unsigned char mv[4] = {umv[0], umv[1], umv[2], umv[3]};
      if constexpr (EXTRA) {
        if (elem) {
          mv[0] = s.m[i] & 0xffu; mv[1] = (s.m[i] >> 8) & 0xffu; mv[2] = (s.m[i] >> 16) & 0xffu; mv[3] = s.m[i] >> 24;
        }
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
    // (the previous publish's readers are done with sh: at least one workgroup barrier lies between)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      sh[0][ty][tx * 4 + e] = s0[e];
      sh[1][ty][tx * 4 + e] = s1[e];
      sh[2][ty][tx * 4 + e] = s2[e];
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
  // ---- the exchange with the other workgroups, one step ahead of its use ------------------------------------
  // A wavefront's memory operations complete in the order they were issued, so a small load that everything
  // depends on completes behind every bulk load and every store issued before it.  The exchange is therefore
  // spread over a step: the count of arrivals for panel p + 1 is asked for in the middle of step p (the others
  // have had the first half of the step to count themselves in) and looked at when step p + 1 starts; the other
  // workgroups' sums of p + 1 are then requested, travel while step p + 1 forms the sums of p + 3, and are added
  // up after that.  Every wait names the younger operations of its wavefront that may
  // stay in flight (they differ between wavefronts: `stored` ones write a share of the workgroup's sums, `sums`
  // ones fetch the others' sums, wavefront 0 polls).
  int const wave_first = static_cast<int>(threadIdx.x & ~63u);
  bool const stored = wave_first < kVals;             // this wavefront issues the one store of publish()
  bool const sums = threadIdx.x < kRSplit * kVals;    // whole wavefronts: kRSplit * kVals is a multiple of 64
  int const extra = kRPer;                            // a thread's loads of the others' sums
  int const ld = EXTRA ? 3 * RPT : 2 * RPT;           // bulk loads of a panel per thread
  int const vc = threadIdx.x % kVals, rs = sums ? threadIdx.x / kVals : 0;
  float v[kRPer];
  // (every thread asks, the ones that do not add anything up for a share that others ask for as well: the
  // registers have no other definition than the loads' results, and every wavefront issues the same operations)
  auto request_sums = [&](int p) {  // every workgroup of this XCD has arrived for panel p
    float const *pp = a.part + (static_cast<size_t>(who.xcd) * npanels + p) * kPanelRanks * kVals + vc;
#pragma unroll
    for (int r = 0; r < kRPer; ++r) issue_load(v[r], pp + static_cast<size_t>(rs * kRPer + r) * kVals);
  };
  // (no other definition than the instruction's result: a value merged with another one would be copied at the
  // merge point, i.e. right behind the instruction, before the result has arrived)
  unsigned polled;
  auto poll_issue = [&](int p) {
    if (threadIdx.x == 0) {
      unsigned zero = 0;
      asm volatile("global_atomic_add %0, %1, %2, off sc0" : "=v"(polled) : "v"(panel_arrivals(who, p)), "v"(zero) : "memory");
    }
  };
  auto poll_check = [&](int p, int younger) {
    if (threadIdx.x == 0) {
      wait_younger_n(younger);
      asm volatile("" : "+v"(polled));
      unsigned const target = static_cast<unsigned>(kPanelRanks) * static_cast<unsigned>(p / 2 + 1);
      if (polled < target && !panel_wait(who, p)) s_ok = 0;  // somebody is late: poll until it has arrived
    }
  };
  // Finishes panel p from the sums requested a step ago; `younger`: operations issued after that request.
  auto finish = [&](Stage const &s, int p, int younger) {
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
    // every wavefront waits for what it asked for: a register whose load is still in flight must not be given
    // to another value
    wait_younger_n(younger);
#pragma unroll
    for (int r = 0; r < kRPer; ++r) asm volatile("" : "+v"(v[r]));
    if (sums) {
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
      int const lc = p * kP + c;
      float const ga = cst[3][lc], sd = cst[5][lc], rr = cst[6][lc];
      if (who.rank == 0) {
        // accumulating like the reference's derivative array; one addition per unit and launch, by this workgroup
        // alone, as an atomic without return value so that nothing here waits behind the loads in flight
        (void)__hip_atomic_fetch_add(a.dgamma + col + c, t0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        (void)__hip_atomic_fetch_add(a.dbeta + col + c, t1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      float const dm = (ga * t1) * (-rr / sd);
      float const ds = (ga * t2) * (-rr / (sd * sd));
      coef[0][c] = ga * (rr / sd);
      coef[1][c] = ds / (a.batch_f * sd);
      coef[2][c] = dm * a.batch_scale;
    }
    __syncthreads();
    pv4f mu, c1, c2, c3, colsum = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mu[e] = cst[0][p * kP + tx * 4 + e];
      c1[e] = coef[0][tx * 4 + e];
      c2[e] = coef[1][tx * 4 + e];
      c3[e] = coef[2][tx * 4 + e];
    }
    // (the column sums of dX only where they are asked for: one more addition per element)
    auto apply = [&](auto with_sums) {
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
          if constexpr (decltype(with_sums)::value) colsum[e] += dx;
        }
        __builtin_nontemporal_store(out, reinterpret_cast<pv4f *>(a.dX + off0 + static_cast<size_t>(i) * kTY * a.H));
      }
    };
    if (a.db_part != nullptr)
      apply(std::true_type{});
    else
      apply(std::false_type{});
    if (a.db_part != nullptr) {
      // column sums of this workgroup's rows of dX, in a fixed order: the rows of a wavefront by lane exchange,
      // the eight wavefronts through LDS (sh is free: publish's readers are two barriers back)
#pragma unroll
      for (int m = kCG; m < 64; m <<= 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) colsum[e] += __shfl_xor(colsum[e], m);
      }
      if ((threadIdx.x & 63u) < static_cast<unsigned>(kCG)) {
#pragma unroll
        for (int e = 0; e < 4; ++e) sh[0][threadIdx.x / 64][tx * 4 + e] = colsum[e];
      }
      __syncthreads();
      if (threadIdx.x < kP) {
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < kPanelThreads / 64; ++w) t += sh[0][w][threadIdx.x];
        a.db_part[static_cast<size_t>(who.rank) * a.H + col + threadIdx.x] = t;
      }
    }
  };

  // Five panels in flight, one step apart: p + 4 loading, p + 3 loaded, sums of p + 2 stored, p + 1 counted in at
  // the barrier word and its count asked for, p finished.
  Stage b0, b1, b2, b3, b4;
  auto clamped = [&](int p) { return p < npanels ? p : npanels - 1; };
  request_constants();
  load(b0, 0);
  load(b1, clamped(1));
  store_constants(2 * ld);  // the loads of panels 0 and 1 are younger
  wait_stage(b0, ld);       // panel 1's loads are younger
  publish(b0, 0);
  load(b2, clamped(2));
  load(b3, clamped(3));
  wait_younger_n(2 * ld);  // the partial of panel 0 is older than the loads of panels 2 and 3
  arrive(0);
  if (npanels > 1) {
    wait_stage(b1, 2 * ld);
    publish(b1, 1);
  }
  if (threadIdx.x == 0 && !panel_wait(who, 0)) s_ok = 0;
  __syncthreads();
  if (!s_ok) return;
  request_sums(0);
  auto step = [&](Stage &cur, Stage &s2, Stage &s4, int p) -> bool {
    bool const more1 = p + 1 < npanels, more2 = p + 2 < npanels, more4 = p + 4 < npanels;
    // younger than the store of publish(p + 1) and than the loads of panel p + 2, both issued before them: the
    // loads of panel p + 3 (if it exists; asked for in the prologue for p = 0), RPT stores of dX (not before the
    // first step)
    int const behind = (p == 0 || p + 3 < npanels ? ld : 0) + (p == 0 ? 0 : RPT);
    if (p > 0) {
      // the arrivals for panel p, asked for in the middle of the last step (the other workgroups had until then
      // to count themselves in).  Younger in wavefront 0: the loads of p + 3, RPT stores of dX
      poll_check(p, (p + 3 < npanels ? ld : 0) + RPT);
    }
    // the partial of p + 1 must have reached the L2 before this workgroup counts itself in (p = 0: only the
    // request for the sums of panel 0 is younger)
    if (more1) wait_younger_n(p == 0 ? extra : behind);
    __syncthreads();
    if (!s_ok) return false;
    if (more1) {
      if (threadIdx.x == 0) panel_count(panel_arrivals(who, p + 1));
    }
    if (p > 0) request_sums(p);
    if (more2) {
      wait_stage(s2, behind + extra);
      publish(s2, p + 2);
    }
    if (more1) poll_issue(p + 1);
    if (more4) load(s4, p + 4);
    // younger than the request for the sums of p: that store of publish, the loads just issued
    finish(cur, p, (more4 ? ld : 0) + (stored && more2 ? 1 : 0));
    return true;
  };
  bool ok = true;
  for (int p = 0; p < npanels && ok; p += 5) {
    ok = step(b0, b2, b4, p);
    if (ok && p + 1 < npanels) ok = step(b1, b3, b0, p + 1);
    if (ok && p + 2 < npanels) ok = step(b2, b4, b1, p + 2);
    if (ok && p + 3 < npanels) ok = step(b3, b0, b2, p + 3);
    if (ok && p + 4 < npanels) ok = step(b4, b1, b3, p + 4);
  }
  if (ok) panel_leave(who);
}

template <int ACT, int P, int RPT, bool EXTRA>
void launch_bwd(dlmi_ctx *ctx, PanelBwdArgs const &a) {
  hipLaunchKernelGGL((k_bwd_panel<ACT, P, RPT, EXTRA>), dim3(kPanelXcds * kPanelRanks), dim3(kPanelThreads), 0, ctx->stream, a);
}

}  // namespace

int panel_bwd_try(dlmi_ctx *ctx, size_t B, size_t H, BwdCall const &c, bool vec4, void *scratch, size_t scratch_bytes,
                  float **db_partials, unsigned *db_rows) {
  if (!ctx->panel_ok || !vec4 || c.xhat_given || c.dmean != nullptr || c.dstd != nullptr) return 0;
  if (H % 512 != 0 || H / kPanelXcds > static_cast<size_t>(kPanelMaxCols)) return 0;  // the per-unit constants of an XCD's columns live in LDS
  // 8192 rows: 32-column panels, and only without a mask stream or an accumulating dX (registers)
  // 1024 rows: no faster than the multi-launch pair in isolation (15 us both) and slower inside a step, where a
  // launch that needs every CU at once cannot start into the tail of the kernel before it
  bool const extra = c.accumulate || c.drop_mode == kDropElem;
  if (B != 2048 && B != 4096 && !(B == 8192 && !extra)) return 0;
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
  // the bias gradient's partials behind the chunk partials, where the caller asked for them and they fit: one row of
  // column sums per workgroup rank, added up by the caller's small second launch.  (dX accumulating: the sums must be
  // those of what ends up in dX, a pass over it follows instead.)
  size_t const db_offset = panel_db_offset(H);
  bool const db_here = db_partials != nullptr && c.db != nullptr && !c.accumulate &&
                       panel_scratch_bytes_db(H) <= scratch_bytes;
  a.db_part = db_here ? reinterpret_cast<float *>(static_cast<char *>(scratch) + db_offset) : nullptr;
  if (db_partials != nullptr) *db_partials = a.db_part;
  if (db_rows != nullptr) *db_rows = static_cast<unsigned>(kPanelRanks);
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
        case 8192: launch_bwd<ACT, 32, 4, false>(ctx, a); break;
        default: launch_bwd<ACT, 64, 4, false>(ctx, a); break;  // 4096 rows
      }
    }
  });
  DLMI_LAUNCH_CHECK(ctx, "k_bwd_panel");
  panel_launched(ctx);
  return 1;
}

}  // namespace dlmi
