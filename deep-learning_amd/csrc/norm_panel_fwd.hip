// Forward batch-(re)normalization + activation + dropout (+ shortcut) in ONE launch that reads x once:
// the column panel scheme described in norm_panel_common.hpp.  Same per-unit arithmetic as the multi-launch
// path (fwd_unit_stats: fwp_st.cpp:4709-4746; apply: fwp_st.cpp:4748-4794, 4830-4904, 5051-5112); the batch is
// summed in 32 chunks of B/32 rows, in rank order.
//
// Geometry: 512 threads = 32 column groups of 4 units x 16 rows; a workgroup owns B/32 = RPT * 16 rows and
// walks panels of 128 columns (512 B per row).  B in {1024, 2048, 4096, 8192}, H a multiple of 1024.
#include <cstdlib>
#include <mutex>

#include "norm_panel_common.hpp"

namespace dlmi {
namespace {

constexpr int kP = 128;               // columns per panel
constexpr int kCG = kP / 4;           // column groups (float4) per panel row
constexpr int kTY = kPanelThreads / kCG;  // rows per sweep of the workgroup: 16
constexpr int kRSplit = kPanelThreads / (2 * kP);  // threads per (statistic, column) in the rank sum: 2
constexpr int kRPer = kPanelRanks / kRSplit;

struct PanelFwdArgs {
  float const *x, *gamma, *beta, *residual;
  uint8_t const *mask;
  float *y;
  size_t B, H;
  FwdFinalize fin;
  int drop_mode;
  float drop_scale;
  PanelSync sync;
  float *part;  // [xcd][panel][rank][2][kP]
};

// EXTRA: the launch may read a per-element mask and / or a shortcut tensor (more registers per thread)
template <int ACT, int RPT, bool EXTRA>
__global__ __launch_bounds__(kPanelThreads) void k_fwd_panel(PanelFwdArgs a) {
  __shared__ float sh[2][kTY][kP];        // per-sweep-row column sums of the panel being published
  __shared__ float sh2[kRSplit][2 * kP];  // halves of the rank sum
  __shared__ float snap[2][2][kP];        // moving mean / std of the two panels in flight, as they were
  __shared__ float coef[3][kP];           // mean, gamma*r/std, gamma*d+beta of the panel being applied
  __shared__ unsigned s_rank, s_ok;
  PanelWho who;
  if (threadIdx.x == 0) s_ok = 1;
  if (!panel_enter(a.sync, who, &s_rank)) return;
  int const tx = threadIdx.x % kCG, ty = threadIdx.x / kCG;
  size_t const Hx = a.H / kPanelXcds;
  int const npanels = static_cast<int>(Hx / kP);
  size_t const row0 = static_cast<size_t>(who.rank) * (RPT * kTY);
  size_t const col_base = static_cast<size_t>(who.xcd) * Hx;

  auto load = [&](pv4f (&buf)[RPT], int p) {
    float const *src = a.x + (row0 + ty) * a.H + col_base + static_cast<size_t>(p) * kP + tx * 4;
#pragma unroll
    for (int i = 0; i < RPT; ++i)
      buf[i] = __builtin_nontemporal_load(reinterpret_cast<pv4f const *>(src + static_cast<size_t>(i) * kTY * a.H));
  };
  // the sums of this workgroup's rows of panel p -> its chunk partial; the moving statistics of the panel
  // are read here, before this workgroup arrives, i.e. before any workgroup can have replaced them
  auto publish = [&](pv4f const (&buf)[RPT], int p) {
    pv4f s = {0, 0, 0, 0}, q = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      s += buf[i];
      q += buf[i] * buf[i];
    }
    __syncthreads();  // the previous publish's readers are done with sh
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      sh[0][ty][tx * 4 + e] = s[e];
      sh[1][ty][tx * 4 + e] = q[e];
    }
    __syncthreads();
    size_t const col = col_base + static_cast<size_t>(p) * kP;
    if (threadIdx.x < 2 * kP) {
      int const w = threadIdx.x / kP, c = threadIdx.x % kP;
      float t = 0.0f;
#pragma unroll
      for (int j = 0; j < kTY; ++j) t += sh[w][j][c];
      a.part[((static_cast<size_t>(who.xcd) * npanels + p) * kPanelRanks + who.rank) * 2 * kP + w * kP + c] = t;
    } else if (threadIdx.x < 4 * kP) {
      int const w = (threadIdx.x - 2 * kP) / kP, c = threadIdx.x % kP;
      snap[p & 1][w][c] = w == 0 ? a.fin.mov_mean[col + c] : a.fin.mov_std[col + c];
    }
  };
  auto arrive = [&](int p) {
    __syncthreads();
    if (threadIdx.x == 0) panel_count(panel_arrivals(who, p));
  };
  // wait for the XCD, finish the statistics of panel p and apply them to the rows in registers
  auto finish = [&](pv4f const (&buf)[RPT], int p) -> bool {
    size_t const col = col_base + static_cast<size_t>(p) * kP;
    size_t const off0 = (row0 + ty) * a.H + col + tx * 4;
    // streams that do not depend on the statistics start before the wait
    pv4f res[EXTRA ? RPT : 1];
    uchar4 mk[EXTRA ? RPT : 1];
    if constexpr (EXTRA) {
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        size_t const off = off0 + static_cast<size_t>(i) * kTY * a.H;
        if (a.residual != nullptr) res[i] = __builtin_nontemporal_load(reinterpret_cast<pv4f const *>(a.residual + off));
        if (a.drop_mode == kDropElem) mk[i] = *reinterpret_cast<uchar4 const *>(a.mask + off);
      }
    }
    pv4f ga = *reinterpret_cast<pv4f const *>(a.gamma + col + tx * 4);
    pv4f be = *reinterpret_cast<pv4f const *>(a.beta + col + tx * 4);
    uchar4 um = make_uchar4(1, 1, 1, 1);
    if (a.drop_mode == kDropUnit) um = *reinterpret_cast<uchar4 const *>(a.mask + col + tx * 4);
    if (threadIdx.x == 0 && !panel_wait(who, p)) s_ok = 0;
    __syncthreads();
    if (!s_ok) return false;
    {
      int const vc = threadIdx.x % (2 * kP), rs = threadIdx.x / (2 * kP);
      float const *pp = a.part + (static_cast<size_t>(who.xcd) * npanels + p) * kPanelRanks * 2 * kP + vc;
      float v[kRPer];
#pragma unroll
      for (int r = 0; r < kRPer; ++r) v[r] = __builtin_nontemporal_load(pp + static_cast<size_t>(rs * kRPer + r) * 2 * kP);
      float t = 0.0f;
#pragma unroll
      for (int r = 0; r < kRPer; ++r) t += v[r];
      sh2[rs][vc] = t;
    }
    __syncthreads();
    if (threadIdx.x < kP) {
      int const c = threadIdx.x;
      float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
      for (int j = 0; j < kRSplit; ++j) {
        s1 += sh2[j][c];
        s2 += sh2[j][kP + c];
      }
      UnitStats const u = fwd_unit_stats(a.fin, s1, s2, snap[p & 1][0][c], snap[p & 1][1][c]);
      if (who.rank == 0) store_unit_stats(a.fin, col + c, u);
      float const inv = fast_rcp(u.stdv);
      coef[0][c] = u.mean;
      coef[1][c] = u.r * inv;  // r / std; gamma joins below, per thread
      coef[2][c] = u.d;
    }
    __syncthreads();
    pv4f mu, rr, dd;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mu[e] = coef[0][tx * 4 + e];
      rr[e] = ga[e] * coef[1][tx * 4 + e];       // gamma * r / std
      dd[e] = ga[e] * coef[2][tx * 4 + e] + be[e];  // gamma * d + beta
    }
    unsigned char const umv[4] = {um.x, um.y, um.z, um.w};
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      size_t const off = off0 + static_cast<size_t>(i) * kTY * a.H;
      unsigned char mv[4] = {umv[0], umv[1], umv[2], umv[3]};
      if constexpr (EXTRA) {
        if (a.drop_mode == kDropElem) { mv[0] = mk[i].x; mv[1] = mk[i].y; mv[2] = mk[i].z; mv[3] = mk[i].w; }
      }
      pv4f out;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float const nn = (buf[i][e] - mu[e]) * rr[e] + dd[e];
        float q = act_fire<ACT>(nn);
        if (a.drop_mode != kDropNone) q = drop_apply(mv[e], a.drop_scale, q);
        if constexpr (EXTRA) {
          if (a.residual != nullptr) {
            asm volatile("" : "+v"(q));  // a rounding of its own, as in the multi-launch path
            q = res[i][e] + q;
          }
        }
        out[e] = q;
      }
      __builtin_nontemporal_store(out, reinterpret_cast<pv4f *>(a.y + off));
    }
    return true;
  };

  pv4f b0[RPT], b1[RPT], b2[RPT];
  load(b0, 0);
  if (npanels > 1) load(b1, 1);
  publish(b0, 0);
  // The partial of panel 0 was stored AFTER the loads of panel 1 were issued, so a counted wait would let it
  // pass while still in flight: everything must have completed before this workgroup counts itself in (the
  // rows of panel 1 are needed by the very next publish anyway).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  arrive(0);
  auto step = [&](pv4f (&cur)[RPT], pv4f (&mid)[RPT], pv4f (&nxt)[RPT], int p) -> bool {
    if (p + 1 < npanels) {
      publish(mid, p + 1);
      if (p + 2 < npanels) {
        load(nxt, p + 2);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(RPT) : "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      arrive(p + 1);
    }
    return finish(cur, p);
  };
  bool ok = true;
  for (int p = 0; p < npanels && ok; p += 3) {
    ok = step(b0, b1, b2, p);
    if (ok && p + 1 < npanels) ok = step(b1, b2, b0, p + 1);
    if (ok && p + 2 < npanels) ok = step(b2, b0, b1, p + 2);
  }
  if (ok) panel_leave(who);
}

// one workgroup per CU reports where it runs
__global__ __launch_bounds__(64) void k_panel_probe(unsigned *out) {
  if (threadIdx.x == 0) out[blockIdx.x] = panel_xcc_id();
}

std::mutex g_order_mutex;
struct DeviceOrder {
  hipEvent_t event = nullptr;
  hipStream_t stream = nullptr;  // the stream of the last panel launch outside a capture
  bool recorded = false;
  // the stream (and its context) that has recorded a panel kernel into a HIP graph: replays of that graph are
  // not seen here, so no other stream of the device may launch panel kernels while this owner exists
  hipStream_t graph_owner = nullptr;
  dlmi_ctx const *graph_owner_ctx = nullptr;
};
DeviceOrder g_order[64];
DeviceOrder &order_of(dlmi_ctx const *ctx) { return g_order[ctx->device >= 0 && ctx->device < 64 ? ctx->device : 0]; }

template <int ACT, int RPT, bool EXTRA>
void launch_fwd(dlmi_ctx *ctx, PanelFwdArgs const &a) {
  hipLaunchKernelGGL((k_fwd_panel<ACT, RPT, EXTRA>), dim3(kPanelXcds * kPanelRanks), dim3(kPanelThreads), 0, ctx->stream, a);
}

}  // namespace

int panel_init(dlmi_ctx *ctx) {
  ctx->panel_ok = 0;
  char const *e = std::getenv("DLMI_NORM_PANEL");
  if (e != nullptr && std::atoi(e) == 0) return DLMI_OK;
  if (ctx->num_cu != kPanelXcds * kPanelRanks) return DLMI_OK;  // another part or partition mode: multi-launch path
  // the bound of every wait, in polls; a small value lets a test drive the give-up branch from the host
  ctx->panel_spin_limit = kPanelSpinLimit;
  if (char const *l = std::getenv("DLMI_PANEL_SPIN_LIMIT"); l != nullptr && std::atoi(l) > 0) ctx->panel_spin_limit = std::atoi(l);
  void *p = nullptr;
  DLMI_HIP(ctx, hipMalloc(&p, (kPanelStateWords + kPanelXcds * kPanelRanks) * sizeof(unsigned)));
  ctx->panel_state = static_cast<unsigned *>(p);
  DLMI_HIP(ctx, hipMemsetAsync(ctx->panel_state, 0, (kPanelStateWords + kPanelXcds * kPanelRanks) * sizeof(unsigned), ctx->stream));
  // two words of pinned, device-visible host memory for the give-up reports
  void *h = nullptr, *hd = nullptr;
  DLMI_HIP(ctx, hipHostMalloc(&h, 64, hipHostMallocMapped));
  ctx->panel_flag_host = static_cast<unsigned *>(h);
  ctx->panel_flag_host[0] = ctx->panel_flag_host[1] = 0;
  DLMI_HIP(ctx, hipHostGetDevicePointer(&hd, h, 0));
  ctx->panel_flag_dev = static_cast<unsigned *>(hd);
  unsigned *where = ctx->panel_state + kPanelStateWords;
  hipLaunchKernelGGL(k_panel_probe, dim3(kPanelXcds * kPanelRanks), dim3(64), 0, ctx->stream, where);
  DLMI_LAUNCH_CHECK(ctx, "k_panel_probe");
  unsigned host[kPanelXcds * kPanelRanks];
  DLMI_HIP(ctx, hipMemcpyAsync(host, where, sizeof host, hipMemcpyDeviceToHost, ctx->stream));
  DLMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
  int count[16] = {0};
  for (unsigned v : host) ++count[v & 0xf];
  bool even = true;
  for (int i = 0; i < 16; ++i) even = even && count[i] == (i < kPanelXcds ? kPanelRanks : 0);
  ctx->panel_ok = even ? 1 : 0;
  return DLMI_OK;
}

void panel_destroy(dlmi_ctx *ctx) {
  if (ctx->panel_state != nullptr) (void)hipFree(ctx->panel_state);
  if (ctx->panel_flag_host != nullptr) (void)hipHostFree(ctx->panel_flag_host);
  ctx->panel_state = nullptr;
  ctx->panel_flag_host = ctx->panel_flag_dev = nullptr;
  ctx->panel_ok = 0;
}

// Panel kernels of different streams must not run side by side (each needs all its workgroups resident).
// As long as one stream launches them, nothing is done.  When a launch comes from another stream than the
// previous one, an event is recorded on the previous stream - behind its last panel kernel - and the new
// stream waits for it.  Stream capture: a kernel recorded into a graph runs whenever the graph is replayed,
// which this library does not see, so no event can order it.  The first stream of a device that records a
// panel kernel therefore becomes the only one that may launch them at all: while it holds that role, panel
// launches of any other stream (recorded or not) are refused and take the multi-launch kernels, and it gives
// the role up when its context is destroyed or given another stream.  A capture on a stream while ANOTHER
// stream has panel kernels in flight outside a capture is refused as well.
static bool panel_capturing(hipStream_t s) {
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &cs) != hipSuccess) { (void)hipGetLastError(); return true; }
  return cs != hipStreamCaptureStatusNone;
}
int panel_admit(dlmi_ctx *ctx) {
  std::lock_guard<std::mutex> lock(g_order_mutex);
  DeviceOrder &o = order_of(ctx);
  if (o.graph_owner_ctx != nullptr && o.graph_owner != ctx->stream) return 0;
  if (panel_capturing(ctx->stream)) {
    if (o.recorded && o.stream != ctx->stream) return 0;  // another stream's panel kernels may still be running
    o.graph_owner = ctx->stream;
    o.graph_owner_ctx = ctx;
    return 1;
  }
  if (!o.recorded || o.stream == ctx->stream) return 1;
  if (o.event == nullptr) DLMI_HIP(ctx, hipEventCreateWithFlags(&o.event, hipEventDisableTiming));
  DLMI_HIP(ctx, hipEventRecord(o.event, o.stream));
  DLMI_HIP(ctx, hipStreamWaitEvent(ctx->stream, o.event, 0));
  return 1;
}
void panel_launched(dlmi_ctx *ctx) {
  std::lock_guard<std::mutex> lock(g_order_mutex);
  DeviceOrder &o = order_of(ctx);
  if (o.graph_owner == ctx->stream && o.graph_owner_ctx == ctx && panel_capturing(ctx->stream)) {
    ctx->panel_in_graph = 1;
    return;  // nothing was launched: the kernel runs when the graph does
  }
  o.stream = ctx->stream;
  o.recorded = true;
}

void panel_release_stream(dlmi_ctx *ctx) {
  std::lock_guard<std::mutex> lock(g_order_mutex);
  DeviceOrder &o = order_of(ctx);
  if (o.graph_owner_ctx == ctx) {
    // graphs recorded on this stream must not be replayed once the context has let go of it
    o.graph_owner = nullptr;
    o.graph_owner_ctx = nullptr;
  }
  if (!o.recorded || o.stream != ctx->stream) return;
  // nothing of this stream is still running (the caller synchronized it): a later launch from another stream
  // has nothing to wait for, and must not touch a stream handle that may be gone by then
  o.recorded = false;
  o.stream = nullptr;
}

// After the stream has been synchronized: did a panel kernel give up, or find the words of an earlier give-up?
// Then the results of the calls since the last check are not valid; the words are cleared and the context
// stays on the multi-launch path.  Costs two reads of host memory when nothing happened.
int panel_check(dlmi_ctx *ctx) {
  if (ctx->panel_flag_host == nullptr) return DLMI_OK;
  unsigned volatile *const flag = ctx->panel_flag_host;
  unsigned const gave_up = flag[0], found_stale = flag[1];
  if (gave_up == 0 && found_stale == 0) return DLMI_OK;
  flag[0] = 0;
  flag[1] = 0;
  ctx->panel_ok = 0;
  (void)hipMemset(ctx->panel_state, 0, kPanelStateWords * sizeof(unsigned));
  return dlmi_fail(ctx, DLMI_E_HIP,
                   "a single-launch normalization kernel did not see all of its workgroups resident and gave up "
                   "(another kernel held compute units for too long)%s: the results of the calls since the last "
                   "synchronization are not valid; this context uses the multi-launch kernels from now on",
                   found_stale != 0 ? ", and later launches found its barrier words still in place" : "");
}

size_t panel_scratch_bytes(size_t H) { return static_cast<size_t>(kPanelRanks) * 3 * H * sizeof(float) + 4096; }
size_t panel_db_offset(size_t H) { return (panel_scratch_bytes(H) + 255) & ~static_cast<size_t>(255); }
size_t panel_scratch_bytes_db(size_t H) { return panel_db_offset(H) + static_cast<size_t>(kPanelRanks) * H * sizeof(float); }

int panel_fwd_try(dlmi_ctx *ctx, size_t B, size_t H, FwdTrainCall const &c, bool vec4, void *scratch, size_t scratch_bytes) {
  if (!ctx->panel_ok || !vec4 || c.partial_in != nullptr || c.xhat != nullptr || c.nrm != nullptr || c.y == nullptr) return 0;
  if (H % (static_cast<size_t>(kPanelXcds) * kP) != 0 || B % (static_cast<size_t>(kPanelRanks) * kTY) != 0) return 0;
  size_t const rpt = B / (static_cast<size_t>(kPanelRanks) * kTY);
  if (rpt != 2 && rpt != 4 && rpt != 8 && rpt != 16) return 0;
  bool const extra = c.residual != nullptr || c.drop_mode == kDropElem;
  if (extra && rpt == 16) return 0;  // the three panels in flight plus the extra streams do not fit the registers
  if (c.drop_mode == kDropElem && (reinterpret_cast<uintptr_t>(c.mask) & 3u) != 0) return 0;
  // the caller's scratch (the context's block, already reserved, or the fixed array of the entry point that
  // allocates nothing): too small for the chunk partials means the multi-launch kernels
  if (scratch == nullptr || scratch_bytes < panel_scratch_bytes(H)) return 0;
  int rc;
  PanelFwdArgs a;
  a.x = c.x; a.gamma = c.gamma; a.beta = c.beta; a.residual = c.residual; a.mask = c.mask; a.y = c.y;
  a.B = B; a.H = H;
  a.fin.mean = c.mean; a.fin.stdv = c.stdv; a.fin.mov_mean = c.mov_mean; a.fin.mov_std = c.mov_std; a.fin.r = c.r; a.fin.d = c.d;
  a.fin.batch_scale = 1.0f / static_cast<float>(B);
  a.fin.momentum = c.momentum; a.fin.eps = c.eps; a.fin.r_max = c.r_max; a.fin.d_max = c.d_max;
  a.fin.renorm = c.norm == DLMI_NORM_BATCH_RENORM ? 1 : 0;
  a.drop_mode = c.drop_mode; a.drop_scale = c.drop_scale;
  a.sync = panel_sync_of(ctx);
  a.part = static_cast<float *>(scratch);
  rc = panel_admit(ctx);
  if (rc <= 0) return rc;
  DLMI_DISPATCH_ACT(c.act, {
    if (extra) {
      switch (rpt) {
        case 2: launch_fwd<ACT, 2, true>(ctx, a); break;
        case 4: launch_fwd<ACT, 4, true>(ctx, a); break;
        default: launch_fwd<ACT, 8, true>(ctx, a); break;
      }
    } else {
      switch (rpt) {
        case 2: launch_fwd<ACT, 2, false>(ctx, a); break;
        case 4: launch_fwd<ACT, 4, false>(ctx, a); break;
        case 8: launch_fwd<ACT, 8, false>(ctx, a); break;
        default: launch_fwd<ACT, 16, false>(ctx, a); break;
      }
    }
  });
  DLMI_LAUNCH_CHECK(ctx, "k_fwd_panel");
  panel_launched(ctx);
  return 1;
}

}  // namespace dlmi
