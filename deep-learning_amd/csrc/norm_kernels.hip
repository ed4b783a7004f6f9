// Batch normalization / batch renormalization kernels (training forward and
// backward, fused with the activation and the dropout mask) for gfx950.
//
// All of them are bound by HBM bandwidth, so the design goal is the minimum
// number of passes over the [B, H] tensors with fully coalesced 16-byte
// accesses, enough independent loads in flight per CU and few enough ALU
// instructions per element that the vector units never become the limit:
//
//   forward : statistics (read x)      -> [finalize H] -> apply (read x, write y)
//   backward: reduce (read dY, x)      -> [finalize H] -> apply (read dY, x, write dX)
//
// x_hat, the pre-activation n = gamma*x_hat + beta and the activation output
// are recomputed in registers instead of being stored and re-read.
//
// Thread geometry of the column passes: a 256-thread block is TX x TY; a
// thread owns VEC (=4, one float4) adjacent units and walks rows with stride
// TY.  Rows that share a wavefront are combined with wavefront shuffles, the
// four wavefronts of the block with a small LDS tree, the chunks of the batch
// in chunk order.  No float atomics, a fixed summation order: results are
// reproducible run to run.
//
// Who combines the chunks.  Where the shape allows at most 16 chunks per unit
// and still a block on most compute units (any layer a few thousand units
// wide), there is NO finalize launch: every block of the apply pass adds the
// 16 partial sums of its own units in its prologue (they sit in L2) and does
// the per-unit arithmetic itself; the blocks of one chunk store the per-unit
// results, and the statistics pass leaves a snapshot of the moving statistics
// so that every block sees them as they were before the step.  Tall, narrow
// tensors need many chunks to fill the machine: there a small finalize kernel
// combines them (TY lanes per unit, then an LDS tree) between the two passes.
// Both alternatives to this were built and measured on MI355X and rejected:
// (a) the reduction's last block of a column group (found with a device-scope
//     ticket) doing the finalize: its chain of device-scope round trips, about
//     2 us each across XCDs, made the statistics pass 22.8 us at [4096 x 4096]
//     against 12.7 + 4.4 us for two launches;
// (b) one launch per direction with a grid-wide barrier and the block's share
//     of x kept in registers (8 instead of 12 B/element forward): forward 36 us
//     against 38, backward 73 us against 58 at [4096 x 4096] - the barrier's
//     round trips and the low occupancy of 1024-thread register-heavy blocks
//     cost more than the saved re-read.
// The apply kernels have nothing to reduce and use TX = 256 when H allows, so
// that every load / store instruction of a block covers 4 KiB of one row.
//
// Everything that is uniform over a launch and would put a branch between two
// loads (dropout mode, materialising x_hat) is a template parameter: a branch
// there makes the compiler wait for each load before issuing the next.
//
// Citations: /root/reference/lib/deep-learning/v1/learner/.
#include <cstdlib>
#include <initializer_list>
#include <mutex>

#include "activations.hpp"
#include "dlmi_common.hpp"
#include "norm_shared.hpp"

// Reduction scratch of the entry point that allocates nothing
// (dlmi_fused_norm_act_fwd_noalloc): part of the code object, so every GPU the
// library runs on holds its own copy from module load until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; the
// device address it yields (per device) is what kernels and copies are given.
constexpr size_t kStaticScratchBytes = size_t(2) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace dlmi {

constexpr int kMaxDevices = 64;
static void *g_static_scratch[kMaxDevices] = {nullptr};
static std::mutex g_static_scratch_mutex;
// Every call of the entry point that allocates nothing uses the device's one array, so calls from different
// streams must not overlap.  The stream of the last such call is remembered per device; a call from another stream
// (outside a stream capture) first makes its stream wait for an event recorded behind that call.  The event is
// created with the first context of the device, so the entry point itself creates nothing.
struct StaticScratchOrder {
  hipEvent_t event = nullptr;
  hipStream_t stream = nullptr;
  bool used = false;
};
static StaticScratchOrder g_static_order[kMaxDevices];

// Called by dlmi_ctx_create with the context's device current: looks up, once
// per device, where that device keeps its copy of the static scratch array.
int static_scratch_init(dlmi_ctx *ctx) {
  if (ctx->device < 0 || ctx->device >= kMaxDevices)
    return dlmi_fail(ctx, DLMI_E_UNSUPPORTED, "device ordinal %d beyond %d", ctx->device, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (g_static_scratch[ctx->device] == nullptr) {
    void *p = nullptr;
    hipError_t const e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return dlmi_fail(ctx, DLMI_E_HIP, "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
    }
    g_static_scratch[ctx->device] = p;
  }
  if (g_static_order[ctx->device].event == nullptr &&
      hipEventCreateWithFlags(&g_static_order[ctx->device].event, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    g_static_order[ctx->device].event = nullptr;  // calls from several streams then race, as documented
  }
  ctx->static_scratch = static_cast<char *>(g_static_scratch[ctx->device]);
  ctx->static_scratch_bytes = kStaticScratchBytes;
  return DLMI_OK;
}

static bool stream_capturing(hipStream_t s) {
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &cs) != hipSuccess) { (void)hipGetLastError(); return true; }
  return cs != hipStreamCaptureStatusNone;
}
// Before a call that uses the device's static scratch array: orders it behind the last one of another stream.
static int static_scratch_order(dlmi_ctx *ctx) {
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  StaticScratchOrder &o = g_static_order[ctx->device];
  if (o.event != nullptr && o.used && o.stream != ctx->stream && !stream_capturing(ctx->stream) && !stream_capturing(o.stream)) {
    DLMI_HIP(ctx, hipEventRecord(o.event, o.stream));
    DLMI_HIP(ctx, hipStreamWaitEvent(ctx->stream, o.event, 0));
  }
  o.stream = ctx->stream;
  o.used = true;
  return DLMI_OK;
}
// The context lets go of its stream (which its owner may destroy next; its work has completed).
void static_scratch_release_stream(dlmi_ctx *ctx) {
  if (ctx->device < 0 || ctx->device >= kMaxDevices) return;
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  StaticScratchOrder &o = g_static_order[ctx->device];
  if (o.used && o.stream == ctx->stream) {
    o.used = false;
    o.stream = nullptr;
  }
}

constexpr int kBlock = 256;
constexpr int kWave = 64;

struct ColGeom {
  int vec;  // 4 (float4 path) or 1 (any H, any alignment)
  int tx_log2;
  unsigned grid_x;
  unsigned nchunks;
  size_t rows_per_chunk;
};

// A region of device memory the reduction kernels may use for partial sums and
// the backward coefficients.
struct ScratchView {
  char *data;
  size_t data_bytes;
};

static size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Geometry of a reduction pass over [B, H] with `nplanes` sums per unit: blocks
// as wide as the cap allows (TX column groups, up to 256: every load of a block
// then covers 4 KiB of one row), a few blocks per compute unit, each thread
// walking at least reduce_min_rows rows.
static ColGeom reduce_geometry(dlmi_ctx const *ctx, size_t B, size_t H, bool vec4, int nplanes, size_t data_bytes,
                               int tx_cap = 0, size_t max_chunks = 65535) {
  dlmi_tuning const &t = ctx->tune;
  ColGeom g;
  g.vec = vec4 ? 4 : 1;
  size_t const groups = dlmi_ceil_div(H, g.vec);
  if (tx_cap == 0) {
    tx_cap = t.reduce_tx_cap;
    // Few units under a tall batch (65536 x 256): blocks of 16 column groups instead of 64 mean four times fewer
    // chunks for the same number of blocks, and the finalize launch that adds the chunks up is what such a shape
    // pays for (64 instead of 256 chunks: forward 38.5 -> 37.4 us, backward 58.1 -> 56.9 us)
    if (vec4 && groups <= 64 && tx_cap > t.reduce_tx_cap_few_units) tx_cap = t.reduce_tx_cap_few_units;
  }
  int tx = 256;
  g.tx_log2 = 8;
  while (tx > 1 && (tx > tx_cap || static_cast<size_t>(tx / 2) >= groups)) {
    tx /= 2;
    --g.tx_log2;
  }
  int const ty = kBlock / tx;
  g.grid_x = static_cast<unsigned>(dlmi_ceil_div(groups, tx));
  size_t want = dlmi_ceil_div(static_cast<size_t>(ctx->num_cu) * t.reduce_blocks_per_cu, g.grid_x);
  size_t const max_by_rows = B / (static_cast<size_t>(ty) * t.reduce_min_rows);
  if (want > max_by_rows) want = max_by_rows;
  // partial sums [nplanes][nchunks][H] must fit the data region (beside 3*H coefficients)
  size_t const fixed = round_up(3 * H * sizeof(float), 256);
  size_t const max_by_scratch =
      data_bytes > fixed ? (data_bytes - fixed) / (static_cast<size_t>(nplanes) * H * sizeof(float)) : 0;
  if (want > max_by_scratch) want = max_by_scratch;
  if (want > max_chunks) want = max_chunks;
  if (want < 1) want = 1;
  if (want > 65535) want = 65535;
  g.rows_per_chunk = dlmi_ceil_div(B, want);
  g.nchunks = static_cast<unsigned>(dlmi_ceil_div(B, g.rows_per_chunk));
  return g;
}

// Reduction geometry for the two-launch scheme (the apply pass does the per-unit arithmetic from the
// partial sums): at most kFoldChunks chunks, blocks as narrow as it takes (64, 32 or 16 column groups)
// to still put a block on most compute units.  False when the shape cannot give both (few units, many
// rows): the finalize kernel then combines as many chunks as the reduction wants.
constexpr size_t kFoldChunks = kNormFoldChunks;
static bool fold_geometry(dlmi_ctx const *ctx, size_t B, size_t H, bool vec4, int nplanes, size_t data_bytes,
                          ColGeom *g) {
  int const level = nplanes == 3 ? ctx->tune.fold_bwd : ctx->tune.fold_fwd;
  if (level <= 0 || (level == 1 && B * H > ctx->tune.fold_fwd_max_elements)) return false;
  for (int tx = 64; tx >= 16; tx /= 2) {
    *g = reduce_geometry(ctx, B, H, vec4, nplanes, data_bytes, tx, kFoldChunks);
    size_t const blocks = static_cast<size_t>(g->grid_x) * g->nchunks;
    if (blocks * 4 >= static_cast<size_t>(ctx->num_cu) * 3) return true;
    // small batches never need more chunks than this: few blocks are then all there is to have
    size_t const ty = kBlock >> g->tx_log2;
    if (B / (ty * ctx->tune.reduce_min_rows) <= kFoldChunks) return true;
  }
  return false;
}

// Geometry of an apply pass: as wide as the row allows (TX up to 256), a few
// blocks per compute unit, each walking its share of the rows.
static ColGeom apply_geometry(dlmi_ctx const *ctx, size_t B, size_t H, bool vec4, int blocks_per_cu) {
  dlmi_tuning const &t = ctx->tune;
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
  size_t want = dlmi_ceil_div(static_cast<size_t>(ctx->num_cu) * blocks_per_cu, g.grid_x);
  size_t const max_by_rows = B / (static_cast<size_t>(ty) * t.apply_min_rows);
  if (want > max_by_rows) want = max_by_rows;
  if (want < 1) want = 1;
  if (want > 65535) want = 65535;
  g.rows_per_chunk = dlmi_ceil_div(B, want);
  g.nchunks = static_cast<unsigned>(dlmi_ceil_div(B, g.rows_per_chunk));
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

// The rows of one thread: first, first + step, ... (count of them).  A block
// either owns a contiguous chunk of rows_per_chunk rows (walked with stride TY)
// or, with rows_per_chunk == 0, every gridDim.y-th group of TY rows: all blocks
// of the launch then sweep through memory together as one moving window.
// (B < 2^32 rows; 32-bit arithmetic and shifts: a 64-bit division here costs
// every thread a hundred instructions before its first load.)
struct RowWalk {
  size_t first, step;
  unsigned count;
};
// `reverse`: block y takes the chunk gridDim.y-1-y.  The apply passes walk the batch from its end: what
// the reduction pass before them read LAST is what the memory-side cache still holds.
__device__ __forceinline__ RowWalk row_walk(size_t B, size_t rows_per_chunk, int tx_log2, int ty, bool reverse = false) {
  int const ty_log2 = 8 - tx_log2;
  unsigned const by = reverse ? gridDim.y - 1u - blockIdx.y : blockIdx.y;
  RowWalk w;
  if (rows_per_chunk == 0) {
    unsigned const first = (by << ty_log2) + ty;
    unsigned const step = gridDim.y << ty_log2;
    w.first = first;
    w.step = step;
    w.count = first < B ? (static_cast<unsigned>(B) - first + step - 1) / step : 0u;
  } else {
    size_t const b0 = by * rows_per_chunk;
    size_t const b1 = (b0 + rows_per_chunk < B) ? b0 + rows_per_chunk : B;
    w.first = b0 + ty;
    w.step = size_t(1) << ty_log2;
    w.count = w.first < b1 ? static_cast<unsigned>((b1 - w.first + w.step - 1) >> ty_log2) : 0u;
  }
  return w;
}

// Keeps the instruction scheduler from moving anything across this point: the
// loads of a batch of rows stay ahead of the arithmetic on them.
__device__ __forceinline__ void sched_fence() { __builtin_amdgcn_sched_barrier(0); }

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

// Column totals of NP planes of partial sums [NP][nchunks][H] for the block's
// TX column groups: thread (tx, ty) adds chunks ty, ty+TY, ... with independent
// loads, then the TY lanes of a column group are combined in a fixed order.  On
// return threads < TX hold the totals (plane a in tot[a*VEC..]).
template <int VEC, int NP>
__device__ __forceinline__ void chunk_totals(float const *partial, unsigned nchunks, size_t H, int tx_log2,
                                             size_t col, bool live, float (&tot)[NP * VEC], float *lds) {
  int const TX = 1 << tx_log2, TY = kBlock >> tx_log2;
  int const ty = threadIdx.x >> tx_log2;
#pragma unroll
  for (int i = 0; i < NP * VEC; ++i) tot[i] = 0.0f;
  if (live) {
#pragma unroll 8
    for (unsigned c = ty; c < nchunks; c += TY) {
#pragma unroll
      for (int a = 0; a < NP; ++a) {
        float v[VEC];
        load_f<VEC>(partial + (a * static_cast<size_t>(nchunks) + c) * H + col, v);
#pragma unroll
        for (int i = 0; i < VEC; ++i) tot[a * VEC + i] += v[i];
      }
    }
  }
  block_rows_reduce<NP * VEC>(tot, TX, lds);
}

// ---------------------------------------------------------------- forward
// Phase 2 of fwp_st.cpp:4709-4746 for one unit: batch mean, moving mean, batch
// std, moving std, then r and d from the UPDATED moving statistics.
struct StatsArgs {
  float const *x;
  size_t B, H, rows_per_chunk;
  int tx_log2;
  float *partial;  // [NP][nchunks][H]: sum x (and sum x^2) per batch chunk
  // optional: the moving statistics are copied to snap [2][H] (by the blocks of chunk 0) for an apply
  // pass that does the per-unit arithmetic itself and must see them as they were before the step
  float const *mov_mean, *mov_std;
  float *snap;
};

// Phase 1 of fwp_st.cpp:4692-4707 / fwp_mp.cpp:4640-4662: column sums of x and
// (NP == 2) x^2 per batch chunk.
template <int VEC, int NP>
__global__ __launch_bounds__(kBlock) void k_col_stats(StatsArgs a) {
  __shared__ float lds[4 * kWave * NP * VEC];
  int const TX = 1 << a.tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> a.tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  bool const live = col < a.H;
  RowWalk const w = row_walk(a.B, a.rows_per_chunk, a.tx_log2, ty);
  float acc[NP * VEC];
#pragma unroll
  for (int i = 0; i < NP * VEC; ++i) acc[i] = 0.0f;
  if (live && w.count > 0) {
    constexpr int U = 8;
    size_t const stride = w.step * a.H;
    float const *p = a.x + w.first * a.H + col;
    unsigned n = w.count;
    for (; n >= U; n -= U, p += U * stride) {
      float v[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) load_f<VEC>(p + u * stride, v[u]);
      sched_fence();
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          acc[i] += v[u][i];
          if constexpr (NP == 2) acc[VEC + i] += v[u][i] * v[u][i];
        }
    }
    for (; n > 0; --n, p += stride) {
      float v[VEC];
      load_f<VEC>(p, v);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        acc[i] += v[i];
        if constexpr (NP == 2) acc[VEC + i] += v[i] * v[i];
      }
    }
  }
  block_rows_reduce<NP * VEC>(acc, TX, lds);
  unsigned const nch = gridDim.y;
  if (threadIdx.x < TX && live) {
#pragma unroll
    for (int a_ = 0; a_ < NP; ++a_) {
      float v[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] = acc[a_ * VEC + i];
      store_f<VEC>(a.partial + (a_ * static_cast<size_t>(nch) + blockIdx.y) * a.H + col, v);
    }
    if constexpr (NP == 2) {
      if (a.snap != nullptr && blockIdx.y == 0) {
        float v[VEC];
        load_f<VEC>(a.mov_mean + col, v);
        store_f<VEC>(a.snap + col, v);
        load_f<VEC>(a.mov_std + col, v);
        store_f<VEC>(a.snap + a.H + col, v);
      }
    }
  }
}

// Geometry of the finalize kernels: a 256-thread block is TX column groups x
// TY lanes over the chunks, TY the power of two nearest the chunk count (2..64).
static int finalize_tx_log2(unsigned nchunks) {
  int ty_log2 = 1;
  while (ty_log2 < 6 && (1u << ty_log2) < nchunks) ++ty_log2;
  return 8 - ty_log2;
}

// Forward finalize from partial sums [2][nchunks][H] (the statistics kernel's,
// or the GEMM epilogue's with one chunk per tile row).
template <int VEC>
__global__ __launch_bounds__(kBlock) void k_fwd_finalize(float const *__restrict__ partial, unsigned nchunks, size_t H,
                                                          int tx_log2, FwdFinalize fin) {
  __shared__ float lds[4 * kWave * 2 * VEC];
  int const TX = 1 << tx_log2;
  int const tx = threadIdx.x & (TX - 1);
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  bool const live = col < H;
  bool const owner = static_cast<int>(threadIdx.x) < TX && live;
  float mm[VEC], ms[VEC];
  if (owner) {
    load_f<VEC>(fin.mov_mean + col, mm);
    load_f<VEC>(fin.mov_std + col, ms);
  }
  float tot[2 * VEC];
  chunk_totals<VEC, 2>(partial, nchunks, H, tx_log2, col, live, tot, lds);
  if (owner) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) fwd_finalize_unit(fin, col + i, tot[i], tot[VEC + i], mm[i], ms[i]);
  }
}

// out[j] (+)= column sum, from one plane of statistics partials.
template <int VEC>
__global__ __launch_bounds__(kBlock) void k_colsum_finalize(float const *__restrict__ partial, unsigned nchunks,
                                                             size_t H, int tx_log2, float *__restrict__ out,
                                                             int accumulate) {
  __shared__ float lds[4 * kWave * VEC];
  int const TX = 1 << tx_log2;
  int const tx = threadIdx.x & (TX - 1);
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  bool const live = col < H;
  float tot[VEC];
  chunk_totals<VEC, 1>(partial, nchunks, H, tx_log2, col, live, tot, lds);
  if (static_cast<int>(threadIdx.x) < TX && live) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) out[col + i] = accumulate ? out[col + i] + tot[i] : tot[i];
  }
}

// Dropout as the forward applies it (fwp_st.cpp:4830-4883): mask ? v*scale : 0
// with scale = 1 for plain Bernoulli, 1/keep for inverted Bernoulli.
struct FwdApplyArgs {
  float const *x, *gamma, *beta, *mean, *stdv, *r, *d;
  uint8_t const *mask;
  float const *residual;  // optional [B,H]: y = residual + (activation output after dropout)
  float *y;     // activation output after dropout
  float *xhat;  // optional materialised x_hat            (MAT only)
  float *nrm;   // optional materialised gamma*x_hat+beta (MAT only)
  size_t B, H, rows_per_chunk;
  int tx_log2;
  float drop_scale;
  // fin_partial != nullptr: no finalize kernel ran.  Every block forms the statistics of its own units
  // from the partial sums [2][fin_chunks][H] (few chunks, summed in chunk order) and the snapshot of the
  // moving statistics; the blocks of one chunk store the per-unit results.
  float const *fin_partial, *mov_mean_in, *mov_std_in;
  unsigned fin_chunks;
  FwdFinalize fin;
};

// Phase 3 of fwp_st.cpp:4748-4765, then AF_FIRE (fwp_st.cpp:4768-4794), then the
// dropout leaf (and, with RES, the identity shortcut of fwp_st.cpp:5051-5112),
// in one pass.
// MAT: materialise x_hat / the pre-activation (the un-fused leaf) with the
// reference's expression order.  Otherwise the per-unit constants are folded so
// that an element costs one subtraction and one fused multiply-add before the
// activation:  n = (x - mean) * (gamma*r/std) + (gamma*d + beta).
template <int VEC, int ACT, int DROPM, bool MAT, bool RES>
__global__ __launch_bounds__(kBlock) void k_fwd_apply(FwdApplyArgs a) {
  int const TX = 1 << a.tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> a.tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  RowWalk const w = row_walk(a.B, a.rows_per_chunk, a.tx_log2, ty, true);
  if (col >= a.H || w.count == 0) return;
  float mu[VEC], inv[VEC], rr[VEC], dd[VEC], ga[VEC], be[VEC];
  uint8_t mk[VEC];
  load_f<VEC>(a.gamma + col, ga);
  load_f<VEC>(a.beta + col, be);
  if (!MAT && a.fin_partial != nullptr) {
    float mm[VEC], ms[VEC], s1[VEC], s2[VEC];
    load_f<VEC>(a.mov_mean_in + col, mm);
    load_f<VEC>(a.mov_std_in + col, ms);
#pragma unroll
    for (int i = 0; i < VEC; ++i) s1[i] = s2[i] = 0.0f;
    float const *p1 = a.fin_partial + col;
    float const *p2 = p1 + static_cast<size_t>(a.fin_chunks) * a.H;
#pragma unroll 8
    for (unsigned c = 0; c < a.fin_chunks; ++c) {
      float v1[VEC], v2[VEC];
      load_f<VEC>(p1 + c * a.H, v1);
      load_f<VEC>(p2 + c * a.H, v2);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        s1[i] += v1[i];
        s2[i] += v2[i];
      }
    }
    bool const writer = blockIdx.y == 0 && ty == 0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      UnitStats const u = fwd_unit_stats(a.fin, s1[i], s2[i], mm[i], ms[i]);
      if (writer) store_unit_stats(a.fin, col + i, u);
      mu[i] = u.mean; inv[i] = u.stdv; rr[i] = u.r; dd[i] = u.d;
    }
  } else {
    load_f<VEC>(a.mean + col, mu);
    load_f<VEC>(a.stdv + col, inv);
    load_f<VEC>(a.r + col, rr);
    load_f<VEC>(a.d + col, dd);
  }
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
  auto body = [&](size_t off, float const (&xv)[VEC], uint8_t const (&mv)[VEC], float const (&rv)[VEC]) {
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
      if constexpr (RES) {
        // a separate rounding, as the reference's own add of two stored arrays: the empty statement makes q a
        // value of its own, so that the add cannot be fused into the activation's last multiply
        asm volatile("" : "+v"(q[i]));
        q[i] = rv[i] + q[i];
      }
    }
    if constexpr (MAT) {
      if (a.xhat != nullptr) store_f<VEC>(a.xhat + off, xh);
      if (a.nrm != nullptr) store_f<VEC>(a.nrm + off, nn);
      if (a.y != nullptr) store_f<VEC>(a.y + off, q);
    } else {
      store_f<VEC>(a.y + off, q);
    }
  };
  size_t const stride = w.step * a.H;
  size_t off = w.first * a.H + col;
  unsigned n = w.count;
  for (; n >= U; n -= U, off += U * stride) {
    float xv[U][VEC], rv[U][VEC];
    uint8_t mv[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      load_f<VEC>(a.x + off + u * stride, xv[u]);
      if constexpr (RES) {
        load_f<VEC>(a.residual + off + u * stride, rv[u]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) rv[u][i] = 0.0f;
      }
      if constexpr (DROPM == kDropElem) {
        load_u8<VEC>(a.mask + off + u * stride, mv[u]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mv[u][i] = mk[i];
      }
    }
    sched_fence();
#pragma unroll
    for (int u = 0; u < U; ++u) body(off + u * stride, xv[u], mv[u], rv[u]);
  }
  for (; n > 0; --n, off += stride) {
    float xv[VEC], rv[VEC];
    uint8_t mv[VEC];
    load_f<VEC>(a.x + off, xv);
    if constexpr (RES) {
      load_f<VEC>(a.residual + off, rv);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) rv[i] = 0.0f;
    }
    if constexpr (DROPM == kDropElem) {
      load_u8<VEC>(a.mask + off, mv);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) mv[i] = mk[i];
    }
    body(off, xv, mv, rv);
  }
}

// ---------------------------------------------------------------- backward
// dgamma += S0, dbeta += S1 (accumulating like the reference's derivative
// array), dmean, dstd, and the three per-unit coefficients of pass 2
// (bwp_st.cpp:1508-1531):  dx = e*(r/std) + dstd*((x-mean)/(B*std)) + dmean*(1/B).
struct BwdFinalize {
  float const *gamma, *stdv, *r;
  float *dgamma, *dbeta, *dmean, *dstd;
  float *coef;  // [3][H]  c1 = gamma*r/std, c2 = dstd/(B*std), c3 = dmean/B
  float batch_f, batch_scale;  // B and 1/B as floats
};

// sd, rr, ga, dg, db: the unit's std, r, gamma and running dgamma, dbeta as loaded
// before the sums were formed.
__device__ __forceinline__ void bwd_finalize_unit(BwdFinalize const &f, size_t H, size_t j, float s0, float s1,
                                                  float s2, float sd, float rr, float ga, float dg, float db) {
  f.dgamma[j] = dg + s0;
  f.dbeta[j] = db + s1;
  float const dm = (ga * s1) * (-rr / sd);
  float const ds = (ga * s2) * (-rr / (sd * sd));
  if (f.dmean != nullptr) f.dmean[j] = dm;
  if (f.dstd != nullptr) f.dstd[j] = ds;
  f.coef[0 * H + j] = ga * (rr / sd);
  f.coef[1 * H + j] = ds / (f.batch_f * sd);
  f.coef[2 * H + j] = dm * f.batch_scale;
}

struct BwdArgs {
  float const *x, *gamma, *beta, *mean, *stdv, *r, *d;
  float const *xhat;  // only when XHAT_GIVEN (un-fused leaf: dn = dY, x_hat stored)
  uint8_t const *mask;
  float const *dY;
  float *partial;     // reduce: [3][nchunks][H]
  float const *coef;  // apply: [3][H]
  // apply, fin_partial != nullptr: no finalize kernel ran; every block forms the coefficients of its
  // own units from the partial sums [3][fin_chunks][H], the blocks of one chunk accumulate dgamma / dbeta
  float const *fin_partial;
  unsigned fin_chunks;
  float *dgamma, *dbeta;
  float batch_f, batch_scale;
  float *dX;
  float *db_partial;  // apply with DBSUM: [apply chunks][H] column sums of the dX rows each block stored
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

// Pass 1 of bwp_st.cpp:1478-1506: column sums of dn*x_hat, dn and dn*(x-mean)
// per batch chunk (dmean and dstd follow from the last two in the finalize
// kernel: sum e*(-r/std) = -(r/std)*gamma*sum dn, sum e*(x-mean)*(-r/std^2) likewise).
template <int VEC, int ACT, int DROPM, bool XHAT_GIVEN>
__global__ __launch_bounds__(kBlock) void k_bwd_reduce(BwdArgs a) {
  __shared__ float lds[4 * kWave * 3 * VEC];
  int const TX = 1 << a.tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> a.tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  bool const live = col < a.H;
  RowWalk const w = row_walk(a.B, a.rows_per_chunk, a.tx_log2, ty);
  float acc[3 * VEC];
#pragma unroll
  for (int i = 0; i < 3 * VEC; ++i) acc[i] = 0.0f;
  if (live && w.count > 0) {
    UnitConsts<VEC> uc;
    load_unit_consts<VEC, DROPM, XHAT_GIVEN>(a, col, uc);
    constexpr int U = 4;
    auto body = [&](float const (&xv)[VEC], float const (&dy)[VEC], float const (&xg)[VEC],
                    uint8_t const (&mv)[VEC]) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float xh = xg[i];
        float const dn = bwd_dn<ACT, DROPM, XHAT_GIVEN>(a.drop_scale, a.drop_bwd_masked, xv[i], dy[i], mv[i], uc.mu[i], uc.rs[i], uc.dd[i],
                                                        uc.ga[i], uc.be[i], xh);
        acc[i] += dn * xh;
        acc[VEC + i] += dn;
        acc[2 * VEC + i] += dn * (xv[i] - uc.mu[i]);
      }
    };
    size_t const stride = w.step * a.H;
    size_t off = w.first * a.H + col;
    unsigned n = w.count;
    for (; n >= U; n -= U, off += U * stride) {
      float xv[U][VEC], dy[U][VEC], xg[U][VEC];
      uint8_t mv[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        load_f<VEC>(a.x + off + u * stride, xv[u]);
        load_f<VEC>(a.dY + off + u * stride, dy[u]);
        if constexpr (XHAT_GIVEN) {
          load_f<VEC>(a.xhat + off + u * stride, xg[u]);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) xg[u][i] = 0.0f;
        }
        if constexpr (DROPM == kDropElem) {
          load_u8<VEC>(a.mask + off + u * stride, mv[u]);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) mv[u][i] = uc.mk[i];
        }
      }
      sched_fence();
#pragma unroll
      for (int u = 0; u < U; ++u) body(xv[u], dy[u], xg[u], mv[u]);
    }
    for (; n > 0; --n, off += stride) {
      float xv[VEC], dy[VEC], xg[VEC];
      uint8_t mv[VEC];
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
  unsigned const nch = gridDim.y;
  if (threadIdx.x < TX && live) {
#pragma unroll
    for (int a_ = 0; a_ < 3; ++a_) {
      float v[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] = acc[a_ * VEC + i];
      store_f<VEC>(a.partial + (a_ * static_cast<size_t>(nch) + blockIdx.y) * a.H + col, v);
    }
  }
}

// Backward finalize from the partial sums [3][nchunks][H].
template <int VEC>
__global__ __launch_bounds__(kBlock) void k_bwd_finalize(float const *__restrict__ partial, unsigned nchunks, size_t H,
                                                          int tx_log2, BwdFinalize fin) {
  __shared__ float lds[4 * kWave * 3 * VEC];
  int const TX = 1 << tx_log2;
  int const tx = threadIdx.x & (TX - 1);
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  bool const live = col < H;
  bool const owner = static_cast<int>(threadIdx.x) < TX && live;
  float sd[VEC], rr[VEC], ga[VEC], dg[VEC], db[VEC];
  if (owner) {
    load_f<VEC>(fin.stdv + col, sd);
    load_f<VEC>(fin.gamma + col, ga);
    load_f<VEC>(fin.dgamma + col, dg);
    load_f<VEC>(fin.dbeta + col, db);
    if (fin.r != nullptr) {
      load_f<VEC>(fin.r + col, rr);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) rr[i] = 1.0f;
    }
  }
  float tot[3 * VEC];
  chunk_totals<VEC, 3>(partial, nchunks, H, tx_log2, col, live, tot, lds);
  if (owner) {
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      bwd_finalize_unit(fin, H, col + i, tot[i], tot[VEC + i], tot[2 * VEC + i], sd[i], rr[i], ga[i], dg[i], db[i]);
  }
}

// Pass 2 of bwp_st.cpp:1508-1531 with the activation derivative recomputed.
// ACC: dX += instead of dX = (the error array of a layer that also receives a
// shortcut's gradient, bwp_st.cpp:1112-1175).
// DBSUM: every block also stores the column sums of the dX rows it wrote (rows of a thread ascending, then the
// block's row lanes in the fixed order of block_rows_reduce) to db_partial [chunks][H]; a finalize launch adds
// the chunks: the bias gradient without a second pass over dX.
template <int VEC, int ACT, int DROPM, bool XHAT_GIVEN, bool ACC, bool DBSUM = false>
__global__ __launch_bounds__(kBlock) void k_bwd_apply(BwdArgs a) {
  __shared__ float lds_db[DBSUM ? 4 * kWave * VEC : 1];
  int const TX = 1 << a.tx_log2;
  int const tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> a.tx_log2;
  size_t const col = (static_cast<size_t>(blockIdx.x) * TX + tx) * VEC;
  RowWalk const w = row_walk(a.B, a.rows_per_chunk, a.tx_log2, ty, true);
  float dbs[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) dbs[i] = 0.0f;
  if constexpr (DBSUM) {
    if (col >= a.H || w.count == 0) {  // idle threads still take part in the block's sum
      block_rows_reduce<VEC>(dbs, TX, lds_db);
      if (static_cast<int>(threadIdx.x) < TX && col < a.H) store_f<VEC>(a.db_partial + static_cast<size_t>(blockIdx.y) * a.H + col, dbs);
      return;
    }
  } else {
    if (col >= a.H || w.count == 0) return;
  }
  UnitConsts<VEC> uc;
  load_unit_consts<VEC, DROPM, XHAT_GIVEN>(a, col, uc);
  float c1[VEC], c2[VEC], c3[VEC];
  if (!XHAT_GIVEN && a.fin_partial != nullptr) {
    float sd[VEC], rr[VEC], s0[VEC], s1[VEC], s2[VEC];
    load_f<VEC>(a.stdv + col, sd);
    load_f<VEC>(a.r + col, rr);
#pragma unroll
    for (int i = 0; i < VEC; ++i) s0[i] = s1[i] = s2[i] = 0.0f;
    size_t const plane = static_cast<size_t>(a.fin_chunks) * a.H;
    float const *p0 = a.fin_partial + col;
#pragma unroll 4
    for (unsigned c = 0; c < a.fin_chunks; ++c) {
      float v0[VEC], v1[VEC], v2[VEC];
      load_f<VEC>(p0 + c * a.H, v0);
      load_f<VEC>(p0 + plane + c * a.H, v1);
      load_f<VEC>(p0 + 2 * plane + c * a.H, v2);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        s0[i] += v0[i];
        s1[i] += v1[i];
        s2[i] += v2[i];
      }
    }
    if (blockIdx.y == 0 && ty == 0) {
      float dg[VEC], db[VEC];
      load_f<VEC>(a.dgamma + col, dg);
      load_f<VEC>(a.dbeta + col, db);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        dg[i] += s0[i];
        db[i] += s1[i];
      }
      store_f<VEC>(a.dgamma + col, dg);
      store_f<VEC>(a.dbeta + col, db);
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {  // as bwd_finalize_unit
      float const dm = (uc.ga[i] * s1[i]) * (-rr[i] / sd[i]);
      float const ds = (uc.ga[i] * s2[i]) * (-rr[i] / (sd[i] * sd[i]));
      c1[i] = uc.ga[i] * (rr[i] / sd[i]);
      c2[i] = ds / (a.batch_f * sd[i]);
      c3[i] = dm * a.batch_scale;
    }
  } else {
    load_f<VEC>(a.coef + 0 * a.H + col, c1);
    load_f<VEC>(a.coef + 1 * a.H + col, c2);
    load_f<VEC>(a.coef + 2 * a.H + col, c3);
  }
  constexpr int U = 4;
  auto body = [&](size_t off, float const (&xv)[VEC], float const (&dy)[VEC], uint8_t const (&mv)[VEC],
                  float const (&old)[VEC]) {
    float dx[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float xh = 0.0f;
      float const dn = bwd_dn<ACT, DROPM, XHAT_GIVEN>(a.drop_scale, a.drop_bwd_masked, xv[i], dy[i], mv[i], uc.mu[i], uc.rs[i], uc.dd[i], uc.ga[i],
                                                      uc.be[i], xh);
      dx[i] = dn * c1[i] + (xv[i] - uc.mu[i]) * c2[i] + c3[i];
      if constexpr (ACC) dx[i] += old[i];
      if constexpr (DBSUM) dbs[i] += dx[i];
    }
    store_f<VEC>(a.dX + off, dx);
  };
  size_t const stride = w.step * a.H;
  size_t off = w.first * a.H + col;
  unsigned n = w.count;
  for (; n >= U; n -= U, off += U * stride) {
    float xv[U][VEC], dy[U][VEC], old[U][VEC];
    uint8_t mv[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      load_f<VEC>(a.x + off + u * stride, xv[u]);
      load_f<VEC>(a.dY + off + u * stride, dy[u]);
      if constexpr (ACC) {
        load_f<VEC>(a.dX + off + u * stride, old[u]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) old[u][i] = 0.0f;
      }
      if constexpr (DROPM == kDropElem) {
        load_u8<VEC>(a.mask + off + u * stride, mv[u]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mv[u][i] = uc.mk[i];
      }
    }
    sched_fence();
#pragma unroll
    for (int u = 0; u < U; ++u) body(off + u * stride, xv[u], dy[u], mv[u], old[u]);
  }
  for (; n > 0; --n, off += stride) {
    float xv[VEC], dy[VEC], old[VEC];
    uint8_t mv[VEC];
    load_f<VEC>(a.x + off, xv);
    load_f<VEC>(a.dY + off, dy);
    if constexpr (ACC) {
      load_f<VEC>(a.dX + off, old);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) old[i] = 0.0f;
    }
    if constexpr (DROPM == kDropElem) {
      load_u8<VEC>(a.mask + off, mv);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) mv[i] = uc.mk[i];
    }
    body(off, xv, dy, mv, old);
  }
  if constexpr (DBSUM) {
    block_rows_reduce<VEC>(dbs, TX, lds_db);
    if (static_cast<int>(threadIdx.x) < TX) store_f<VEC>(a.db_partial + static_cast<size_t>(blockIdx.y) * a.H + col, dbs);
  }
}

// ---------------------------------------------------------------- host drivers
static bool use_vec4(size_t H, std::initializer_list<void const *> ptrs) {
  if (H % 4 != 0) return false;
  for (void const *p : ptrs)
    if (p != nullptr && !dlmi_aligned16(p)) return false;
  return true;
}

// Runs the statement with DROPM bound to the runtime dropout mode.
#define DLMI_DISPATCH_DROP(mode, ...)                                         \
  switch (mode) {                                                             \
    case kDropUnit: { constexpr int DROPM = kDropUnit; __VA_ARGS__; } break;  \
    case kDropElem: { constexpr int DROPM = kDropElem; __VA_ARGS__; } break;  \
    default: { constexpr int DROPM = kDropNone; __VA_ARGS__; } break;         \
  }

// The context's own scratch, grown to what a reduction over [*, H] can use:
// 3 planes of partial sums [chunks][H] with chunks * H <= blocks * (widest
// block: 256 column groups of 4 units) + H, and the 3*H backward coefficients.
size_t norm_scratch_bytes(dlmi_ctx const *ctx, size_t H) {
  size_t const blocks = static_cast<size_t>(ctx->num_cu) * ctx->tune.reduce_blocks_per_cu;
  // (+ one plane [apply chunks][H] for the bias-gradient partials of the backward apply pass)
  size_t const apply_blocks = static_cast<size_t>(ctx->num_cu) * ctx->tune.apply_bwd_blocks_per_cu;
  size_t const multi = 3 * sizeof(float) * (blocks * 1024 + 2 * H) + round_up(3 * H * sizeof(float), 256) + 4096 +
                       sizeof(float) * (apply_blocks * 1024 + H) + 256;
  size_t const panel = panel_scratch_bytes_db(H);
  return multi > panel ? multi : panel;
}
static int ctx_scratch(dlmi_ctx *ctx, size_t H, ScratchView *v) {
  int rc = dlmi_scratch_reserve(ctx, norm_scratch_bytes(ctx, H));
  if (rc != DLMI_OK) return rc;
  v->data = dlmi_scratch_data(ctx);
  v->data_bytes = ctx->scratch_bytes;
  return DLMI_OK;
}

static int run_fwd_train(dlmi_ctx *ctx, ScratchView const &sv, size_t B, size_t H, FwdTrainCall const &c) {
  bool const vec4 = use_vec4(H, {c.x, c.gamma, c.beta, c.mean, c.stdv, c.mov_mean, c.mov_std, c.r, c.d, c.y, c.xhat, c.nrm,
                                 c.residual}) &&
                    (c.drop_mode == kDropNone || (reinterpret_cast<uintptr_t>(c.mask) & 3u) == 0);
  // a mini-batch of a few hundred rows: one launch, a workgroup per 8 columns
  if (int const took = small_fwd_try(ctx, B, H, c); took != 0) return took < 0 ? took : DLMI_OK;
  // a few thousand rows, H a multiple of 1024: one launch that reads x once
  if (int const took = panel_fwd_try(ctx, B, H, c, vec4, sv.data, sv.data_bytes); took != 0) return took < 0 ? took : DLMI_OK;
  dim3 const block(kBlock);
  FwdFinalize fin;
  fin.mean = c.mean; fin.stdv = c.stdv; fin.mov_mean = c.mov_mean; fin.mov_std = c.mov_std; fin.r = c.r; fin.d = c.d;
  fin.batch_scale = 1.0f / static_cast<float>(B);
  fin.momentum = c.momentum; fin.eps = c.eps; fin.r_max = c.r_max; fin.d_max = c.d_max;
  fin.renorm = c.norm == DLMI_NORM_BATCH_RENORM ? 1 : 0;
  float const *partial = c.partial_in;
  unsigned nchunks = c.partial_chunks;
  // data region: [2][H] snapshot of the moving statistics (two-launch scheme), then the partial sums
  size_t const fixed = round_up(3 * H * sizeof(float), 256);
  float *const snap = reinterpret_cast<float *>(sv.data);
  float const *snap_rd = snap;
  bool fold = false;
  if (partial != nullptr) {
    // the producer's partial sums and its copy of the moving statistics: few chunks go straight to the apply pass
    fold = c.snapshot_in != nullptr && nchunks <= kFoldChunks && c.xhat == nullptr && c.nrm == nullptr && c.y != nullptr &&
           ctx->tune.fold_fwd > 0 && (ctx->tune.fold_fwd > 1 || B * H <= ctx->tune.fold_fwd_epilogue_max_elements);
    if (fold) snap_rd = c.snapshot_in;
  } else {
    ColGeom g;
    fold = c.xhat == nullptr && c.nrm == nullptr && c.y != nullptr && fold_geometry(ctx, B, H, vec4, 2, sv.data_bytes, &g);
    if (!fold) g = reduce_geometry(ctx, B, H, vec4, 2, sv.data_bytes);
    if (fixed + static_cast<size_t>(2) * g.nchunks * H * sizeof(float) > sv.data_bytes)
      return dlmi_fail(ctx, DLMI_E_UNSUPPORTED, "%zu units need more scratch than the %zu bytes at hand", H,
                       sv.data_bytes);
    StatsArgs s{};
    s.x = c.x; s.B = B; s.H = H;
    s.rows_per_chunk = ctx->tune.reduce_interleave ? 0 : g.rows_per_chunk; s.tx_log2 = g.tx_log2;
    s.partial = reinterpret_cast<float *>(sv.data + fixed);
    if (fold) {
      s.mov_mean = c.mov_mean; s.mov_std = c.mov_std; s.snap = snap;
    }
    dim3 const grid(g.grid_x, g.nchunks);
    if (vec4)
      hipLaunchKernelGGL((k_col_stats<4, 2>), grid, block, 0, ctx->stream, s);
    else
      hipLaunchKernelGGL((k_col_stats<1, 2>), grid, block, 0, ctx->stream, s);
    DLMI_LAUNCH_CHECK(ctx, "k_col_stats");
    partial = s.partial;
    nchunks = g.nchunks;
  }
  if (!fold) {
    bool const pvec4 = vec4 && dlmi_aligned16(partial);
    size_t const groups = dlmi_ceil_div(H, pvec4 ? 4 : 1);
    int const ftx = finalize_tx_log2(nchunks);
    dim3 const grid(static_cast<unsigned>(dlmi_ceil_div(groups, size_t(1) << ftx)));
    if (pvec4)
      hipLaunchKernelGGL(k_fwd_finalize<4>, grid, block, 0, ctx->stream, partial, nchunks, H, ftx, fin);
    else
      hipLaunchKernelGGL(k_fwd_finalize<1>, grid, block, 0, ctx->stream, partial, nchunks, H, ftx, fin);
    DLMI_LAUNCH_CHECK(ctx, "k_fwd_finalize");
  }
  ColGeom const ga = apply_geometry(ctx, B, H, vec4, ctx->tune.apply_fwd_blocks_per_cu);
  FwdApplyArgs a;
  a.x = c.x; a.gamma = c.gamma; a.beta = c.beta; a.mean = c.mean; a.stdv = c.stdv; a.r = c.r; a.d = c.d;
  a.mask = c.mask; a.residual = c.residual; a.y = c.y; a.xhat = c.xhat; a.nrm = c.nrm;
  a.B = B; a.H = H; a.rows_per_chunk = ctx->tune.apply_interleave ? 0 : ga.rows_per_chunk; a.tx_log2 = ga.tx_log2;
  a.drop_scale = c.drop_scale;
  a.fin_partial = fold ? partial : nullptr; a.mov_mean_in = snap_rd; a.mov_std_in = snap_rd + H; a.fin_chunks = nchunks;
  a.fin = fin;
  dim3 const agrid(ga.grid_x, ga.nchunks);
  if (c.xhat != nullptr || c.nrm != nullptr) {  // un-fused leaf: LINEAR, no dropout by construction
    if (vec4)
      hipLaunchKernelGGL((k_fwd_apply<4, DLMI_ACT_LINEAR, kDropNone, true, false>), agrid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((k_fwd_apply<1, DLMI_ACT_LINEAR, kDropNone, true, false>), agrid, block, 0, ctx->stream, a);
  } else if (c.y != nullptr) {
    if (c.residual != nullptr) {
      DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_DROP(c.drop_mode, {
        if (vec4)
          hipLaunchKernelGGL((k_fwd_apply<4, ACT, DROPM, false, true>), agrid, block, 0, ctx->stream, a);
        else
          hipLaunchKernelGGL((k_fwd_apply<1, ACT, DROPM, false, true>), agrid, block, 0, ctx->stream, a);
      }));
    } else {
      DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_DROP(c.drop_mode, {
        if (vec4)
          hipLaunchKernelGGL((k_fwd_apply<4, ACT, DROPM, false, false>), agrid, block, 0, ctx->stream, a);
        else
          hipLaunchKernelGGL((k_fwd_apply<1, ACT, DROPM, false, false>), agrid, block, 0, ctx->stream, a);
      }));
    }
  }
  DLMI_LAUNCH_CHECK(ctx, "k_fwd_apply");
  return DLMI_OK;
}

static int run_bwd(dlmi_ctx *ctx, ScratchView const &sv, size_t B, size_t H, BwdCall const &c) {
  bool const vec4 = use_vec4(H, {c.x, c.gamma, c.beta, c.mean, c.stdv, c.r, c.d, c.xhat, c.dY, c.dX, c.dgamma, c.dbeta}) &&
                    (c.drop_mode == kDropNone || (reinterpret_cast<uintptr_t>(c.mask) & 3u) == 0);
  // the one-launch kernels do not form the bias gradient: where it is asked for, a pass over dX follows them
  auto then_db = [&](int took) { return took < 0 ? took : (c.db != nullptr ? column_sums(ctx, B, H, c.dX, c.db, c.db_accumulate ? 1 : 0) : DLMI_OK); };
  if (int const took = small_bwd_try(ctx, B, H, c); took != 0) return then_db(took);
  // a few thousand rows, H a multiple of 512: one launch that reads dY and x once
  float *panel_db = nullptr;
  unsigned panel_db_rows = 0;
  if (int const took = panel_bwd_try(ctx, B, H, c, vec4, sv.data, sv.data_bytes, &panel_db, &panel_db_rows); took != 0) {
    if (took < 0 || panel_db == nullptr) return then_db(took);
    // the kernel left one row of column sums of dX per workgroup rank: the bias gradient is their sum
    int const ftx = finalize_tx_log2(panel_db_rows);
    dim3 const fgrid(static_cast<unsigned>(dlmi_ceil_div(H / 4, size_t(1) << ftx)));
    hipLaunchKernelGGL(k_colsum_finalize<4>, fgrid, dim3(kBlock), 0, ctx->stream, panel_db, panel_db_rows, H, ftx, c.db,
                       c.db_accumulate ? 1 : 0);
    DLMI_LAUNCH_CHECK(ctx, "k_colsum_finalize");
    return DLMI_OK;
  }
  ColGeom g;
  bool const fold = !c.xhat_given && c.dmean == nullptr && c.dstd == nullptr &&
                    fold_geometry(ctx, B, H, vec4, 3, sv.data_bytes, &g);
  if (!fold) g = reduce_geometry(ctx, B, H, vec4, 3, sv.data_bytes);
  // data region: coefficients [3][H] first, then the partial sums [3][nchunks][H]
  size_t const coef_bytes = round_up(3 * H * sizeof(float), 256);
  if (coef_bytes + static_cast<size_t>(3) * g.nchunks * H * sizeof(float) > sv.data_bytes)
    return dlmi_fail(ctx, DLMI_E_UNSUPPORTED, "%zu units need more scratch than the %zu bytes at hand", H,
                     sv.data_bytes);
  float *coef = reinterpret_cast<float *>(sv.data);
  float *partial = reinterpret_cast<float *>(sv.data + coef_bytes);
  BwdArgs a{};
  a.x = c.x; a.gamma = c.gamma; a.beta = c.beta; a.mean = c.mean; a.stdv = c.stdv; a.r = c.r; a.d = c.d;
  a.xhat = c.xhat; a.mask = c.mask; a.dY = c.dY; a.partial = partial; a.coef = coef;
  a.dX = c.dX;
  a.fin_partial = fold ? partial : nullptr; a.fin_chunks = g.nchunks; a.dgamma = c.dgamma; a.dbeta = c.dbeta;
  a.batch_f = static_cast<float>(B); a.batch_scale = 1.0f / static_cast<float>(B);
  BwdFinalize fin;
  fin.gamma = c.gamma; fin.stdv = c.stdv; fin.r = c.r; fin.dgamma = c.dgamma; fin.dbeta = c.dbeta;
  fin.dmean = c.dmean; fin.dstd = c.dstd; fin.coef = coef;
  fin.batch_f = static_cast<float>(B); fin.batch_scale = 1.0f / static_cast<float>(B);
  a.B = B; a.H = H; a.rows_per_chunk = ctx->tune.reduce_interleave ? 0 : g.rows_per_chunk; a.tx_log2 = g.tx_log2;
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
  if (!fold) {
    size_t const groups = dlmi_ceil_div(H, vec4 ? 4 : 1);
    int const ftx = finalize_tx_log2(g.nchunks);
    dim3 const fgrid(static_cast<unsigned>(dlmi_ceil_div(groups, size_t(1) << ftx)));
    if (vec4)
      hipLaunchKernelGGL(k_bwd_finalize<4>, fgrid, block, 0, ctx->stream, partial, g.nchunks, H, ftx, fin);
    else
      hipLaunchKernelGGL(k_bwd_finalize<1>, fgrid, block, 0, ctx->stream, partial, g.nchunks, H, ftx, fin);
    DLMI_LAUNCH_CHECK(ctx, "k_bwd_finalize");
  }
  ColGeom const ga = apply_geometry(ctx, B, H, vec4, ctx->tune.apply_bwd_blocks_per_cu);
  a.rows_per_chunk = ctx->tune.apply_interleave ? 0 : ga.rows_per_chunk;
  a.tx_log2 = ga.tx_log2;
  dim3 const agrid(ga.grid_x, ga.nchunks);
  // the bias gradient as a by-product of this pass: block partials behind the reduction's, then one small launch
  size_t const db_offset = round_up(coef_bytes + static_cast<size_t>(3) * g.nchunks * H * sizeof(float), 256);
  bool const db_here = c.db != nullptr && vec4 && !c.xhat_given && !c.accumulate &&
                       db_offset + static_cast<size_t>(ga.nchunks) * H * sizeof(float) <= sv.data_bytes;
  a.db_partial = db_here ? reinterpret_cast<float *>(sv.data + db_offset) : nullptr;
  if (db_here) {
    DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_DROP(c.drop_mode, {
      hipLaunchKernelGGL((k_bwd_apply<4, ACT, DROPM, false, false, true>), agrid, block, 0, ctx->stream, a);
    }));
    DLMI_LAUNCH_CHECK(ctx, "k_bwd_apply");
    int const ftx = finalize_tx_log2(ga.nchunks);
    dim3 const fgrid(static_cast<unsigned>(dlmi_ceil_div(H / 4, size_t(1) << ftx)));
    hipLaunchKernelGGL(k_colsum_finalize<4>, fgrid, block, 0, ctx->stream, a.db_partial, ga.nchunks, H, ftx, c.db,
                       c.db_accumulate ? 1 : 0);
    DLMI_LAUNCH_CHECK(ctx, "k_colsum_finalize");
    return DLMI_OK;
  }
  if (c.xhat_given) {
    if (vec4)
      hipLaunchKernelGGL((k_bwd_apply<4, DLMI_ACT_LINEAR, kDropNone, true, false>), agrid, block, 0, ctx->stream, a);
    else
      hipLaunchKernelGGL((k_bwd_apply<1, DLMI_ACT_LINEAR, kDropNone, true, false>), agrid, block, 0, ctx->stream, a);
  } else if (c.accumulate) {
    DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_DROP(c.drop_mode, {
      if (vec4)
        hipLaunchKernelGGL((k_bwd_apply<4, ACT, DROPM, false, true>), agrid, block, 0, ctx->stream, a);
      else
        hipLaunchKernelGGL((k_bwd_apply<1, ACT, DROPM, false, true>), agrid, block, 0, ctx->stream, a);
    }));
  } else {
    DLMI_DISPATCH_ACT(c.act, DLMI_DISPATCH_DROP(c.drop_mode, {
      if (vec4)
        hipLaunchKernelGGL((k_bwd_apply<4, ACT, DROPM, false, false>), agrid, block, 0, ctx->stream, a);
      else
        hipLaunchKernelGGL((k_bwd_apply<1, ACT, DROPM, false, false>), agrid, block, 0, ctx->stream, a);
    }));
  }
  DLMI_LAUNCH_CHECK(ctx, "k_bwd_apply");
  return c.db != nullptr ? column_sums(ctx, B, H, c.dX, c.db, c.db_accumulate ? 1 : 0) : DLMI_OK;
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

static FwdTrainCall fused_fwd_call(dlmi_fused_desc const *desc, float const *x, float const *gamma, float const *beta,
                                   uint8_t const *mask, float *mean, float *stdv, float *mov_mean, float *mov_std,
                                   float *r, float *d, float *y) {
  FwdTrainCall c;
  c.norm = desc->norm; c.act = desc->act; c.drop_mode = drop_mode_of(desc);
  c.momentum = desc->momentum; c.eps = desc->eps; c.r_max = desc->r_max; c.d_max = desc->d_max;
  c.drop_scale = drop_scale_of(desc);
  c.x = x; c.gamma = gamma; c.beta = beta; c.mask = mask;
  c.mean = mean; c.stdv = stdv; c.mov_mean = mov_mean; c.mov_std = mov_std; c.r = r; c.d = d;
  c.y = y; c.xhat = nullptr; c.nrm = nullptr;
  return c;
}

int fused_fwd_from_partials(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                            float const *gamma, float const *beta, uint8_t const *mask, float const *residual,
                            float *mean, float *stdv, float *mov_mean, float *mov_std, float *r, float *d, float *y,
                            float const *partial, unsigned nchunks, float const *slices, unsigned nslices,
                            float const *mov_snapshot) {
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && mov_mean && mov_std && r && d && y, "null pointer");
  FwdTrainCall c = fused_fwd_call(desc, x, gamma, beta, mask, mean, stdv, mov_mean, mov_std, r, d, y);
  c.residual = residual;
  c.partial_in = partial; c.partial_chunks = nchunks; c.snapshot_in = partial != nullptr ? mov_snapshot : nullptr;
  if (nslices > 0) {
    c.slices = slices; c.nslices = nslices; c.z_out = const_cast<float *>(x);
  }
  ScratchView sv{};
  if (partial == nullptr && nslices == 0) {
    rc = ctx_scratch(ctx, H, &sv);
    if (rc != DLMI_OK) return rc;
  }
  return run_fwd_train(ctx, sv, B, H, c);
}

int fused_bwd_from_slices(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                          float const *gamma, float const *beta, uint8_t const *mask, float const *mean,
                          float const *stdv, float const *r, float const *d, float const *slices, unsigned nslices,
                          float *dgamma, float *dbeta, float *dX) {
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && r && d && slices && nslices > 0 && dgamma && dbeta && dX,
               "null pointer");
  BwdCall c;
  c.act = desc->act; c.xhat_given = false; c.drop_mode = drop_mode_of(desc);
  c.drop_bwd_masked = desc->dropout_bwd == DLMI_DROP_BWD_MASKED ? 1 : 0;
  c.drop_scale = drop_scale_of(desc);
  c.x = x; c.gamma = gamma; c.beta = beta; c.mean = mean; c.stdv = stdv; c.r = r; c.d = d; c.xhat = nullptr;
  c.dY = nullptr; c.mask = mask; c.dy_slices = slices; c.nslices = nslices;
  c.dgamma = dgamma; c.dbeta = dbeta; c.dmean = nullptr; c.dstd = nullptr; c.dX = dX;
  int const took = small_bwd_try(ctx, B, H, c);
  if (took == 0) return dlmi_fail(ctx, DLMI_E_INVALID, "fused_bwd_from_slices: not a small-batch shape");
  return took < 0 ? took : DLMI_OK;
}

unsigned fused_bwd_narrow_max() { return kNarrowMaxUnits; }

int fused_bwd_from_narrow(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                          float const *gamma, float const *beta, uint8_t const *mask, float const *mean,
                          float const *stdv, float const *r, float const *d, float const *dZn, float const *Wn,
                          size_t Hn, float *dgamma, float *dbeta, float *dX) {
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && r && d && dZn && Wn && dgamma && dbeta && dX, "null pointer");
  DLMI_REQUIRE(ctx, Hn > 0 && Hn <= kNarrowMaxUnits, "not a narrow layer");
  BwdCall c;
  c.act = desc->act; c.xhat_given = false; c.drop_mode = drop_mode_of(desc);
  c.drop_bwd_masked = desc->dropout_bwd == DLMI_DROP_BWD_MASKED ? 1 : 0;
  c.drop_scale = drop_scale_of(desc);
  c.x = x; c.gamma = gamma; c.beta = beta; c.mean = mean; c.stdv = stdv; c.r = r; c.d = d; c.xhat = nullptr;
  c.dY = nullptr; c.mask = mask; c.narrow_dz = dZn; c.narrow_w = Wn; c.narrow_h = static_cast<unsigned>(Hn);
  c.dgamma = dgamma; c.dbeta = dbeta; c.dmean = nullptr; c.dstd = nullptr; c.dX = dX;
  int const took = small_bwd_try(ctx, B, H, c);
  if (took == 0) return dlmi_fail(ctx, DLMI_E_INVALID, "fused_bwd_from_narrow: not a small-batch shape");
  return took < 0 ? took : DLMI_OK;
}

int column_sums(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float *out, int accumulate) {
  if (int const took = small_colsum_try(ctx, B, H, x, out, accumulate); took != 0) return took < 0 ? took : DLMI_OK;
  ScratchView sv{};
  int rc = ctx_scratch(ctx, H, &sv);
  if (rc != DLMI_OK) return rc;
  bool const vec4 = use_vec4(H, {x, out});
  ColGeom const g = reduce_geometry(ctx, B, H, vec4, 1, sv.data_bytes);
  StatsArgs s{};
  s.x = x; s.B = B; s.H = H; s.rows_per_chunk = ctx->tune.reduce_interleave ? 0 : g.rows_per_chunk; s.tx_log2 = g.tx_log2;
  s.partial = reinterpret_cast<float *>(sv.data);
  dim3 const grid(g.grid_x, g.nchunks), block(kBlock);
  if (vec4)
    hipLaunchKernelGGL((k_col_stats<4, 1>), grid, block, 0, ctx->stream, s);
  else
    hipLaunchKernelGGL((k_col_stats<1, 1>), grid, block, 0, ctx->stream, s);
  DLMI_LAUNCH_CHECK(ctx, "k_col_stats");
  size_t const groups = dlmi_ceil_div(H, vec4 ? 4 : 1);
  int const ftx = finalize_tx_log2(g.nchunks);
  dim3 const fgrid(static_cast<unsigned>(dlmi_ceil_div(groups, size_t(1) << ftx)));
  if (vec4)
    hipLaunchKernelGGL(k_colsum_finalize<4>, fgrid, block, 0, ctx->stream, s.partial, g.nchunks, H, ftx, out, accumulate);
  else
    hipLaunchKernelGGL(k_colsum_finalize<1>, fgrid, block, 0, ctx->stream, s.partial, g.nchunks, H, ftx, out, accumulate);
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
  ScratchView sv{};
  int rc = ctx_scratch(ctx, H, &sv);
  if (rc != DLMI_OK) return rc;
  return run_fwd_train(ctx, sv, B, H, c);
}

int dlmi_fused_norm_act_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                            float const *gamma, float const *beta, uint8_t const *mask, float *mean,
                            float *stdv, float *mov_mean, float *mov_std, float *r, float *d, float *y) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, B > 0 && H > 0, "empty tensor");
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && mov_mean && mov_std && r && d && y, "null pointer");
  FwdTrainCall const c = fused_fwd_call(desc, x, gamma, beta, mask, mean, stdv, mov_mean, mov_std, r, d, y);
  ScratchView sv{};
  rc = ctx_scratch(ctx, H, &sv);
  if (rc != DLMI_OK) return rc;
  return run_fwd_train(ctx, sv, B, H, c);
}

int dlmi_fused_norm_act_residual_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                                     float const *gamma, float const *beta, uint8_t const *mask,
                                     float const *shortcut, float *mean, float *stdv, float *mov_mean, float *mov_std,
                                     float *r, float *d, float *y) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, B > 0 && H > 0, "empty tensor");
  DLMI_REQUIRE(ctx, shortcut != nullptr, "null pointer");
  return fused_fwd_from_partials(ctx, desc, B, H, x, gamma, beta, mask, shortcut, mean, stdv, mov_mean, mov_std, r, d, y,
                                 nullptr, 0);
}

int dlmi_fused_norm_act_fwd_noalloc(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                                    float const *gamma, float const *beta, uint8_t const *mask, float *mean,
                                    float *stdv, float *mov_mean, float *mov_std, float *r, float *d, float *y) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, B > 0 && H > 0, "empty tensor");
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && mov_mean && mov_std && r && d && y, "null pointer");
  if (H > DLMI_NOALLOC_MAX_UNITS)
    return dlmi_fail(ctx, DLMI_E_UNSUPPORTED,
                     "dlmi_fused_norm_act_fwd_noalloc: %zu units exceed the %d its fixed scratch of %zu bytes is sized for "
                     "(use dlmi_fused_norm_act_fwd)", H, DLMI_NOALLOC_MAX_UNITS, kStaticScratchBytes);
  if (ctx->static_scratch == nullptr) return dlmi_fail(ctx, DLMI_E_HIP, "the static scratch of device %d was not found", ctx->device);
  FwdTrainCall const c = fused_fwd_call(desc, x, gamma, beta, mask, mean, stdv, mov_mean, mov_std, r, d, y);
  // the device's own copy of the file-scope array, by its device address: no hipMalloc, no hipFree, no
  // memset (every partial sum the finalize kernel reads is written by the statistics kernel first)
  rc = static_scratch_order(ctx);
  if (rc != DLMI_OK) return rc;
  ScratchView sv{};
  sv.data = ctx->static_scratch;
  sv.data_bytes = ctx->static_scratch_bytes;
  return run_fwd_train(ctx, sv, B, H, c);
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
  ScratchView sv{};
  int rc = ctx_scratch(ctx, H, &sv);
  if (rc != DLMI_OK) return rc;
  return run_bwd(ctx, sv, B, H, c);
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
  ScratchView sv{};
  rc = ctx_scratch(ctx, H, &sv);
  if (rc != DLMI_OK) return rc;
  return run_bwd(ctx, sv, B, H, c);
}

int dlmi_fused_norm_act_bwd_db(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                               float const *gamma, float const *beta, uint8_t const *mask, float const *mean,
                               float const *stdv, float const *r, float const *d, float const *dY, float *dgamma,
                               float *dbeta, float *dX, float *db, int accumulate_db) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  int rc = check_desc(ctx, desc, mask);
  if (rc != DLMI_OK) return rc;
  DLMI_REQUIRE(ctx, B > 0 && H > 0, "empty tensor");
  DLMI_REQUIRE(ctx, x && gamma && beta && mean && stdv && r && d && dY && dgamma && dbeta && dX && db, "null pointer");
  BwdCall c;
  c.act = desc->act; c.xhat_given = false; c.drop_mode = drop_mode_of(desc);
  c.drop_bwd_masked = desc->dropout_bwd == DLMI_DROP_BWD_MASKED ? 1 : 0;
  c.drop_scale = drop_scale_of(desc);
  c.x = x; c.gamma = gamma; c.beta = beta; c.mean = mean; c.stdv = stdv; c.r = r; c.d = d; c.xhat = nullptr;
  c.dY = dY; c.mask = mask;
  c.dgamma = dgamma; c.dbeta = dbeta; c.dmean = nullptr; c.dstd = nullptr; c.dX = dX;
  c.db = db; c.db_accumulate = accumulate_db != 0;
  ScratchView sv{};
  rc = ctx_scratch(ctx, H, &sv);
  if (rc != DLMI_OK) return rc;
  return run_bwd(ctx, sv, B, H, c);
}

}  // extern "C"
