// Shared host-side plumbing of the dlmi library: the context object, error
// capture and launch-geometry helpers.  HIP only, gfx950 only.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/dlmi.h"

// Launch-geometry knobs of the normalization kernels, read once per context
// from the environment (DLMI_NORM_*; tuning aids, the defaults are the measured
// best on MI355X).
struct dlmi_tuning {
  int reduce_tx_cap = 128;        // widest column span of a reduction block, in column groups
  int reduce_tx_cap_few_units = 16;  // ... when the tensor has at most 64 column groups (256 units)
  int reduce_blocks_per_cu = 1;   // reduction blocks per compute unit
  int reduce_min_rows = 4;        // fewest rows a thread of a reduction block walks
  int apply_fwd_blocks_per_cu = 16;  // blocks per compute unit in the forward apply pass (one read, one write stream)
  int apply_bwd_blocks_per_cu = 2;   // ... in the backward apply pass (two read streams, one write stream)
  int apply_min_rows = 4;
  int reduce_interleave = 1;      // 1: blocks take every n-th group of rows instead of a contiguous chunk
  int apply_interleave = 0;
  // Folding the finalize into the apply pass's prologue (two launches instead of three).  Backward: a gain
  // at every size measured.  Forward: its apply pass wants many small blocks, each of which would repeat the
  // prologue, so it pays only for small, launch-bound tensors.  0 never, 1 up to fold_fwd_max_elements, 2 always.
  int fold_fwd = 1;
  int fold_bwd = 2;
  size_t fold_fwd_max_elements = size_t(1) << 20;
  // ... with the partial sums already there (the product's epilogue wrote them, at most 16 tile rows): the
  // finalize launch is all that is left to save, which pays up to this many elements
  size_t fold_fwd_epilogue_max_elements = size_t(1) << 22;
  int fc_narrow = 1;              // layers of at most 16 units on a mini-batch run the narrow-layer kernels (fc_small.hip)
  int norm_small = 1;             // mini-batches (at most 256 rows, 2^20 elements) run the one-launch small-batch kernels
  int minibatch_dw = 1;           // weight gradients of a mini-batch (at most 256 rows, 2^20 weights) run the one-block-per-tile kernel of fc_small.hip
  int narrow_dx_fused = 1;        // ... which also form dY = dZn . Wn below a layer of at most 16 units themselves
  int db_in_product = 1;          // a weight gradient split over K forms the bias gradient on its way (no pass over dZ)
};

struct dlmi_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  int num_cu = 256;
  // Device scratch for reduction partials and per-unit constants, grown on
  // demand.  A block that has been handed to kernels is never freed before the
  // context is destroyed (recorded HIP graphs keep its address): growing
  // retires it and allocates a larger one.
  char *scratch = nullptr;
  size_t scratch_bytes = 0;
  char *retired[32] = {nullptr};
  int n_retired = 0;
  // this device's copy of the fixed scratch array of the entry point that allocates nothing
  char *static_scratch = nullptr;
  size_t static_scratch_bytes = 0;
  dlmi_tuning tune;
  // single-launch (column panel) normalization kernels: barrier words in device memory, whether this
  // device qualifies (256 CUs, 32 workgroups of a 256-workgroup launch on each of 8 XCDs), and whether
  // a kernel of this context has been recorded into a HIP graph.  A kernel that gives up says so in two words
  // of pinned host memory (panel_flag_host; the same memory as the device sees it: panel_flag_dev), which the
  // host reads after every synchronization of the stream.
  unsigned *panel_state = nullptr;
  unsigned *panel_flag_host = nullptr, *panel_flag_dev = nullptr;
  int panel_spin_limit = 1 << 20;
  int panel_ok = 0;
  int panel_in_graph = 0;
  // one word in device memory, 0 between launches: the ticket by which the blocks of a seed-gradient kernel find
  // the one that finishes last (block_pairs.hpp)
  unsigned *pair_ticket = nullptr;
  // measurement aid (DLMI_GEMM_CLOCK=1 when the context is created): two 64-bit words in which the first tile of
  // every product launch leaves the engine clock ticks and the 100 MHz reference ticks it spent
  unsigned long long *gemm_clock = nullptr;
  char err[512] = {0};
};

inline char *dlmi_scratch_data(dlmi_ctx const *ctx) { return ctx->scratch; }

inline int dlmi_fail(dlmi_ctx *ctx, int code, char const *fmt, ...) {
  if (ctx != nullptr) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ctx->err, sizeof(ctx->err), fmt, ap);
    va_end(ap);
  }
  return code;
}

#define DLMI_HIP(ctx, call)                                                              \
  do {                                                                                   \
    hipError_t e_ = (call);                                                              \
    if (e_ != hipSuccess)                                                                \
      return dlmi_fail((ctx), DLMI_E_HIP, "%s failed: %s (%s:%d)", #call,                \
                       hipGetErrorString(e_), __FILE__, __LINE__);                       \
  } while (0)

// After a kernel launch: surfaces launch-configuration errors without syncing.
#define DLMI_LAUNCH_CHECK(ctx, what)                                                     \
  do {                                                                                   \
    hipError_t e_ = hipGetLastError();                                                   \
    if (e_ != hipSuccess)                                                                \
      return dlmi_fail((ctx), DLMI_E_HIP, "launch of %s failed: %s", (what),             \
                       hipGetErrorString(e_));                                           \
  } while (0)

#define DLMI_REQUIRE(ctx, cond, msg)                                                     \
  do {                                                                                   \
    if (!(cond)) return dlmi_fail((ctx), DLMI_E_INVALID, "%s: %s", __func__, (msg));      \
  } while (0)

// Makes sure the context's scratch holds at least `bytes`.
// Growing allocates (and synchronizes the stream): it is refused while the
// stream is being captured into a HIP graph.
int dlmi_scratch_reserve(dlmi_ctx *ctx, size_t bytes);

namespace dlmi {
// Finds the device address of the library's fixed scratch array for the context's device (current).
int static_scratch_init(dlmi_ctx *ctx);
void static_scratch_release_stream(dlmi_ctx *ctx);
// Batch-(re)norm forward tail (finalize + apply) from column-sum partials
// [2][nchunks][H] that a producer (the GEMM epilogue) already wrote.
// partial == nullptr: the statistics come from a pass over x.  mov_snapshot != nullptr: [2][H], the moving
// statistics as they were before this step (the producer copied them); with at most kNormFoldChunks chunks the
// apply pass then does the per-unit arithmetic itself and no finalize kernel runs.  residual != nullptr:
// y = residual + (activation output after dropout), the identity shortcut of a block.
int fused_fwd_from_partials(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                            float const *gamma, float const *beta, uint8_t const *mask, float const *residual,
                            float *mean, float *stdv, float *mov_mean, float *mov_std, float *r, float *d, float *y,
                            float const *partial, unsigned nchunks, float const *slices = nullptr,
                            unsigned nslices = 0, float const *mov_snapshot = nullptr);
// Most chunks of partial sums an apply pass adds up itself (its prologue) instead of a finalize kernel.
constexpr unsigned kNormFoldChunks = 16;
// Whether a [B, H] tensor runs the small-batch normalization kernels.  Those also accept x as `nslices`
// partial products [nslices][B][H] still to be added (the slices of a split-K product, passed to
// fused_fwd_from_partials with x = where the sum is to be stored): a producer may skip its own reduction then.
bool small_norm_eligible(dlmi_ctx const *ctx, size_t B, size_t H);
// out[j] (+)= sum over the B rows of x[b, j], in a fixed order (the statistics
// pass of the normalization kernels with its second plane unused).
int column_sums(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float *out, int accumulate);
// Scratch bytes the calls of this library may ask for on a layer [B, K] -> [B, H] / on [*, H] normalized units.
size_t fc_scratch_bytes(dlmi_ctx const *ctx, size_t B, size_t K, size_t H);
size_t norm_scratch_bytes(dlmi_ctx const *ctx, size_t H);
// Column panel kernels (norm_panel_*.hip): set-up at context creation, inspection after a synchronize,
// scratch they need for [*, H].
int panel_init(dlmi_ctx *ctx);
void panel_destroy(dlmi_ctx *ctx);
int panel_check(dlmi_ctx *ctx);
// The context lets go of its stream (destroyed, or given another one), which the caller may destroy next:
// after the stream's work has completed, the cross-stream ordering of panel launches forgets it.
void panel_release_stream(dlmi_ctx *ctx);
size_t panel_scratch_bytes(size_t H);
size_t panel_db_offset(size_t H);        // where the backward kernel's bias-gradient partials start in the scratch
size_t panel_scratch_bytes_db(size_t H);  // scratch of a backward launch that also leaves those partials
// Narrow layers on a mini-batch (fc_small.hip).  narrow_fc_fwd: Z = X W^T + bias and, with Q != nullptr,
// Q = softmax(Z), one launch, and with Y != nullptr (targets [B,H]; Q and dZ required) also the cross-entropy seed
// gradient dZ and stats[0] += loss sum, stats[1] += correct predictions (stats may be nullptr); call only when
// narrow_fc_fwd_eligible.  narrow_dw_try: dW and db in one launch;
// returns 1 when launched, 0 when the shape does not qualify, < 0 on failure.
bool narrow_fc_fwd_eligible(dlmi_ctx const *ctx, size_t B, size_t H);
int narrow_fc_fwd(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *X, float const *W, float const *bias, float *Z,
                  float *Q, float const *Y = nullptr, float *dZ = nullptr, double *stats = nullptr);
int narrow_dw_try(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *Xin, float const *dZ, float *dW, float *db,
                  int accumulate);
// The weight gradient of a layer of any width on a mini-batch (fc_small.hip): dW only, the bias gradient is the
// caller's.  _try: 1 when launched, 0 when the shape or the operands do not qualify, < 0 on failure.
bool minibatch_dw_eligible(dlmi_ctx const *ctx, size_t B, size_t K, size_t H, float const *Xin, float const *dZ, float const *dW);
int minibatch_dw_try(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *Xin, float const *dZ, float *dW, int accumulate);
// ... of several layers in one launch (every problem must be minibatch_dw_eligible; same bits as one by one)
constexpr int kMinibatchDwGroupMax = 8;
struct MinibatchDwProblem {
  size_t B, K, H;
  float const *X, *dZ;
  float *dW;
};
// `narrow`: optionally the weight and bias gradient (db may be null) of one narrow layer (narrow_dw_eligible: at most
// 16 units, 256 rows) rides along in the first launch, computed as the narrow-layer kernel of its own would
struct NarrowDwProblem {
  size_t B, K, H;
  float const *X, *dZ;
  float *dW, *db;
};
bool narrow_dw_eligible(dlmi_ctx const *ctx, size_t B, size_t H);
int minibatch_dw_group(dlmi_ctx *ctx, size_t n, MinibatchDwProblem const *problems, int accumulate,
                       NarrowDwProblem const *narrow = nullptr);
// The fused backward of dlmi_fused_norm_act_bwd whose upstream gradient dY is still `nslices` partial products
// [nslices][B][H] (split-K slices of the dX product above it); small-batch shapes only.
int fused_bwd_from_slices(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                          float const *gamma, float const *beta, uint8_t const *mask, float const *mean,
                          float const *stdv, float const *r, float const *d, float const *slices, unsigned nslices,
                          float *dgamma, float *dbeta, float *dX);
// The same with dY = dZn [B][Hn] . Wn [Hn][H] of a narrow layer above (Hn <= fused_bwd_narrow_max()), formed inside
// the small-batch kernel: no product launch at all.
unsigned fused_bwd_narrow_max();
int fused_bwd_from_narrow(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H, float const *x,
                          float const *gamma, float const *beta, uint8_t const *mask, float const *mean,
                          float const *stdv, float const *r, float const *d, float const *dZn, float const *Wn,
                          size_t Hn, float *dgamma, float *dbeta, float *dX);
}  // namespace dlmi

inline bool dlmi_aligned16(void const *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline size_t dlmi_ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }
