// Context management of the dlmi C ABI.
#include <cstdlib>

#include "dlmi_common.hpp"

int dlmi_scratch_reserve(dlmi_ctx *ctx, size_t bytes) {
  if (ctx->scratch != nullptr && bytes <= ctx->scratch_bytes) return DLMI_OK;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(ctx->stream, &cap) != hipSuccess) (void)hipGetLastError();
  if (cap != hipStreamCaptureStatusNone)
    return dlmi_fail(ctx, DLMI_E_INVALID,
                     "scratch would have to grow to %zu bytes while the stream is being captured: run the "
                     "same calls once outside the capture first", bytes);
  if (ctx->scratch != nullptr && ctx->n_retired >= static_cast<int>(sizeof(ctx->retired) / sizeof(ctx->retired[0])))
    return dlmi_fail(ctx, DLMI_E_NOMEM, "scratch grew too many times");
  // at least double, so that a context retires only a handful of blocks in its life
  size_t want = bytes > 2 * ctx->scratch_bytes ? bytes : 2 * ctx->scratch_bytes;
  want = (want + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
  void *p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) {
    (void)hipGetLastError();
    return dlmi_fail(ctx, DLMI_E_NOMEM, "scratch allocation of %zu bytes failed", want);
  }
  // Work already queued (or recorded into a graph) may still use the old block:
  // it stays allocated until the context goes.
  if (ctx->scratch != nullptr) ctx->retired[ctx->n_retired++] = ctx->scratch;
  ctx->scratch = static_cast<char *>(p);
  ctx->scratch_bytes = want;
  return DLMI_OK;
}

static int env_knob(char const *name, int dflt) {
  char const *e = getenv(name);
  if (e == nullptr || *e == 0) return dflt;
  int const v = atoi(e);
  return v > 0 ? v : dflt;
}

static int env_level(char const *name, int dflt) {
  char const *e = getenv(name);
  return (e == nullptr || *e == 0) ? dflt : atoi(e);
}
static int env_flag(char const *name, int dflt) {
  char const *e = getenv(name);
  return (e == nullptr || *e == 0) ? dflt : (atoi(e) != 0 ? 1 : 0);
}

extern "C" {

int dlmi_ctx_create(dlmi_ctx **out, int device, void *stream) {
  if (out == nullptr) return DLMI_E_INVALID;
  *out = nullptr;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0 || device < 0 || device >= n) {
    (void)hipGetLastError();
    return DLMI_E_HIP;  // no GPU: there is no CPU path to fall back to
  }
  if (hipSetDevice(device) != hipSuccess) return DLMI_E_HIP;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess) return DLMI_E_HIP;
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    fprintf(stderr, "dlmi: device %d is %s; this library is built for gfx950 only\n", device,
            prop.gcnArchName);
    return DLMI_E_UNSUPPORTED;
  }
  dlmi_ctx *ctx = new dlmi_ctx;
  ctx->device = device;
  ctx->stream = static_cast<hipStream_t>(stream);
  ctx->num_cu = prop.multiProcessorCount;
  dlmi_tuning &t = ctx->tune;
  t.reduce_tx_cap = env_knob("DLMI_NORM_REDUCE_TX", t.reduce_tx_cap);
  t.reduce_tx_cap_few_units = env_knob("DLMI_NORM_REDUCE_TX_FEW_UNITS", t.reduce_tx_cap_few_units);
  t.reduce_blocks_per_cu = env_knob("DLMI_NORM_REDUCE_BLOCKS_PER_CU", t.reduce_blocks_per_cu);
  t.reduce_min_rows = env_knob("DLMI_NORM_REDUCE_MIN_ROWS", t.reduce_min_rows);
  t.apply_fwd_blocks_per_cu = env_knob("DLMI_NORM_APPLY_FWD_BLOCKS_PER_CU", t.apply_fwd_blocks_per_cu);
  t.apply_bwd_blocks_per_cu = env_knob("DLMI_NORM_APPLY_BWD_BLOCKS_PER_CU", t.apply_bwd_blocks_per_cu);
  t.apply_min_rows = env_knob("DLMI_NORM_APPLY_MIN_ROWS", t.apply_min_rows);
  t.reduce_interleave = env_flag("DLMI_NORM_REDUCE_INTERLEAVE", t.reduce_interleave);
  t.apply_interleave = env_flag("DLMI_NORM_APPLY_INTERLEAVE", t.apply_interleave);
  t.fold_fwd = env_level("DLMI_NORM_FOLD_FWD", t.fold_fwd);
  t.fold_bwd = env_level("DLMI_NORM_FOLD_BWD", t.fold_bwd);
  t.norm_small = env_flag("DLMI_NORM_SMALL", t.norm_small);
  t.narrow_dx_fused = env_flag("DLMI_NARROW_DX_FUSED", t.narrow_dx_fused);
  t.minibatch_dw = env_flag("DLMI_MINIBATCH_DW", t.minibatch_dw);
  t.fc_narrow = env_flag("DLMI_FC_NARROW", t.fc_narrow);
  t.db_in_product = env_flag("DLMI_DB_IN_PRODUCT", t.db_in_product);
  if (env_flag("DLMI_GEMM_CLOCK", 0)) {
    void *p = nullptr;
    if (hipMalloc(&p, (2 + 4 * 4096) * sizeof(unsigned long long)) == hipSuccess) {
      ctx->gemm_clock = static_cast<unsigned long long *>(p);
      (void)hipMemset(p, 0, (2 + 4 * 4096) * sizeof(unsigned long long));
    } else {
      (void)hipGetLastError();
    }
  }
  int rc = DLMI_OK;
  {
    void *p = nullptr;
    if (hipMalloc(&p, 256) == hipSuccess && hipMemset(p, 0, 256) == hipSuccess) {
      ctx->pair_ticket = static_cast<unsigned *>(p);
    } else {
      (void)hipGetLastError();
      if (p != nullptr) (void)hipFree(p);
      rc = dlmi_fail(ctx, DLMI_E_HIP, "dlmi_ctx_create: no device memory for the ticket word");
    }
  }
  if (rc == DLMI_OK) rc = dlmi_scratch_reserve(ctx, size_t(16) << 20);
  if (rc == DLMI_OK) rc = dlmi::static_scratch_init(ctx);
  if (rc == DLMI_OK) rc = dlmi::panel_init(ctx);
  if (rc != DLMI_OK) {
    fprintf(stderr, "dlmi: %s\n", ctx->err);
    if (ctx->scratch != nullptr) (void)hipFree(ctx->scratch);
    if (ctx->pair_ticket != nullptr) (void)hipFree(ctx->pair_ticket);
    if (ctx->gemm_clock != nullptr) (void)hipFree(ctx->gemm_clock);
    dlmi::panel_destroy(ctx);
    delete ctx;
    return rc;
  }
  *out = ctx;
  return DLMI_OK;
}

int dlmi_ctx_destroy(dlmi_ctx *ctx) {
  if (ctx == nullptr) return DLMI_OK;
  (void)hipStreamSynchronize(ctx->stream);
  dlmi::panel_release_stream(ctx);
  dlmi::static_scratch_release_stream(ctx);
  if (ctx->scratch != nullptr) (void)hipFree(ctx->scratch);
  for (int i = 0; i < ctx->n_retired; ++i) (void)hipFree(ctx->retired[i]);
  dlmi::panel_destroy(ctx);
  if (ctx->gemm_clock != nullptr) (void)hipFree(ctx->gemm_clock);
  if (ctx->pair_ticket != nullptr) (void)hipFree(ctx->pair_ticket);
  delete ctx;
  return DLMI_OK;
}

int dlmi_ctx_set_stream(dlmi_ctx *ctx, void *stream) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  if (ctx->stream == static_cast<hipStream_t>(stream)) return DLMI_OK;
  // the old stream may be destroyed by its owner once the context has let go of it (not while it is being
  // recorded, which is also when it cannot be waited for)
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(ctx->stream, &capturing) != hipSuccess) (void)hipGetLastError();
  if (capturing == hipStreamCaptureStatusNone) {
    DLMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
    dlmi::panel_release_stream(ctx);
    dlmi::static_scratch_release_stream(ctx);
  }
  ctx->stream = static_cast<hipStream_t>(stream);
  return DLMI_OK;
}

int dlmi_ctx_synchronize(dlmi_ctx *ctx) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return dlmi::panel_check(ctx);
}

int dlmi_ctx_reserve_layer(dlmi_ctx *ctx, size_t B, size_t K, size_t H) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  size_t need = dlmi::norm_scratch_bytes(ctx, H);
  if (K != 0) {
    size_t const fc = dlmi::fc_scratch_bytes(ctx, B, K, H);
    if (fc > need) need = fc;
    size_t const nk = dlmi::norm_scratch_bytes(ctx, K);  // a block layer normalizes its input
    if (nk > need) need = nk;
  }
  size_t const pairs = (B / 4 + 2) * 2 * sizeof(double);  // loss / accuracy pairs of a seed kernel
  if (pairs > need) need = pairs;
  return dlmi_scratch_reserve(ctx, need);
}

unsigned long long dlmi_ctx_scratch_generation(dlmi_ctx const *ctx) {
  return ctx != nullptr ? static_cast<unsigned long long>(ctx->n_retired) + 1ull : 0ull;
}

char const *dlmi_last_error(dlmi_ctx const *ctx) { return ctx != nullptr ? ctx->err : "null context"; }

int dlmi_ctx_compute_units(dlmi_ctx const *ctx) { return ctx != nullptr ? ctx->num_cu : 0; }

int dlmi_ctx_gemm_clock(dlmi_ctx *ctx, double *engine_mhz, double *tile_us) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, ctx->gemm_clock != nullptr, "the context was created without DLMI_GEMM_CLOCK=1");
  DLMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
  unsigned long long t[2] = {0, 0};
  DLMI_HIP(ctx, hipMemcpy(t, ctx->gemm_clock, sizeof t, hipMemcpyDeviceToHost));
  DLMI_REQUIRE(ctx, t[1] != 0, "no product has been launched yet");
  double const us = static_cast<double>(t[1]) / 100.0;  // the reference counter runs at 100 MHz
  if (tile_us != nullptr) *tile_us = us;
  if (engine_mhz != nullptr) *engine_mhz = static_cast<double>(t[0]) / us;
  return DLMI_OK;
}

int dlmi_ctx_gemm_timeline(dlmi_ctx *ctx, unsigned long long *out, size_t workgroups) {
  if (ctx == nullptr || out == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, ctx->gemm_clock != nullptr, "the context was created without DLMI_GEMM_CLOCK=1");
  DLMI_REQUIRE(ctx, workgroups <= 4096, "at most 4096 workgroups are kept");
  DLMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
  DLMI_HIP(ctx, hipMemcpy(out, ctx->gemm_clock + 2, 4 * workgroups * sizeof(unsigned long long), hipMemcpyDeviceToHost));
  return DLMI_OK;
}

int dlmi_ctx_norm_panel_enabled(dlmi_ctx const *ctx) { return ctx != nullptr && ctx->panel_ok ? 1 : 0; }

int dlmi_ctx_norm_panel_poke(dlmi_ctx *ctx, unsigned xcd, unsigned word, unsigned value) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, ctx->panel_state != nullptr, "this context has no single-launch normalization kernels");
  DLMI_REQUIRE(ctx, xcd < 8 && word < 16, "no such word");
  DLMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
  DLMI_HIP(ctx, hipMemcpy(ctx->panel_state + xcd * 16 + word, &value, sizeof value, hipMemcpyHostToDevice));
  return DLMI_OK;
}

}  // extern "C"
