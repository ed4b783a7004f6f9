// Context management of the dlmi C ABI.
#include "dlmi_common.hpp"

int dlmi_scratch_reserve(dlmi_ctx *ctx, size_t bytes) {
  if (bytes <= ctx->scratch_bytes) return DLMI_OK;
  // Work already queued on the stream may still read the old block.
  DLMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
  if (ctx->scratch != nullptr) DLMI_HIP(ctx, hipFree(ctx->scratch));
  ctx->scratch = nullptr;
  ctx->scratch_bytes = 0;
  size_t const want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
  void *p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) {
    (void)hipGetLastError();
    return dlmi_fail(ctx, DLMI_E_NOMEM, "scratch allocation of %zu bytes failed", want);
  }
  ctx->scratch = static_cast<char *>(p);
  ctx->scratch_bytes = want;
  return DLMI_OK;
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
  int rc = dlmi_scratch_reserve(ctx, size_t(16) << 20);
  if (rc != DLMI_OK) {
    delete ctx;
    return rc;
  }
  *out = ctx;
  return DLMI_OK;
}

int dlmi_ctx_destroy(dlmi_ctx *ctx) {
  if (ctx == nullptr) return DLMI_OK;
  (void)hipStreamSynchronize(ctx->stream);
  if (ctx->scratch != nullptr) (void)hipFree(ctx->scratch);
  delete ctx;
  return DLMI_OK;
}

int dlmi_ctx_set_stream(dlmi_ctx *ctx, void *stream) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  ctx->stream = static_cast<hipStream_t>(stream);
  return DLMI_OK;
}

int dlmi_ctx_synchronize(dlmi_ctx *ctx) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return DLMI_OK;
}

char const *dlmi_last_error(dlmi_ctx const *ctx) { return ctx != nullptr ? ctx->err : "null context"; }

int dlmi_ctx_compute_units(dlmi_ctx const *ctx) { return ctx != nullptr ? ctx->num_cu : 0; }

}  // extern "C"
