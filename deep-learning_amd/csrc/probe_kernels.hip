// Measurement aid, not part of any product path: how fast this device streams a [B, H] fp32 tensor when it is
// walked the way the single-launch (column panel) normalization kernels walk it - 256 workgroups of 512 threads,
// XCD x (workgroup id % 8) owns columns [x * H / 8, (x + 1) * H / 8) and goes through them in panels of 64 columns,
// workgroup rank r (id / 8) owns rows [r * B / 32, (r + 1) * B / 32) - and nothing else is done with the data.
// The time of this kernel is the memory floor of those kernels' access pattern; the rate of a plain device copy or
// the 8 TB/s of the data sheet are not.
#include "dlmi_common.hpp"

namespace dlmi {
namespace {

typedef float v4 __attribute__((ext_vector_type(4)));
constexpr int kPanel = 64;                    // columns of a panel
constexpr int kLanesPerRow = kPanel / 4;      // 16 lanes x 16 bytes
constexpr int kRowsPerSweep = 512 / kLanesPerRow;

// y = x (TWO == false) or y = x + x2 (TWO == true): one or two tensors read once, one written once.
template <bool TWO>
__global__ __launch_bounds__(512) void k_probe_strip(float const *__restrict__ x, float const *__restrict__ x2,
                                                      float *__restrict__ y, int B, int H) {
  int const xcd = blockIdx.x % 8, rank = blockIdx.x / 8;
  int const cols = H / 8, rows = B / 32;
  int const tx = threadIdx.x % kLanesPerRow, ty = threadIdx.x / kLanesPerRow;
  for (int p = 0; p < cols / kPanel; ++p) {
    size_t const first = (static_cast<size_t>(rank) * rows + ty) * H + static_cast<size_t>(xcd) * cols + p * kPanel + tx * 4;
    for (int r = 0; r < rows; r += kRowsPerSweep * 4) {
      v4 v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[i] = __builtin_nontemporal_load(reinterpret_cast<v4 const *>(x + first + static_cast<size_t>(r + i * kRowsPerSweep) * H));
      if constexpr (TWO) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          v[i] += __builtin_nontemporal_load(reinterpret_cast<v4 const *>(x2 + first + static_cast<size_t>(r + i * kRowsPerSweep) * H));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
        __builtin_nontemporal_store(v[i], reinterpret_cast<v4 *>(y + first + static_cast<size_t>(r + i * kRowsPerSweep) * H));
    }
  }
}

}  // namespace
}  // namespace dlmi

using namespace dlmi;

extern "C" int dlmi_probe_strip_stream(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float const *x2, float *y) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, x != nullptr && y != nullptr, "null pointer");
  // whole panels for every XCD, whole sweeps of 4 x 32 rows for every rank
  DLMI_REQUIRE(ctx, H % (8 * kPanel) == 0 && B % (32 * kRowsPerSweep * 4) == 0 && B * H < (size_t(1) << 40),
               "the probe takes H in multiples of 512 and B in multiples of 4096");
  DLMI_REQUIRE(ctx, dlmi_aligned16(x) && dlmi_aligned16(y) && (x2 == nullptr || dlmi_aligned16(x2)), "16-byte alignment");
  if (x2 != nullptr)
    hipLaunchKernelGGL(k_probe_strip<true>, dim3(256), dim3(512), 0, ctx->stream, x, x2, y, static_cast<int>(B), static_cast<int>(H));
  else
    hipLaunchKernelGGL(k_probe_strip<false>, dim3(256), dim3(512), 0, ctx->stream, x, x2, y, static_cast<int>(B), static_cast<int>(H));
  DLMI_LAUNCH_CHECK(ctx, "k_probe_strip");
  return DLMI_OK;
}
