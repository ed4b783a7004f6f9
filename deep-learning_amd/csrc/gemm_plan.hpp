// Host-side launch planning of the FP32 MFMA products (csrc/gemm_f32_mfma.hip): which tile shape, how many K
// slices and how many register stages a product C[M,N] = A[M,K] . B[K,N] takes, from its shape and the number of
// compute units alone.  Pure host arithmetic (host/gemm_plan.cpp); the kernels live in the .hip file.
#ifndef DLMI_GEMM_PLAN_HPP
#define DLMI_GEMM_PLAN_HPP

#include <cstddef>

struct dlmi_ctx;

namespace dlmi {

// Tile shape and K split of a product, from its shape alone.
struct GemmPlan {
  int choice, bm, bn, bk;  // choice: 0 128x128, 1 256x128, 2 256x256, 3 64x64 (4 wavefronts); 4 128x128 (8 wavefronts)
  int waves;               // wavefronts per workgroup: 4 or 8
  unsigned splits;         // K slices (1: none)
  size_t scratch_bytes;    // partial products of the slices
};
GemmPlan plan_gemm(int num_cu, size_t M, size_t N, size_t K);
// Register stages of the K loop: two for the small tiles from 32 K tiles per slice on, one otherwise.
int gemm_register_stages(int bm, int bn, size_t kt_per_split);

}  // namespace dlmi

#endif  // DLMI_GEMM_PLAN_HPP
