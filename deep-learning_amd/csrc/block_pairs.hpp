// Two reported sums (loss and accuracy count) of a seed-gradient kernel, without a second launch and without
// floating-point atomics: every block stores its pair, takes a ticket, and the block that draws the last ticket
// adds all pairs in a fixed order.  Which block that is differs from run to run; the order of the additions,
// and with it the result, does not.
#pragma once
#include <hip/hip_runtime.h>

namespace dlmi {

// Called by all threads of every block of the launch (any block size that is a multiple of 64), after thread 0
// knows this block's pair (l, c).
//   pairs  [2 * gridDim.x] doubles in device memory
//   acc    acc[0] += sum of all l, acc[1] += sum of all c: lane t of one wavefront adds blocks t, t + 64, ...,
//          then the 64 lane totals are added pairwise (lanes 32 apart, then 16, ... 1)
//   ticket one word in device memory, 0 before the launch; the last block leaves it at 0 for the next one
//          (launches that share it must be ordered on one stream)
__device__ __forceinline__ void finish_block_pairs(double l, double c, double *__restrict__ pairs,
                                                   double *__restrict__ acc, unsigned *__restrict__ ticket) {
  __shared__ unsigned s_last;
  unsigned const nblocks = gridDim.x;
  if (threadIdx.x == 0) {
    pairs[2 * blockIdx.x] = l;
    pairs[2 * blockIdx.x + 1] = c;
    // release: the pair is visible on the whole device before the ticket is; acquire: the block that draws the
    // last ticket sees every other block's pair
    unsigned const t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    s_last = t + 1 == nblocks ? 1u : 0u;
    if (t + 1 == nblocks) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (s_last == 0u || threadIdx.x >= 64) return;
  double tl = 0.0, tc = 0.0;
  for (unsigned b = threadIdx.x; b < nblocks; b += 64) {
    tl += __hip_atomic_load(pairs + 2 * b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    tc += __hip_atomic_load(pairs + 2 * b + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  for (int off = 32; off > 0; off >>= 1) {
    tl += __shfl_xor(tl, off, 64);
    tc += __shfl_xor(tc, off, 64);
  }
  if (threadIdx.x == 0) {
    acc[0] += tl;
    acc[1] += tc;
  }
}

}  // namespace dlmi
