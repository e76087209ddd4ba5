// "Last workgroup finishes the job": a grid-wide hand-off without a second launch.
//
// Every workgroup calls last_block_done() after its global writes. The call that brings
// the counter to `total` returns true in exactly one workgroup, after every other
// workgroup's writes have been made visible device-wide (release fence before the
// increment, acquire fence after it; on a multi-die GPU these fences are what write
// back and invalidate the per-die L2, so ordinary loads in the tail see the data).
// The winner also resets the counter, so the same counter serves the next launch on
// the stream. No workgroup ever waits on another: there is nothing here that can hang.
#pragma once

#include <hip/hip_runtime.h>

__device__ __forceinline__ bool last_block_done(unsigned int* counter, unsigned int total) {
  __shared__ int s_last;
  __threadfence();  // each thread publishes its own stores
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned int prev = atomicAdd(counter, 1u);
    const int last = prev + 1u == total;
    if (last) atomicExch(counter, 0u);
    s_last = last;
  }
  __syncthreads();
  const bool last = s_last != 0;
  if (last) __threadfence();  // acquire: drop stale cached lines before reading others' results
  return last;
}
