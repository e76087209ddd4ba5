// Hand-offs between workgroups of ONE launch.
//
// A launch boundary costs about 2.5 us on this part and forces the consumer's weight loads
// to start cold. Where a small intermediate (router gates, expert activations) is all that
// separates two phases, both run in one grid and the intermediate crosses through memory:
//
//   producer   data with agent-scope relaxed stores (`sc1`: written through, never left
//              dirty in the die's L2), s_waitcnt vmcnt(0) (the stores have been acknowledged),
//              workgroup barrier, then ONE agent-scope store of the launch's epoch number to the
//              workgroup's own flag word;
//   consumer   a wavefront polls the flag words it depends on with agent-scope relaxed loads
//              (one coalesced load a round), then reads the data with agent-scope loads
//              (they bypass the die's L2, so no stale line can be hit).
//
// No atomics (1152 adds on one counter measured 27 us: about 24 ns each, serialised across the
// eight dies) and no fences (a device-scope release per workgroup writes the die's L2 back and
// measured 130 us for the same pattern). An epoch is used once: the host hands every launch
// the next number, so a flag left by an earlier launch never matches.
//
// Deadlock freedom: workgroups are dispatched in index order and a consumer only ever waits
// for workgroups of lower index, so the lowest unfinished workgroup can always run. Every
// wait is also bounded: after `max_spins` rounds the wavefront gives up, reports through
// `*err` (a word the host checks at its next synchronisation) and finishes with whatever it
// reads, so the grid always drains.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

// The stores are written as instructions rather than as agent-scope atomic builtins: the
// builtin forms act as scheduling fences for everything around them (the expert kernel grew
// from 94 to 150 vector registers with one of them at its end); `sc1` is the bit the compiler
// itself sets for an agent-scope store. ho_wait_stores() orders them where order matters.
__device__ __forceinline__ void ho_store_u16(void* p, uint16_t v) {
  asm volatile("global_store_short %0, %1, off sc1" ::"v"(p), "v"((uint32_t)v));
}
__device__ __forceinline__ void ho_store_u32(void* p, uint32_t v) {
  asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v));
}
__device__ __forceinline__ void ho_store_u64(void* p, uint64_t v) {
  asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(p), "v"(v));
}
__device__ __forceinline__ uint16_t ho_load_u16(const void* p) {
  return __hip_atomic_load(static_cast<const uint16_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ho_load_u32(const void* p) {
  return __hip_atomic_load(static_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ho_load_u64(const void* p) {
  return __hip_atomic_load(static_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// every store this wavefront has issued has been acknowledged by memory
__device__ __forceinline__ void ho_wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Producer side, called by all threads of the workgroup after their data stores.
__device__ __forceinline__ void ho_publish(uint32_t* flag, uint32_t epoch) {
  ho_wait_stores();
  __syncthreads();
  if (threadIdx.x == 0) ho_store_u32(flag, epoch);
}

// Consumer side, called by all 64 lanes of a wavefront: waits until flags[0..n) all hold
// `epoch`. Returns false (and leaves a mark in *err) if the bound ran out.
__device__ __forceinline__ bool ho_wait(const uint32_t* flags, int n, uint32_t epoch, int max_spins,
                                        uint32_t* err, int lane) {
  for (int base = 0; base < n; base += 64) {
    const int i = base + lane;
    int spins = 0;
    for (;;) {
      const uint32_t f = i < n ? ho_load_u32(flags + i) : epoch;
      if (__all(f == epoch)) break;
      if (++spins >= max_spins) {
        if (lane == 0) __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        return false;
      }
      __builtin_amdgcn_s_sleep(1);
    }
  }
  asm volatile("" ::: "memory");
  return true;
}
