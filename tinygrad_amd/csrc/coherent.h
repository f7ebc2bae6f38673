// Accesses for data that one workgroup writes and another workgroup reads inside the same launch.
#pragma once
#include "qfmt.h"

// Data that one workgroup writes and another reads inside the launch (activations, attention partials) moves through relaxed
// device-scope atomic loads / stores: they carry the sc1 cache-policy bit on this ISA, i.e. stores write through to the point
// where every XCD sees them and loads do not hit stale lines in the per-CU L1 or in another XCD's L2.  That keeps cache
// write-back / invalidate instructions (which walk a whole L2 per call) out of the barrier, and unlike volatile accesses they
// do not make the compiler wait for every outstanding load after each one.  Weights, norm weights, the RoPE table and KV rows
// of earlier tokens are read-only during a launch and use plain loads.
__device__ __forceinline__ float cld(const float* p) {
  return __builtin_bit_cast(float, __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ u32x4 cld16(const void* p) {
  const uint64_t lo = __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint64_t hi = __hip_atomic_load((const uint64_t*)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  u32x4 v = {(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
  return v;
}
__device__ __forceinline__ f32x4 cld16f(const void* p) { return __builtin_bit_cast(f32x4, cld16(p)); }
__device__ __forceinline__ void cst(float* p, float v) { __hip_atomic_store((uint32_t*)p, __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void cst_h(_Float16* p, float v) {
  __hip_atomic_store((uint16_t*)p, __builtin_bit_cast(uint16_t, (_Float16)v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// all of this thread's stores have reached memory
__device__ __forceinline__ void stores_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

