// Shared device helpers for the gfx950 decode kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ohara_decode.h"

typedef uint16_t bf16_t;  // raw bfloat16 bits

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define WAVE 64

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Every pointer these helpers take addresses device memory.  Saying so (address space 1) matters
// where the compiler cannot see it - pointers fetched from tables in memory or LDS - because a
// generic ("flat") access also counts as an LDS access, so waiting for LDS data would wait for
// every weight or cache load in flight.
#define OHARA_GLOBAL __attribute__((address_space(1)))
#define OHARA_LDS __attribute__((address_space(3)))

__device__ __forceinline__ uint4 ldg16(const void* p) {
  const u32x4 v = *(const OHARA_GLOBAL u32x4*)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 ldg8(const void* p) {
  const u32x2 v = *(const OHARA_GLOBAL u32x2*)p;
  return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t ldg4(const void* p) { return *(const OHARA_GLOBAL uint32_t*)p; }
// 16-byte load flagged as streaming (read once): keeps reusable data in L2.
__device__ __forceinline__ uint4 ldg16_nt(const void* p) {
  u32x4 v = __builtin_nontemporal_load((const OHARA_GLOBAL u32x4*)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ int64_t ldg_i64(const int64_t* p) { return *(const OHARA_GLOBAL int64_t*)p; }
__device__ __forceinline__ void stg8(void* p, uint2 v) { *(OHARA_GLOBAL u32x2*)p = (u32x2){v.x, v.y}; }
// LDS accesses through a pointer whose address space the compiler cannot see
__device__ __forceinline__ void sts8(void* p, uint2 v) { *(OHARA_LDS u32x2*)p = (u32x2){v.x, v.y}; }
__device__ __forceinline__ void sts16(void* p, uint4 v) {
  *(OHARA_LDS u32x4*)p = (u32x4){v.x, v.y, v.z, v.w};
}
__device__ __forceinline__ uint4 lds16(const void* p) {
  const u32x4 v = *(const OHARA_LDS u32x4*)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float bf2f(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// Round-to-nearest-even, the rounding torch applies when a float result is stored
// to a bfloat16 tensor (hardware v_cvt_pk_bf16_f32).
__device__ __forceinline__ bf16_t f2bf(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }

// Round a float through bfloat16 and back: one reference rounding point.
__device__ __forceinline__ float rbf(float f) { return bf2f(f2bf(f)); }

__device__ __forceinline__ float lo_bf(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float hi_bf(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }
__device__ __forceinline__ uint32_t pack_bf(float lo, float hi) {
  return (uint32_t)f2bf(lo) | ((uint32_t)f2bf(hi) << 16);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Device-coherent accesses without fences.  The eight XCDs' L2 caches are not coherent with
// each other; relaxed agent-scope atomics compile to write-through stores / cache-bypassing
// loads (sc1), so data handed from one workgroup to another is published by such stores, a
// wait of EVERY storing wave for their completion (wait_own_stores below), a workgroup barrier
// and then a relaxed atomic counter, and is read with such loads.  An agent-scope fence instead
// writes back / invalidates a whole L2, which serialises across workgroups (~0.2 us each on
// this chip).
__device__ __forceinline__ void st_coh8(void* p, uint2 v) {
  __hip_atomic_store((OHARA_GLOBAL unsigned long long*)p, ((unsigned long long)v.y << 32) | v.x, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_coh4(void* p, uint32_t v) {
  __hip_atomic_store((OHARA_GLOBAL uint32_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint2 ld_coh8(const void* p) {
  const unsigned long long v =
      __hip_atomic_load((const OHARA_GLOBAL unsigned long long*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_uint2((uint32_t)v, (uint32_t)(v >> 32));
}
__device__ __forceinline__ uint4 ld_coh16(const void* p) {
  const uint2 a = ld_coh8(p), b = ld_coh8(reinterpret_cast<const char*>(p) + 8);
  return make_uint4(a.x, a.y, b.x, b.y);
}
__device__ __forceinline__ uint32_t ld_coh4(const void* p) {
  return __hip_atomic_load((const OHARA_GLOBAL uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Waits until every global store (and load) this wave has issued has completed: s_waitcnt
// vmcnt(0) lgkmcnt(0).  A workgroup-scope release fence does NOT do this on gfx950 (the L1 keeps
// a workgroup's accesses in order, so the fence emits no vmcnt wait): a wave that only passes the
// workgroup barrier may still have write-through stores in flight when another wave bumps the
// cross-workgroup counter.  So every wave calls this before that barrier.
__device__ __forceinline__ void wait_own_stores() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x0070);
  asm volatile("" ::: "memory");
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }

// Host-side launch check: every entry point returns OHARA_ELAUNCH when the
// launch itself was rejected.
static inline int ohara_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? OHARA_OK : OHARA_ELAUNCH;
}
