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

// 16 bytes from an LDS byte address (a 32-bit address the compiler need not prove to be LDS: through a
// generic pointer every read carries a null check and a select)
__device__ __forceinline__ uint4 lds16_at(uint32_t addr) {
  const u32x4 v = *(const OHARA_LDS u32x4*)(uintptr_t)addr;
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float bf2f(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// Round-to-nearest-even, the rounding torch applies when a float result is stored
// to a bfloat16 tensor (hardware v_cvt_pk_bf16_f32).
__device__ __forceinline__ bf16_t f2bf(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }

// Round a float through bfloat16 and back: one reference rounding point.
__device__ __forceinline__ float rbf(float f) { return bf2f(f2bf(f)); }

// Softmax bookkeeping of the bf16 attention kernels.  The library kernel the reference calls rounds the
// softmax weights to bf16 before their product with V (ohara/models/llama.py:116-123 ->
// F.scaled_dot_product_attention).  A bf16 rounding commutes with a scaling by a power of two, so the
// kernels here keep scores in log2 units, take the running maximum up to the next INTEGER and form
// p = 2^(s - M): whatever M a chunk, a wave or a tile happens to use, the rounded weights are the same
// bits times an exact power of two, and every later rescale 2^(M_old - M_new) is exact too.  The result
// then depends on how the context is cut (chunks, tiles, kernels) only through the order of fp32 sums.
#define OHARA_LOG2E 1.4426950408889634f
// 2^d for an integer-valued d <= 0 (d = -inf or NaN gives 2^-126, which only ever multiplies a zero)
__device__ __forceinline__ float pow2_neg_int(float d) {
  return __int_as_float(((int)fmaxf(d, -126.f) + 127) << 23);
}

__device__ __forceinline__ float lo_bf(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float hi_bf(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }
// (as a two-element vector conversion this is ONE v_cvt_pk_bf16_f32; two scalar conversions glued together with a
// shift and an or were four instructions)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// (q + 128) * scale + min in fp32, rounded to bf16 (kv_cache.py:30-32, 116-118): four bytes -> two
// packed bf16 pairs.  `w` already has 0x80 xor-ed in, i.e. holds q + 128 as unsigned bytes.  The
// scales written by the quantiser are bf16 values (8 significant bits) and q + 128 has at most 8,
// so the product is exact in fp32 and one fused multiply-add gives bit for bit what the separate
// multiply and add of the reference give.
__device__ __forceinline__ uint2 dequant4(uint32_t w, float s, float m) {
  const float f0 = __fmaf_rn((float)(w & 0xffu), s, m);
  const float f1 = __fmaf_rn((float)((w >> 8) & 0xffu), s, m);
  const float f2 = __fmaf_rn((float)((w >> 16) & 0xffu), s, m);
  const float f3 = __fmaf_rn((float)(w >> 24), s, m);
  return make_uint2(pack_bf(f0, f1), pack_bf(f2, f3));
}

// Butterfly exchanges across the wave without the LDS crossbar.  __shfl_xor compiles to
// ds_bpermute_b32 (an LDS-pipeline round trip of ~100 cycles per step of a reduction); for a
// compile-time lane mask the same exchange is a DPP move (masks 1, 2, 4, 8: inside a row of 16
// lanes) or one of gfx950's row swaps (v_permlane16_swap / v_permlane32_swap: masks 16, 32), a few
// cycles each.  All lanes of the wave must be active.  lane_xor<M>(v) returns v of lane ^ M for
// M < 16; for 16 and 32 only the combined forms below exist (the swap hands every lane its own and
// its partner's value in an order that depends on the row, which a commutative op does not care
// about, so the results equal those of the shuffle butterfly bit for bit).
template <int M>
__device__ __forceinline__ uint32_t lane_xor_u32(uint32_t u) {
  static_assert(M == 1 || M == 2 || M == 4 || M == 8, "DPP masks");
  if (M == 1) return (uint32_t)__builtin_amdgcn_mov_dpp((int)u, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
  if (M == 2) return (uint32_t)__builtin_amdgcn_mov_dpp((int)u, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
  if (M == 8) return (uint32_t)__builtin_amdgcn_mov_dpp((int)u, 0x128, 0xF, 0xF, true);  // row_ror:8
  // mask 4: lanes 0-3 and 8-11 of a row read four lanes up, the others four lanes down
  uint32_t r = (uint32_t)__builtin_amdgcn_update_dpp((int)u, (int)u, 0x104, 0xF, 0x5, false);  // row_shl:4
  return (uint32_t)__builtin_amdgcn_update_dpp((int)r, (int)u, 0x114, 0xF, 0xA, false);        // row_shr:4
}
template <int M>
__device__ __forceinline__ float lane_xor(float v) {
  return __uint_as_float(lane_xor_u32<M>(__float_as_uint(v)));
}
template <int M>
__device__ __forceinline__ void lane_swap(float v, float& a, float& b) {  // {a, b} = {own, partner} in some order
  static_assert(M == 16 || M == 32, "row swaps");
  const uint32_t u = __float_as_uint(v);
  const u32x2 r = M == 16 ? __builtin_amdgcn_permlane16_swap(u, u, false, false)
                          : __builtin_amdgcn_permlane32_swap(u, u, false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
// One butterfly step of an arg-max under the strict order "larger value, then lower index" (a value
// that is not greater than -inf, such as NaN, never wins): (v, i) becomes the better of this lane's and
// lane ^ M's pair.  The winner of a strict order does not depend on the order of the exchanges, so a
// butterfly of these steps returns what the shuffle butterfly returns.
template <int M>
__device__ __forceinline__ void lane_xor_argmax(float& v, int& i) {
  if constexpr (M >= 16) {
    const u32x2 vv = M == 16 ? __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false)
                             : __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const u32x2 ii = M == 16 ? __builtin_amdgcn_permlane16_swap((uint32_t)i, (uint32_t)i, false, false)
                             : __builtin_amdgcn_permlane32_swap((uint32_t)i, (uint32_t)i, false, false);
    const float v0 = __uint_as_float(vv[0]), v1 = __uint_as_float(vv[1]);
    const int i0 = (int)ii[0], i1 = (int)ii[1];
    const bool first = v0 > v1 || (v0 == v1 && i0 < i1) || !(v1 > v0 || (v1 == v0 && i1 < i0)) && i0 <= i1;
    v = first ? v0 : v1;
    i = first ? i0 : i1;
  } else {
    const float ov = lane_xor<M>(v);
    const int oi = (int)lane_xor_u32<M>((uint32_t)i);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

// Inclusive prefix sum across the 64 lanes of a wave, in lane order, through DPP moves (shifts
// inside a row of 16 lanes, then the last lane of a row broadcast into the rows after it): six
// moves instead of six LDS-crossbar shuffles.  All lanes of the wave must be active.
__device__ __forceinline__ int wave_incl_scan_i(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

template <int M>
__device__ __forceinline__ float lane_xor_sum(float v) {  // v + v of lane ^ M
  if constexpr (M >= 16) {
    float a, b;
    lane_swap<M>(v, a, b);
    return a + b;
  } else {
    return v + lane_xor<M>(v);
  }
}
template <int M>
__device__ __forceinline__ float lane_xor_max(float v) {  // fmaxf(v, v of lane ^ M)
  if constexpr (M >= 16) {
    float a, b;
    lane_swap<M>(v, a, b);
    return fmaxf(a, b);
  } else {
    return fmaxf(v, lane_xor<M>(v));
  }
}

template <int M>
__device__ __forceinline__ float lane_xor_min(float v) {  // fminf(v, v of lane ^ M)
  if constexpr (M >= 16) {
    float a, b;
    lane_swap<M>(v, a, b);
    return fminf(a, b);
  } else {
    return fminf(v, lane_xor<M>(v));
  }
}
template <int M>
__device__ __forceinline__ int lane_xor_sum(int v) {  // v + v of lane ^ M
  if constexpr (M >= 16) {
    const u32x2 r = M == 16 ? __builtin_amdgcn_permlane16_swap((uint32_t)v, (uint32_t)v, false, false)
                            : __builtin_amdgcn_permlane32_swap((uint32_t)v, (uint32_t)v, false, false);
    return (int)(r[0] + r[1]);
  } else {
    return v + (int)lane_xor_u32<M>((uint32_t)v);
  }
}
template <int M>
__device__ __forceinline__ int lane_xor_max(int v) {  // max(v, v of lane ^ M)
  if constexpr (M >= 16) {
    const u32x2 r = M == 16 ? __builtin_amdgcn_permlane16_swap((uint32_t)v, (uint32_t)v, false, false)
                            : __builtin_amdgcn_permlane32_swap((uint32_t)v, (uint32_t)v, false, false);
    return max((int)r[0], (int)r[1]);
  } else {
    return max(v, (int)lane_xor_u32<M>((uint32_t)v));
  }
}
// Butterfly steps for masks HI, HI / 2, ..., LO (powers of two), in that order.
template <int HI, int LO, typename T>
__device__ __forceinline__ T lanes_sum(T v) {
  v = lane_xor_sum<HI>(v);
  if constexpr (HI > LO) return lanes_sum<HI / 2, LO, T>(v);
  else return v;
}
template <int HI, int LO, typename T>
__device__ __forceinline__ T lanes_max(T v) {
  v = lane_xor_max<HI>(v);
  if constexpr (HI > LO) return lanes_max<HI / 2, LO, T>(v);
  else return v;
}
template <int HI, int LO>
__device__ __forceinline__ float lanes_min(float v) {
  v = lane_xor_min<HI>(v);
  if constexpr (HI > LO) return lanes_min<HI / 2, LO>(v);
  else return v;
}

// Sum / maximum over the wave, every lane gets the result; the order of the adds is that of the
// butterfly 32, 16, 8, 4, 2, 1.
__device__ __forceinline__ float wave_sum(float v) {
  v = lane_xor_sum<32>(v);
  v = lane_xor_sum<16>(v);
  v = lane_xor_sum<8>(v);
  v = lane_xor_sum<4>(v);
  v = lane_xor_sum<2>(v);
  return lane_xor_sum<1>(v);
}
__device__ __forceinline__ float wave_max(float v) {
  v = lane_xor_max<32>(v);
  v = lane_xor_max<16>(v);
  v = lane_xor_max<8>(v);
  v = lane_xor_max<4>(v);
  v = lane_xor_max<2>(v);
  return lane_xor_max<1>(v);
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

// x * sigmoid(x) with the hardware exponential and reciprocal (v_exp_f32, v_rcp_f32: about 1 ulp
// each; every use rounds the result to bf16 right away).  The library expf and the IEEE division
// are some forty instructions, which sixteen fragments per thread in the tiled GEMM's SwiGLU
// epilogue made a fifth of that kernel's time.
__device__ __forceinline__ float silu_f(float x) { return x * __frcp_rn(1.0f + __expf(-x)); }

// Host-side launch check: every entry point returns OHARA_ELAUNCH when the
// launch itself was rejected.
static inline int ohara_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? OHARA_OK : OHARA_ELAUNCH;
}
