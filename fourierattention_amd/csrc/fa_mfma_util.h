// Types and small device helpers shared by the MFMA kernels (gfx950, wave64).
#pragma once

#include "fa_common.h"

namespace fa_mfma {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));

template <typename E> struct Mma;
template <> struct Mma<bf16_t> {
  using vec8 = bf16x8;
  using elem = __bf16;
  static __device__ __forceinline__ float4v mma(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ elem from_bits(bf16_t x) { return __builtin_bit_cast(__bf16, x.bits); }
};
template <> struct Mma<f16_t> {
  using vec8 = half8;
  using elem = _Float16;
  static __device__ __forceinline__ float4v mma(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ elem from_bits(f16_t x) { return x.v; }
};

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt[3:0] | expcnt 7 << 4 | lgkmcnt 15 << 8 | vmcnt[5:4] << 14)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}
// one fragment (64 lanes x 16 bytes) from global memory straight into LDS at lds_frag + lane * 16
// AUX: cache-policy bits of the load (0 = default, 2 = non-temporal: data that is read once should not
// displace what the neighbouring kernels want to find in the last-level cache)
template <int AUX = 0, typename E>
__device__ __forceinline__ void load_frag_to_lds(const E* g_lane_ptr, void* lds_frag) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g_lane_ptr,
                                   (__attribute__((address_space(3))) void*)lds_frag, 16, 0, AUX);
}

// LDS accesses that the compiler must not tie to the asynchronous page loads (it would otherwise wait
// for every outstanding global_load_lds before each read and before each barrier)
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4v lds_read_b128_async(const void* lds_ptr) {
  uint4v r;
  const unsigned addr = (unsigned)(size_t)(const __attribute__((address_space(3))) void*)lds_ptr;
  asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr));
  return r;
}
// the same at lds_addr + OFF with OFF in the instruction's immediate field: reads of one structure share one
// address register instead of computing (and keeping) an address each
__device__ __forceinline__ unsigned lds_addr_of(const void* lds_ptr) {
  return (unsigned)(size_t)(const __attribute__((address_space(3))) void*)lds_ptr;
}
template <int OFF>
__device__ __forceinline__ uint4v lds_read_b128_async_at(unsigned lds_addr) {
  static_assert(OFF >= 0 && OFF < 65536 && OFF % 16 == 0, "immediate offset of ds_read_b128");
  uint4v r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(lds_addr), "n"(OFF));
  return r;
}
// the read above completes asynchronously: tie the wait to the value so no use can be scheduled before it
__device__ __forceinline__ void lds_wait_for(uint4v& r) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r)::"memory"); }
// same for a batch of four reads, leaving the AFTER LDS operations issued after the batch in flight (LDS
// operations complete in issue order, so a count is enough; later LDS traffic only makes the wait longer)
template <int AFTER>
__device__ __forceinline__ void lds_wait_for4(uint4v (&r)[4]) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]) : "n"(AFTER) : "memory");
}
// the same for two reads
template <int AFTER>
__device__ __forceinline__ void lds_wait_for2(uint4v& a, uint4v& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(AFTER) : "memory");
}
// sum of eight floats STEP bytes apart, read like the accesses above and complete on return
template <int STEP>
__device__ __forceinline__ float lds_sum8_b32(unsigned lds_addr) {
  static_assert(STEP % 4 == 0 && 7 * STEP < 65536, "immediate offsets of ds_read_b32");
  float v0, v1, v2, v3, v4, v5, v6, v7;
  asm volatile(
      "ds_read_b32 %0, %8\n\tds_read_b32 %1, %8 offset:%9\n\tds_read_b32 %2, %8 offset:%10\n\t"
      "ds_read_b32 %3, %8 offset:%11\n\tds_read_b32 %4, %8 offset:%12\n\tds_read_b32 %5, %8 offset:%13\n\t"
      "ds_read_b32 %6, %8 offset:%14\n\tds_read_b32 %7, %8 offset:%15\n\ts_waitcnt lgkmcnt(0)"
      : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5), "=&v"(v6), "=&v"(v7)
      : "v"(lds_addr), "n"(STEP), "n"(2 * STEP), "n"(3 * STEP), "n"(4 * STEP), "n"(5 * STEP), "n"(6 * STEP), "n"(7 * STEP)
      : "memory");
  return ((v0 + v1) + (v2 + v3)) + ((v4 + v5) + (v6 + v7));
}
// workgroup barrier that orders LDS traffic only (global loads stay in flight)
__device__ __forceinline__ void barrier_lds_only() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// native sin/cos of 2*pi*((a*b) mod T)/T (hardware takes the angle in revolutions)
__device__ __forceinline__ void fast_sincos_phase(int64_t a, int64_t b, int T, float* s, float* c) {
  const float x = (float)fa_phase_mod(a, b, T) / (float)T;
  *s = __builtin_amdgcn_sinf(x);
  *c = __builtin_amdgcn_cosf(x);
}

}  // namespace fa_mfma
