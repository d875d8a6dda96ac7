// Shared host/device helpers for the gfx950 Fourier-attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/fourier_attn_hip.h"

#define FA_WAVE 64

// ---- error reporting --------------------------------------------------------
void fa_set_error(const char* fmt, ...);
int fa_check_launch(const char* what);

#define FA_REQUIRE(cond, code, ...)      \
  do {                                   \
    if (!(cond)) {                       \
      fa_set_error(__VA_ARGS__);         \
      return (code);                     \
    }                                    \
  } while (0)

// matrix-core spectral compression (fa_spectral_mfma.hip)
bool fa_spectral_mfma_ok(int a_dtype, int K, int Mc, int N);
bool fa_recon_stats_mfma_ok(int N, int Mc, int K);
size_t fa_recon_stats_mfma_workspace(int B, int N, int Mc, int K);
// partial sums / maxima / minima of the reconstruction, [B][row blocks][Mc] each; returns the number of row blocks
int fa_recon_stats_mfma_launch(const float* c, int B, int N, int Mc, int K, int T, void* workspace, float** psum,
                               float** pmax, float** pmin, hipStream_t st);
// the last launch of the column statistics (fa_spectral.hip): partials [B][nsplit][Mc] -> mean and maximum deviation
void fa_stats_finalize_launch(const float* psum, const float* pmax, const float* pmin, float* avg, float* dev, int B, int K,
                              int Mc, int nsplit, int round_dtype, hipStream_t st);
size_t fa_spectral_mfma_workspace(int B, int K, int Mc, int N);
int fa_spectral_mfma_launch(const void* a, int a_dtype, int64_t a_bs, int64_t a_rs, const int32_t* cols, float* c, int B,
                            int K, int Mc, int N, int T, int64_t k_start, int accumulate, void* workspace,
                            hipStream_t st);

static inline hipStream_t fa_hip_stream(fa_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
static inline int fa_cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }
static inline size_t fa_align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---- element types ----------------------------------------------------------
struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

__device__ __forceinline__ float fa_to_float(bf16_t x) { return __uint_as_float(((uint32_t)x.bits) << 16); }
__device__ __forceinline__ float fa_to_float(f16_t x) { return (float)x.v; }
__device__ __forceinline__ float fa_to_float(float x) { return x; }

// round-to-nearest-even float -> bf16 bits (NaN kept quiet)
__device__ __forceinline__ uint16_t fa_f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float fa_round_through(float v, int dtype) {
  if (dtype == FA_BF16) return __uint_as_float(((uint32_t)fa_f32_to_bf16_bits(v)) << 16);
  if (dtype == FA_FP16) return (float)(_Float16)v;
  return v;
}

// ---- exact Fourier phases ---------------------------------------------------
// cos/sin of 2*pi*((a*b) mod T)/T; the product is reduced in integers so the
// angle handed to the float unit is always inside one period.
// (a*b) mod T for non-negative a, b: the 64-bit division is a long software routine, so products that fit
// 32 bits (all but very long contexts) take the short one
__device__ __forceinline__ uint32_t fa_phase_mod(int64_t a, int64_t b, int T) {
  const uint64_t prod = (uint64_t)a * (uint64_t)b;
  if ((prod >> 32) == 0) return (uint32_t)prod % (uint32_t)T;
  return (uint32_t)(prod % (uint64_t)T);
}
__device__ __forceinline__ void fa_sincos_phase(int64_t a, int64_t b, int T, float* s, float* c) {
  const uint32_t r = fa_phase_mod(a, b, T);
  float x = 2.0f * (float)r / (float)T;  // in [0, 2)
  sincospif(x, s, c);
}

// ---- wave / block reductions ------------------------------------------------
__device__ __forceinline__ float fa_wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, FA_WAVE);
  return v;
}
__device__ __forceinline__ float fa_wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, FA_WAVE));
  return v;
}
__device__ __forceinline__ float fa_wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, FA_WAVE));
  return v;
}

// ---- cross-lane helpers without LDS traffic -----------------------------------
template <int CTRL>
__device__ __forceinline__ float fa_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// butterfly partners inside a 16-lane row: xor 1, xor 2, (7 - i within 8 lanes), (15 - i), rotate by 8
#define FA_DPP_XOR1 0xB1
#define FA_DPP_XOR2 0x4E
#define FA_DPP_HALF_MIRROR 0x141
#define FA_DPP_MIRROR 0x140
#define FA_DPP_ROR8 0x128

// sum over the LANES consecutive lanes (4, 8 or 16, aligned) that contain this lane; every lane gets it
template <int LANES>
__device__ __forceinline__ float fa_group_sum(float v) {
  v += fa_dpp<FA_DPP_XOR1>(v);
  v += fa_dpp<FA_DPP_XOR2>(v);
  if (LANES >= 8) v += fa_dpp<FA_DPP_HALF_MIRROR>(v);
  if (LANES >= 16) v += fa_dpp<FA_DPP_MIRROR>(v);
  return v;
}

// partner values across the four 16-lane rows of a wave (lane i, i+16, i+32, i+48):
// one v_permlane16_swap / v_permlane32_swap each (gfx950); the two operands must sit in
// different registers, which the empty asm enforces
__device__ __forceinline__ void fa_swap16(float x, float* lo, float* hi) {
  unsigned a = __builtin_bit_cast(unsigned, x), b = a;
  asm volatile("" : "+v"(b));
  auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
  const unsigned r0 = r[0], r1 = r[1];  // scalars first: bit_cast of a vector element reads element 0
  *lo = __builtin_bit_cast(float, r0);
  *hi = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ void fa_swap32(float x, float* lo, float* hi) {
  unsigned a = __builtin_bit_cast(unsigned, x), b = a;
  asm volatile("" : "+v"(b));
  auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  const unsigned r0 = r[0], r1 = r[1];  // scalars first: bit_cast of a vector element reads element 0
  *lo = __builtin_bit_cast(float, r0);
  *hi = __builtin_bit_cast(float, r1);
}
// Maximum / minimum that hand a NaN on (v_maximum3_f32 / v_minimum3_f32 of gfx950, three operands per instruction).
// fmaxf / fminf must drop a NaN, for which the compiler first passes every operand that comes out of a matrix
// instruction or a lane exchange through an instruction of its own: three instructions per maximum instead of one.
__device__ __forceinline__ float fa_fmax(float a, float b) { return __builtin_elementwise_maximum(a, b); }
__device__ __forceinline__ float fa_fmin(float a, float b) { return __builtin_elementwise_minimum(a, b); }
__device__ __forceinline__ float fa_fmax8(const float (&v)[8]) {
  return fa_fmax(fa_fmax(fa_fmax(fa_fmax(fa_fmax(fa_fmax(fa_fmax(v[0], v[1]), v[2]), v[3]), v[4]), v[5]), v[6]), v[7]);
}
// max / sum over the four lanes that share (lane % 16); every lane gets the result
__device__ __forceinline__ float fa_rows_max(float x) {
  float a, b;
  fa_swap16(x, &a, &b);
  x = fa_fmax(a, b);
  fa_swap32(x, &a, &b);
  return fa_fmax(a, b);
}
__device__ __forceinline__ float fa_rows_min(float x) {
  float a, b;
  fa_swap16(x, &a, &b);
  x = fa_fmin(a, b);
  fa_swap32(x, &a, &b);
  return fa_fmin(a, b);
}
__device__ __forceinline__ float fa_rows_sum(float x) {
  float a, b;
  fa_swap16(x, &a, &b);
  x = a + b;
  fa_swap32(x, &a, &b);
  return a + b;
}
