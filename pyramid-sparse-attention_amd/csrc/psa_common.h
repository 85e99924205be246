// Shared device/host helpers for the PSA kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/psa_hip.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define PSA_WAVE 64

// ---- host side: error reporting -------------------------------------------------------
void psa_set_error(const char* fmt, ...);
int psa_check_launch(const char* what);

#define PSA_REQUIRE(cond, code, ...) \
  do {                               \
    if (!(cond)) {                   \
      psa_set_error(__VA_ARGS__);    \
      return (code);                 \
    }                                \
  } while (0)

static inline int psa_ilog2(int x) {
  int r = 0;
  while ((1 << r) < x) ++r;
  return r;
}
static inline bool psa_is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

// ---- device side ----------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b16) { return __builtin_bit_cast(float, b16 << 16); }

// round-to-nearest-even fp32 -> bf16 bits (no NaN special-casing beyond keeping it a NaN)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  bf16_t h = (bf16_t)f;
  return (uint32_t) __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2 v = {lo, hi};
  bf16x2 h = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// max of three: compiles to one v_max3_f32 in translation units built without NaN semantics (the compiler then
// needs no canonicalising pass over its inputs).  Plain C on purpose: hand-written assembly would not get the
// wait states that reading a fresh MFMA result requires.
__device__ __forceinline__ float max3f(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

// Exchange between the two 32-lane halves of a wave (v_permlane32_swap: no LDS round trip).
// After the swap r[0] holds lanes 0-31 of v in both halves and r[1] holds lanes 32-63 in both halves.
__device__ __forceinline__ void half_wave_swap(float v, float& lo, float& hi) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const uint32_t r0 = r[0], r1 = r[1];  // element-wise extraction first: a bit_cast of r[i] itself reads element 0
  lo = __builtin_bit_cast(float, r0);
  hi = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float half_wave_max(float v) {
  float lo, hi;
  half_wave_swap(v, lo, hi);
  return fmaxf(lo, hi);
}
// Maxima over both half-waves of a and of b with one exchange: lanes 0-31 return it for a, lanes 32-63 for b.
__device__ __forceinline__ float half_wave_max_pair(float a, float b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b), false, false);
  const uint32_t r0 = r[0], r1 = r[1];  // r0 = (a low half, b low half), r1 = (a high half, b high half)
  return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}
__device__ __forceinline__ float half_wave_sum(float v) {
  float lo, hi;
  half_wave_swap(v, lo, hi);
  return lo + hi;
}

// Row of a token index (token re-ordering), never out of bounds: a value outside 0 .. L-1 - the caller's mistake, the
// Python mirror rejects such an index - reads row 0 / L-1 instead of faulting.
__device__ __forceinline__ int clamp_row(int v, int L) { return v < 0 ? 0 : (v < L ? v : L - 1); }

// level value (0,1,2,4,8) of a map element of 1 or 4 bytes
__device__ __forceinline__ int load_map(const void* map, int64_t idx, int elem_bytes) {
  return elem_bytes == 1 ? (int)((const int8_t*)map)[idx] : ((const int32_t*)map)[idx];
}
__device__ __forceinline__ void store_map(void* map, int64_t idx, int elem_bytes, int v) {
  if (elem_bytes == 1)
    ((int8_t*)map)[idx] = (int8_t)v;
  else
    ((int32_t*)map)[idx] = v;
}
