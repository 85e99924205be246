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
typedef _Float16 f16_t;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

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

// ---- the 16-bit element types the MFMA kernels compute in (operands in the caller's type, fp32 accumulation) ------
// bf16: v_mfma_f32_32x32x16_bf16; fp16: v_mfma_f32_32x32x16_f16 - same rate, same operand and accumulator layouts, so
// a kernel is written once over one of these traits.
#define PSA_LDS_PTR(T) __attribute__((address_space(3))) T*
struct EtBf16 {
  static constexpr int id = PSA_DTYPE_BF16;
  using t = bf16_t;
  using x8 = bf16x8;
  static __device__ __forceinline__ float from_bits(uint32_t b16) { return bf16_bits_to_f32(b16); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
  static __device__ __forceinline__ f32x16 mfma(x8 a, x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  // transposing LDS read: 4 keys of one channel
  static __device__ __forceinline__ u32x2 read_tr(PSA_LDS_PTR(unsigned char) a) {
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((PSA_LDS_PTR(bf16x4))a));
  }
  // acc + lo + hi of a packed pair (the rounded values)
  static __device__ __forceinline__ float add_pair(uint32_t packed, float acc) {
    const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed), ones, acc, false);
  }
};
struct EtF16 {
  static constexpr int id = PSA_DTYPE_F16;
  using t = f16_t;
  using x8 = f16x8;
  static __device__ __forceinline__ float from_bits(uint32_t b16) { return (float)__builtin_bit_cast(f16_t, (uint16_t)b16); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));  // round to nearest even
  }
  static __device__ __forceinline__ f32x16 mfma(x8 a, x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ u32x2 read_tr(PSA_LDS_PTR(unsigned char) a) {
    return EtBf16::read_tr(a);  // (the transposing read moves 16-bit words whatever they hold)
  }
  static __device__ __forceinline__ float add_pair(uint32_t packed, float acc) {
    const f16x2 ones = {(f16_t)1.0f, (f16_t)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, packed), ones, acc, false);
  }
};
// calls f(trait) for a 16-bit dtype id; false for any other id
template <class F>
static inline bool psa_dispatch16(int dtype, F&& f) {
  if (dtype == PSA_DTYPE_BF16) {
    f(EtBf16{});
    return true;
  }
  if (dtype == PSA_DTYPE_F16) {
    f(EtF16{});
    return true;
  }
  return false;
}

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
