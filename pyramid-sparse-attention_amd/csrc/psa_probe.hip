// Diagnostic: the bf16 MFMA rate and the core clock the chip sustains under a pure, register-only MFMA load.
//
// The published 2.5 PFLOP/s bf16 peak assumes the boost clock; under a dense MFMA stream the chip lowers its clock
// (power management), and how far depends on how much the operands toggle.  bench.py runs this next to the
// attention kernels so that their MFMA utilisation can be read against what the same chip sustains at that moment.
// Every wave keeps 4 A and 4 B operands in registers and issues iters * 4 independent 32x32x16 MFMAs on 4
// accumulators; nothing touches LDS or memory inside the loop (modes 0 and 1), or every MFMA takes its A operand from
// LDS (mode 2).
#include "psa_common.h"

namespace {

__global__ __launch_bounds__(256) void psa_probe_mfma_kernel(int iters, int random_operands, float* sink, long long* clocks) {
  bf16x8 a[4], b[4];
  uint32_t r = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // random: values in (-1/64, 1/64) from a linear congruential sequence; constant: one value everywhere
      r = r * 1664525u + 1013904223u;
      a[j][i] = (bf16_t)(random_operands ? ((int)(r >> 8) % 2001 - 1000) * (1.0f / 64000.f) : 0.0078125f);
      r = r * 1664525u + 1013904223u;
      b[j][i] = (bf16_t)(random_operands ? ((int)(r >> 8) % 2001 - 1000) * (1.0f / 64000.f) : 0.0078125f);
    }
  f32x16 c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) c[j][i] = 0.f;
  // mode 2: the A operand of every MFMA is read from LDS (one 128-bit read per MFMA, the ratio of the attention
  // kernels), 16 KiB of pseudo-random bf16 per wave slot, conflict-free addresses
  __shared__ __align__(16) unsigned char lds[4 * 16 * 1024];
  if (random_operands == 2) {
    uint32_t* w = (uint32_t*)lds;
    for (int i = threadIdx.x; i < (int)sizeof(lds) / 4; i += 256) {
      r = r * 1664525u + 1013904223u;
      const uint32_t lo = __builtin_bit_cast(uint16_t, (bf16_t)(((int)(r >> 8) % 2001 - 1000) * (1.0f / 64000.f)));
      r = r * 1664525u + 1013904223u;
      const uint32_t hi = __builtin_bit_cast(uint16_t, (bf16_t)(((int)(r >> 8) % 2001 - 1000) * (1.0f / 64000.f)));
      w[i] = lo | (hi << 16);
    }
    __syncthreads();
  }
  const unsigned char* my = lds + (threadIdx.x >> 6) * 16 * 1024 + (threadIdx.x & 63) * 16;
  const long long w0 = wall_clock64(), c0 = clock64();
  if (random_operands == 2) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        bf16x8 al[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) al[j] = *(const bf16x8*)(my + (((it + u) & 3) * 4 + j) * 1024);  // varies with `it`: stays in the loop
#pragma unroll
        for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[j], b[(j + u) & 3], c[j], 0, 0, 0);
      }
    }
  } else {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], b[(j + u) & 3], c[j], 0, 0, 0);
    }
  }
  const long long w1 = wall_clock64(), c1 = clock64();
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += c[j][i];
  if (s == 1.2345f) sink[threadIdx.x] = s;  // keeps the loop alive; never true for these operands in practice
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = w1 - w0;  // constant 100 MHz counter
    clocks[1] = c1 - c0;  // core clock counter
  }
}

}  // namespace

extern "C" int psa_probe_mfma(int workgroups, int iters, int random_operands, float* sink, int64_t* clocks, double* flops,
                              psa_stream_t stream) {
  PSA_REQUIRE(workgroups > 0 && iters > 0 && sink && clocks, PSA_ERR_ARG, "psa_probe_mfma: bad arguments");
  hipLaunchKernelGGL(psa_probe_mfma_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, iters, random_operands, sink,
                     (long long*)clocks);
  if (flops) *flops = (double)workgroups * 4.0 * iters * 16.0 * (2.0 * 32 * 32 * 16);  // 4 waves x 16 MFMAs per iteration
  return psa_check_launch("psa_probe_mfma");
}
