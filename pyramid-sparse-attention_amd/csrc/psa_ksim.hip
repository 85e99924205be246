// Key-similarity cap ("sim mask"): per kv-block, the mean cosine similarity of token pairs at
// distance 1, 3 and 7 inside aligned groups of 2, 4 and 8 tokens decides up to which level the
// block's keys may be pooled.
//
// HBM-bound: one pass over K.  A workgroup owns one kv-block; a thread owns 8 consecutive tokens x 8
// channels (16-byte loads, D/8 lanes per row), forms the partial dot products and squared norms of
// its channels, and the D/8 lanes of a token group reduce them with butterflies.
#include "psa_common.h"

namespace {

struct KsimParams {
  const uint16_t* k;  // bf16 or fp16
  int64_t sb, sh, sl;
  int32_t* out;
  int H, L, D, bn, Nk;
  float t2, t4, t8;
};

template <class ET>
__global__ __launch_bounds__(256) void psa_ksim_kernel(KsimParams p) {
  __shared__ float s_part[3][16];
  const int lpr = p.D >> 3;
  const int J = blockIdx.x, bh = blockIdx.y, b = bh / p.H, h = bh % p.H;
  const int g = threadIdx.x / lpr, c = threadIdx.x % lpr;
  const uint16_t* src = p.k + b * p.sb + h * p.sh + c * 8;
  float f[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int64_t row = (int64_t)J * p.bn + g * 8 + i;
    row = row < p.L ? row : (int64_t)(p.L - 1);  // replicate padding
    const u32x4 w = *(const u32x4*)(src + row * p.sl);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[i][2 * j] = ET::from_bits(w[j] & 0xffffu);
      f[i][2 * j + 1] = ET::from_bits(w[j] >> 16);
    }
  }
  // 8 squared norms, dots (0,1) (2,3) (4,5) (6,7) | (0,3) (4,7) | (0,7)
  float v[15];
#pragma unroll
  for (int i = 0; i < 15; ++i) v[i] = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] += f[i][e] * f[i][e];
    v[8] += f[0][e] * f[1][e];
    v[9] += f[2][e] * f[3][e];
    v[10] += f[4][e] * f[5][e];
    v[11] += f[6][e] * f[7][e];
    v[12] += f[0][e] * f[3][e];
    v[13] += f[4][e] * f[7][e];
    v[14] += f[0][e] * f[7][e];
  }
  for (int o = lpr >> 1; o > 0; o >>= 1) {
#pragma unroll
    for (int i = 0; i < 15; ++i) v[i] += __shfl_xor(v[i], o, 64);
  }
  if (c == 0) {
    float n[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) n[i] = sqrtf(v[i] + 1e-12f);
    s_part[0][g] = v[8] / (n[0] * n[1] + 1e-6f) + v[9] / (n[2] * n[3] + 1e-6f) + v[10] / (n[4] * n[5] + 1e-6f) +
                   v[11] / (n[6] * n[7] + 1e-6f);
    s_part[1][g] = v[12] / (n[0] * n[3] + 1e-6f) + v[13] / (n[4] * n[7] + 1e-6f);
    s_part[2][g] = v[14] / (n[0] * n[7] + 1e-6f);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const int ng = p.bn >> 3;
    float s2 = 0.f, s4 = 0.f, s8 = 0.f;
    for (int i = 0; i < ng; ++i) {
      s2 += s_part[0][i];
      s4 += s_part[1][i];
      s8 += s_part[2][i];
    }
    s2 /= (float)(p.bn >> 1);
    s4 /= (float)(p.bn >> 2);
    s8 /= (float)(p.bn >> 3);
    int lv = 1;
    if (s2 > p.t2) lv = 2;
    if (s4 > p.t4) lv = 4;
    if (s8 > p.t8) lv = 8;
    p.out[(int64_t)bh * p.Nk + J] = lv;
  }
}

}  // namespace

extern "C" int psa_ksim(psa_tensor4 k, int32_t* cap_out, int B, int H, int L, int D, int block_n, float thr2, float thr4,
                        float thr8, psa_stream_t stream) {
  PSA_REQUIRE(k.ptr && cap_out, PSA_ERR_ARG, "psa_ksim: null pointer");
  PSA_REQUIRE(B > 0 && H > 0 && L > 0, PSA_ERR_ARG, "psa_ksim: B, H, L must be positive");
  PSA_REQUIRE(D == 64 || D == 128, PSA_ERR_UNSUPPORTED, "psa_ksim: head dim %d not in {64, 128}", D);
  PSA_REQUIRE(block_n == 32 || block_n == 64 || block_n == 128, PSA_ERR_UNSUPPORTED, "psa_ksim: block_n=%d not in {32, 64, 128}", block_n);
  PSA_REQUIRE((int64_t)B * H <= 65535, PSA_ERR_UNSUPPORTED, "psa_ksim: B*H too large");
  PSA_REQUIRE(((uintptr_t)k.ptr % 16 == 0) && k.stride_b % 8 == 0 && k.stride_h % 8 == 0 && k.stride_l % 8 == 0, PSA_ERR_UNSUPPORTED,
              "psa_ksim: K must be 16-byte aligned with strides that are multiples of 8 elements");
  KsimParams p;
  p.k = (const uint16_t*)k.ptr; p.sb = k.stride_b; p.sh = k.stride_h; p.sl = k.stride_l;
  p.out = cap_out; p.H = H; p.L = L; p.D = D; p.bn = block_n; p.Nk = (L + block_n - 1) / block_n;
  p.t2 = thr2; p.t4 = thr4; p.t8 = thr8;
  const bool known = psa_dispatch16(k.dtype, [&](auto et) {
    hipLaunchKernelGGL(psa_ksim_kernel<decltype(et)>, dim3((unsigned)p.Nk, (unsigned)(B * H)), dim3((unsigned)((block_n / 8) * (D / 8))), 0,
                       (hipStream_t)stream, p);
  });
  PSA_REQUIRE(known, PSA_ERR_UNSUPPORTED, "psa_ksim: bf16 or fp16 keys only");
  return psa_check_launch("psa_ksim");
}
