// Pyramid pooling of K and V: one pass over the inputs writes the 2x, 4x and 8x mean-pooled levels.
//
// HBM-bound.  Every thread owns 8 consecutive tokens x 8 channels (one 16-byte load per token), so a
// group of D/8 neighbouring lanes reads whole rows; the three levels are reduced in registers and each
// level is rounded to bf16 before it feeds the next (the reference materialises every level in bf16).
// Rows past L replicate row L-1 (replicate padding to a multiple of block_n).
//
// Indexed form (token re-ordering fused into the pass): position i of the sequence that is pooled is source row
// index[i]; the re-ordered rows themselves are written out as well (the level-1 keys / values of the attention
// kernel), so no separate gather pass over K and V is needed.
#include "psa_common.h"

struct PoolParams {
  const bf16_t* src[2];
  int64_t sb[2], sh[2], sl[2];
  bf16_t* dst[2];
  int H, L, D;
  int64_t npad;
  const int32_t* index;  // indexed form: source row of every position, else null
  bf16_t* ord[2];        // indexed form: the re-ordered rows [B, H, L, D] (strides ob / oh / ol)
  int64_t ob[2], oh[2], ol[2];
};

__device__ __forceinline__ void unpack8(const u32x4& w, float* f) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = bf16_bits_to_f32(w[j] & 0xffffu);
    f[2 * j + 1] = __builtin_bit_cast(float, w[j] & 0xffff0000u);
  }
}

// mean of two rows -> bf16-rounded, returned both packed and as floats for the next level
__device__ __forceinline__ u32x4 mean2(const float* a, const float* b, float* out) {
  u32x4 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float lo = (a[2 * j] + b[2 * j]) * 0.5f;
    float hi = (a[2 * j + 1] + b[2 * j + 1]) * 0.5f;
    uint32_t p = pack_bf16x2(lo, hi);
    r[j] = p;
    out[2 * j] = bf16_bits_to_f32(p & 0xffffu);
    out[2 * j + 1] = __builtin_bit_cast(float, p & 0xffff0000u);
  }
  return r;
}

template <bool INDEXED>
__global__ __launch_bounds__(256) void psa_pool_kernel(PoolParams p) {
  const int which = blockIdx.z;
  const int bh = blockIdx.y;
  const int b = bh / p.H, h = bh % p.H;
  const int chunks = p.D >> 3;
  const int64_t unit = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t g = unit / chunks;  // group of 8 tokens
  const int c = (int)(unit % chunks);
  const int64_t n8 = p.npad >> 3;
  if (g >= n8) return;

  const bf16_t* src = p.src[which] + b * p.sb[which] + h * p.sh[which] + c * 8;
  const int64_t sl = p.sl[which];
  float f[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int64_t row = g * 8 + i;
    const bool real = row < p.L;
    row = real ? row : (int64_t)(p.L - 1);
    const int64_t srow = INDEXED ? (int64_t)clamp_row(p.index[row], p.L) : row;
    u32x4 w = *(const u32x4*)(src + srow * sl);
    if (INDEXED && real)
      __builtin_nontemporal_store(w, (u32x4*)(p.ord[which] + b * p.ob[which] + h * p.oh[which] + row * p.ol[which] + c * 8));
    unpack8(w, f[i]);
  }
  float l2[4][8], l4[2][8], l8[8];
  u32x4 o2[4], o4[2], o8;
#pragma unroll
  for (int i = 0; i < 4; ++i) o2[i] = mean2(f[2 * i], f[2 * i + 1], l2[i]);
#pragma unroll
  for (int i = 0; i < 2; ++i) o4[i] = mean2(l2[2 * i], l2[2 * i + 1], l4[i]);
  o8 = mean2(l4[0], l4[1], l8);

  // pooled buffer: [level 2 | level 4 | level 8], each [B*H, npad/l, D] contiguous
  const int64_t D = p.D;
  const int64_t BH = (int64_t)gridDim.y;
  bf16_t* d2 = p.dst[which];
  bf16_t* d4 = d2 + BH * (p.npad >> 1) * D;
  bf16_t* d8 = d4 + BH * (p.npad >> 2) * D;
#pragma unroll
  // streaming stores: the pooled rows are not read again by this kernel and would only push the inputs of the
  // next rows out of the caches (measured at the Wan2.1 shape: 70 -> 55 us)
  for (int i = 0; i < 4; ++i) __builtin_nontemporal_store(o2[i], (u32x4*)(d2 + ((int64_t)bh * (p.npad >> 1) + g * 4 + i) * D + c * 8));
#pragma unroll
  for (int i = 0; i < 2; ++i) __builtin_nontemporal_store(o4[i], (u32x4*)(d4 + ((int64_t)bh * (p.npad >> 2) + g * 2 + i) * D + c * 8));
  __builtin_nontemporal_store(o8, (u32x4*)(d8 + ((int64_t)bh * (p.npad >> 3) + g) * D + c * 8));
}

static int pool_run(psa_tensor4 k, psa_tensor4 v, const int32_t* index, const psa_tensor4* k_ord, const psa_tensor4* v_ord,
                    void* k_pool, void* v_pool, int B, int Hkv, int L, int D, int block_n, psa_stream_t stream) {
  PSA_REQUIRE(k.ptr && v.ptr && k_pool && v_pool, PSA_ERR_ARG, "psa_pool_kv: null pointer");
  PSA_REQUIRE(B > 0 && Hkv > 0 && L > 0, PSA_ERR_ARG, "psa_pool_kv: B, Hkv, L must be positive");
  PSA_REQUIRE(D > 0 && D % 8 == 0 && D <= 256, PSA_ERR_UNSUPPORTED, "psa_pool_kv: D=%d must be a multiple of 8, <= 256", D);
  PSA_REQUIRE(block_n >= 8 && block_n % 8 == 0, PSA_ERR_UNSUPPORTED, "psa_pool_kv: block_n=%d must be a multiple of 8", block_n);
  PSA_REQUIRE((int64_t)B * Hkv <= 65535, PSA_ERR_UNSUPPORTED, "psa_pool_kv: B*Hkv too large");
  PSA_REQUIRE(k.stride_l % 8 == 0 && v.stride_l % 8 == 0 && k.stride_h % 8 == 0 && v.stride_h % 8 == 0 &&
                  k.stride_b % 8 == 0 && v.stride_b % 8 == 0 && ((uintptr_t)k.ptr % 16 == 0) && ((uintptr_t)v.ptr % 16 == 0),
              PSA_ERR_UNSUPPORTED, "psa_pool_kv: inputs must be 16-byte aligned with strides that are multiples of 8");
  PoolParams p;
  p.src[0] = (const bf16_t*)k.ptr;
  p.src[1] = (const bf16_t*)v.ptr;
  p.sb[0] = k.stride_b; p.sh[0] = k.stride_h; p.sl[0] = k.stride_l;
  p.sb[1] = v.stride_b; p.sh[1] = v.stride_h; p.sl[1] = v.stride_l;
  p.dst[0] = (bf16_t*)k_pool;
  p.dst[1] = (bf16_t*)v_pool;
  p.H = Hkv; p.L = L; p.D = D;
  p.npad = (int64_t)((L + block_n - 1) / block_n) * block_n;
  p.index = index;
  p.ord[0] = p.ord[1] = nullptr;
  p.ob[0] = p.ob[1] = p.oh[0] = p.oh[1] = p.ol[0] = p.ol[1] = 0;
  if (index != nullptr) {
    const psa_tensor4* o[2] = {k_ord, v_ord};
    for (int t = 0; t < 2; ++t) {
      PSA_REQUIRE(o[t] && o[t]->ptr && ((uintptr_t)o[t]->ptr % 16 == 0) && o[t]->stride_l % 8 == 0 && o[t]->stride_h % 8 == 0 &&
                      o[t]->stride_b % 8 == 0,
                  PSA_ERR_ARG, "psa_pool_kv_indexed: the re-ordered outputs must be 16-byte aligned with strides that are multiples of 8");
      p.ord[t] = (bf16_t*)o[t]->ptr;
      p.ob[t] = o[t]->stride_b; p.oh[t] = o[t]->stride_h; p.ol[t] = o[t]->stride_l;
    }
  }
  int64_t units = (p.npad / 8) * (D / 8);
  dim3 grid((unsigned)((units + 255) / 256), (unsigned)(B * Hkv), 2);
  if (index != nullptr)
    hipLaunchKernelGGL(psa_pool_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, p);
  else
    hipLaunchKernelGGL(psa_pool_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, p);
  return psa_check_launch("psa_pool_kv");
}

extern "C" int psa_pool_kv(psa_tensor4 k, psa_tensor4 v, void* k_pool, void* v_pool, int B, int Hkv, int L, int D,
                           int block_n, psa_stream_t stream) {
  return pool_run(k, v, nullptr, nullptr, nullptr, k_pool, v_pool, B, Hkv, L, D, block_n, stream);
}

extern "C" int psa_pool_kv_indexed(psa_tensor4 k, psa_tensor4 v, const int32_t* index, psa_tensor4 k_ord, psa_tensor4 v_ord,
                                   void* k_pool, void* v_pool, int B, int Hkv, int L, int D, int block_n, psa_stream_t stream) {
  PSA_REQUIRE(index != nullptr, PSA_ERR_ARG, "psa_pool_kv_indexed: null index");
  return pool_run(k, v, index, &k_ord, &v_ord, k_pool, v_pool, B, Hkv, L, D, block_n, stream);
}
