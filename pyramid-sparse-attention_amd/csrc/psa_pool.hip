// Pyramid pooling of K and V: one pass over the inputs writes the 2x, 4x and 8x mean-pooled levels.
//
// HBM-bound.  Every thread owns 8 consecutive tokens x 16 bytes of channels (one 16-byte load per token: 8 channels
// of bf16 / fp16, 4 of fp32), so a group of neighbouring lanes reads whole rows; the three levels are reduced in
// registers and each level is rounded to the tensors' element type before it feeds the next (the reference
// materialises every level in that type).
// Rows past L replicate row L-1 (replicate padding to a multiple of block_n).
//
// Indexed form (token re-ordering fused into the pass): position i of the sequence that is pooled is source row
// index[i]; the re-ordered rows themselves are written out as well (the level-1 keys / values of the attention
// kernel), so no separate gather pass over K and V is needed.
#include "psa_common.h"

struct PoolParams {
  const char* src[2];    // element pointers as bytes; strides below are in elements
  int64_t sb[2], sh[2], sl[2];
  char* dst[2];
  int H, L, D;
  int64_t npad;
  const int32_t* index;  // indexed form: source row of every position, else null
  char* ord[2];          // indexed form: the re-ordered rows [B, H, L, D] (strides ob / oh / ol)
  int64_t ob[2], oh[2], ol[2];
};

// a 16-byte chunk of a row as floats, and back (rounded to the element type, nearest even)
struct PoolF32 {
  static constexpr int CH = 4, ES = 4;
  typedef float f32x4_t __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ void unpack(const u32x4& w, float* f) {
    const f32x4_t x = __builtin_bit_cast(f32x4_t, w);  // (the whole vector at once: a bit cast of one element of a vector is not addressable)
    f[0] = x.x; f[1] = x.y; f[2] = x.z; f[3] = x.w;
  }
  static __device__ __forceinline__ u32x4 pack(float* f) {  // (fp32: nothing to round)
    f32x4_t x;
    x.x = f[0]; x.y = f[1]; x.z = f[2]; x.w = f[3];
    return __builtin_bit_cast(u32x4, x);
  }
};
template <class ET>
struct Pool16 {
  static constexpr int CH = 8, ES = 2;
  static __device__ __forceinline__ void unpack(const u32x4& w, float* f) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = ET::from_bits(w[j] & 0xffffu);
      f[2 * j + 1] = ET::from_bits(w[j] >> 16);
    }
  }
  static __device__ __forceinline__ u32x4 pack(float* f) {  // rounds f in place
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      r[j] = ET::pack2(f[2 * j], f[2 * j + 1]);
      f[2 * j] = ET::from_bits(r[j] & 0xffffu);
      f[2 * j + 1] = ET::from_bits(r[j] >> 16);
    }
    return r;
  }
};

// mean of two rows, rounded to the element type: returned both packed and as floats for the next level
template <class PT>
__device__ __forceinline__ u32x4 mean2(const float* a, const float* b, float* out) {
#pragma unroll
  for (int j = 0; j < PT::CH; ++j) out[j] = (a[j] + b[j]) * 0.5f;
  return PT::pack(out);
}

template <bool INDEXED, class PT>
__global__ __launch_bounds__(256) void psa_pool_kernel(PoolParams p) {
  constexpr int CH = PT::CH, ES = PT::ES;
  const int which = blockIdx.z;
  const int bh = blockIdx.y;
  const int b = bh / p.H, h = bh % p.H;
  const int chunks = p.D / CH;
  const int64_t unit = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t g = unit / chunks;  // group of 8 tokens
  const int c = (int)(unit % chunks);
  const int64_t n8 = p.npad >> 3;
  if (g >= n8) return;

  const char* src = p.src[which] + (b * p.sb[which] + h * p.sh[which] + c * CH) * ES;
  const int64_t sl = p.sl[which] * ES;
  float f[8][CH];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int64_t row = g * 8 + i;
    const bool real = row < p.L;
    row = real ? row : (int64_t)(p.L - 1);
    const int64_t srow = INDEXED ? (int64_t)clamp_row(p.index[row], p.L) : row;
    u32x4 w = *(const u32x4*)(src + srow * sl);
    if (INDEXED && real)
      __builtin_nontemporal_store(w, (u32x4*)(p.ord[which] + (b * p.ob[which] + h * p.oh[which] + row * p.ol[which] + c * CH) * ES));
    PT::unpack(w, f[i]);
  }
  float l2[4][CH], l4[2][CH], l8[CH];
  u32x4 o2[4], o4[2], o8;
#pragma unroll
  for (int i = 0; i < 4; ++i) o2[i] = mean2<PT>(f[2 * i], f[2 * i + 1], l2[i]);
#pragma unroll
  for (int i = 0; i < 2; ++i) o4[i] = mean2<PT>(l2[2 * i], l2[2 * i + 1], l4[i]);
  o8 = mean2<PT>(l4[0], l4[1], l8);

  // pooled buffer: [level 2 | level 4 | level 8], each [B*H, npad/l, D] contiguous
  const int64_t D = (int64_t)p.D * ES;  // bytes per row
  const int64_t BH = (int64_t)gridDim.y;
  char* d2 = p.dst[which];
  char* d4 = d2 + BH * (p.npad >> 1) * D;
  char* d8 = d4 + BH * (p.npad >> 2) * D;
#pragma unroll
  // streaming stores: the pooled rows are not read again by this kernel and would only push the inputs of the
  // next rows out of the caches (measured at the Wan2.1 shape: 70 -> 55 us)
  for (int i = 0; i < 4; ++i) __builtin_nontemporal_store(o2[i], (u32x4*)(d2 + ((int64_t)bh * (p.npad >> 1) + g * 4 + i) * D + c * 16));
#pragma unroll
  for (int i = 0; i < 2; ++i) __builtin_nontemporal_store(o4[i], (u32x4*)(d4 + ((int64_t)bh * (p.npad >> 2) + g * 2 + i) * D + c * 16));
  __builtin_nontemporal_store(o8, (u32x4*)(d8 + ((int64_t)bh * (p.npad >> 3) + g) * D + c * 16));
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
  PSA_REQUIRE(k.dtype == v.dtype && (k.dtype == PSA_DTYPE_BF16 || k.dtype == PSA_DTYPE_F16 || k.dtype == PSA_DTYPE_F32), PSA_ERR_ARG,
              "psa_pool_kv: K and V must share one element type (bf16, fp16 or fp32)");
  PoolParams p;
  p.src[0] = (const char*)k.ptr;
  p.src[1] = (const char*)v.ptr;
  p.sb[0] = k.stride_b; p.sh[0] = k.stride_h; p.sl[0] = k.stride_l;
  p.sb[1] = v.stride_b; p.sh[1] = v.stride_h; p.sl[1] = v.stride_l;
  p.dst[0] = (char*)k_pool;
  p.dst[1] = (char*)v_pool;
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
      PSA_REQUIRE(o[t]->dtype == k.dtype, PSA_ERR_ARG, "psa_pool_kv_indexed: the re-ordered outputs must have the inputs' element type");
      p.ord[t] = (char*)o[t]->ptr;
      p.ob[t] = o[t]->stride_b; p.oh[t] = o[t]->stride_h; p.ol[t] = o[t]->stride_l;
    }
  }
  auto launch = [&](auto pt) {
    using PT = decltype(pt);
    const int64_t units = (p.npad / 8) * (D / PT::CH);
    dim3 grid((unsigned)((units + 255) / 256), (unsigned)(B * Hkv), 2);
    if (index != nullptr)
      hipLaunchKernelGGL((psa_pool_kernel<true, PT>), grid, dim3(256), 0, (hipStream_t)stream, p);
    else
      hipLaunchKernelGGL((psa_pool_kernel<false, PT>), grid, dim3(256), 0, (hipStream_t)stream, p);
  };
  if (k.dtype == PSA_DTYPE_F32) launch(PoolF32{});
  else if (k.dtype == PSA_DTYPE_F16) launch(Pool16<EtF16>{});
  else launch(Pool16<EtBf16>{});
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
