// Pyramid sparse attention forward on fp32 tensors: fp32 operands, fp32 arithmetic throughout (vector FMAs; the matrix
// cores' fp32 rate is no higher at these shapes, and this path exists for the small fp32 layers the reference accepts -
// its Triton kernels compute in the tensors' type).  Same walk as the 16-bit kernels (psa_tiles.h: the map row is
// compacted into tiles of 64 pooled keys of one level), same softmax (base 2, +log2(level) bias, online), same masks.
//
// One workgroup of 256 threads per QR = 16 RI query rows, RI = 4, 2 or 1 (the largest that still gives the launch two
// workgroups per CU: the small layers this path serves would otherwise leave most of the chip idle; a 128-row q-block
// takes 128 / QR workgroups).  Per tile: the K tile goes
// to LDS transposed (channel-major, so that the 16 threads that share a query row read consecutive keys), the V tile
// row-major; thread (ty, tx) = (t / 16, t % 16) owns the logits of rows ty + 16 i and keys tx + 16 j (RI x 4), reduces
// row maxima and sums over its 16-lane row group with shuffles, leaves the probabilities in LDS, and accumulates the
// output channels tx + 16 c of its rows.  LDS-bound (two LDS operands per 16 FMAs); about 10 % of the fp32 vector peak.
#include "psa_common.h"
#include "psa_tiles.h"

namespace {

constexpr int TK32 = 64;

struct F32Params {
  const float *q, *k, *v, *kp, *vp;
  float* o;
  float* lse;
  const void* map;
  int map_elem;
  int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, o_sb, o_sh, o_sl;
  int B, Hq, Hkv, L, Mq, Nk, bn_log2, bm, halves;
  int64_t npad;
  float scale_log2;
  int causal, max_tiles;
  const int32_t* q_index;
};

template <int D, int RI>
__global__ __launch_bounds__(256) void psa_fwd_f32_kernel(F32Params p) {
  constexpr int QR = 16 * RI;  // query rows per workgroup
  constexpr int DP = D + 1, KP = TK32 + 1, CPT = D / 16;  // padded strides; output channels per thread
  extern __shared__ __align__(16) unsigned char smem[];
  float* Qs = (float*)smem;         // [QR][DP]
  float* Kt = Qs + QR * DP;         // [D][KP]: K tile, channel-major
  float* Vs = Kt + D * KP;          // [TK32][D]
  float* Ps = Vs + TK32 * D;        // [QR][KP]
  int* s_src = (int*)(Ps + QR * KP);  // [TK32]: source row of every tile slot, -1 = empty
  u32x2* tdesc = (u32x2*)(s_src + TK32);
  uint16_t* ids = (uint16_t*)(tdesc + p.max_tiles);
  __shared__ int s_cnt[4], s_ioff[4], s_toff[5], s_wcnt[16];

  const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
  const int unit = blockIdx.x;  // (b, h, q-block, half)
  const int half = unit % p.halves, logical = unit / p.halves;
  const int I = logical % p.Mq, bh = logical / p.Mq, h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);
  const int q0 = I * p.bm + half * QR;  // first query position of this workgroup
  int jmax = p.Nk;
  if (p.causal) {
    const int ce = (int)((((int64_t)(I + 1) * p.bm) + (1 << p.bn_log2) - 1) >> p.bn_log2);
    jmax = ce < jmax ? ce : jmax;
  }
  // Q rows (rows past the sequence replicate the last one; their results are not stored)
  for (int u = tid; u < QR * (D / 4); u += 256) {
    const int r = u / (D / 4), c4 = u % (D / 4);
    int qr = q0 + r < p.L ? q0 + r : p.L - 1;
    if (p.q_index != nullptr) qr = clamp_row(p.q_index[qr], p.L);
    const f32x4 x = *(const f32x4*)(p.q + b * p.q_sb + h * p.q_sh + (int64_t)qr * p.q_sl + c4 * 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) Qs[r * DP + c4 * 4 + e] = x[e];
  }
  const int T = psa_tiles::build_row_schedule<256>(p.map, p.map_elem, ((int64_t)bh * p.Mq + I) * p.Nk, p.Nk, jmax, p.bn_log2, p.L,
                                                  p.causal != 0, (int64_t)I * p.bm, ids, tdesc, s_cnt, s_ioff, s_toff, s_wcnt);
  const float* kb0 = p.k + b * p.k_sb + hk * p.k_sh;
  const float* vb0 = p.v + b * p.v_sb + hk * p.v_sh;
  const int64_t BHkv = (int64_t)p.B * p.Hkv, bhk = (int64_t)b * p.Hkv + hk;

  float acc[RI][CPT];
  float m_run[RI], l_run[RI];
#pragma unroll
  for (int i = 0; i < RI; ++i) {
    m_run[i] = -INFINITY;
    l_run[i] = 0.f;
#pragma unroll
    for (int c = 0; c < CPT; ++c) acc[i][c] = 0.f;
  }
  for (int t = 0; t < T; ++t) {
    const psa_tiles::TileRef tr = psa_tiles::tile_ref(tdesc, ids, t, p.bn_log2);
    const float* kbase = tr.lv == 0 ? kb0 : p.kp + psa_tiles::pool_row_offset(tr.lv, BHkv, bhk, p.npad) * D;
    const float* vbase = tr.lv == 0 ? vb0 : p.vp + psa_tiles::pool_row_offset(tr.lv, BHkv, bhk, p.npad) * D;
    const int64_t kstr = tr.lv == 0 ? p.k_sl : D, vstr = tr.lv == 0 ? p.v_sl : D;
    __syncthreads();  // the previous tile's readers are done
    if (tid < TK32) s_src[tid] = psa_tiles::slot_src(tr.lv, tr.lt, tid, tr.sbs_log2, tr.cnt, tr.ids, p.L);
    __syncthreads();
    for (int u = tid; u < TK32 * (D / 4); u += 256) {
      const int r = u / (D / 4), c4 = u % (D / 4);
      const int src = s_src[r];
      f32x4 xk = {0.f, 0.f, 0.f, 0.f}, xv = {0.f, 0.f, 0.f, 0.f};
      if (src >= 0) {
        xk = *(const f32x4*)(kbase + (int64_t)src * kstr + c4 * 4);
        xv = *(const f32x4*)(vbase + (int64_t)src * vstr + c4 * 4);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) Kt[(c4 * 4 + e) * KP + r] = xk[e];
      *(f32x4*)(Vs + r * D + c4 * 4) = xv;
    }
    __syncthreads();
    // S = Q K^T: rows ty + 16 i, keys tx + 16 j
    float s[RI][4];
#pragma unroll
    for (int i = 0; i < RI; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) s[i][j] = 0.f;
    for (int d = 0; d < D; ++d) {
      float qv[RI], kv[4];
#pragma unroll
      for (int i = 0; i < RI; ++i) qv[i] = Qs[(ty + 16 * i) * DP + d];
#pragma unroll
      for (int j = 0; j < 4; ++j) kv[j] = Kt[d * KP + tx + 16 * j];
#pragma unroll
      for (int i = 0; i < RI; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) s[i][j] = __builtin_fmaf(qv[i], kv[j], s[i][j]);
    }
    // masks: empty slots; causal: a pooled key of level lv is visible to query i once its last token is
    const float bias = (float)tr.lv;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int src = s_src[tx + 16 * j];
#pragma unroll
      for (int i = 0; i < RI; ++i) {
        const int qi = q0 + ty + 16 * i;
        const bool vis = src >= 0 && (!p.causal || (((int64_t)src + 1) << tr.lv) - 1 <= qi);
        s[i][j] = vis ? __builtin_fmaf(s[i][j], p.scale_log2, bias) : -INFINITY;
      }
    }
    // online softmax per row over the 16 lanes of the row group
#pragma unroll
    for (int i = 0; i < RI; ++i) {
      float mx = fmaxf(fmaxf(s[i][0], s[i][1]), fmaxf(s[i][2], s[i][3]));
      for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      const float m_new = fmaxf(m_run[i], mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = fast_exp2(m_run[i] - m_use);
      float sum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float pr = fast_exp2(s[i][j] - m_use);
        sum += pr;
        Ps[(ty + 16 * i) * KP + tx + 16 * j] = pr;
      }
      for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
      l_run[i] = l_run[i] * alpha + sum;
      m_run[i] = m_new;
#pragma unroll
      for (int c = 0; c < CPT; ++c) acc[i][c] *= alpha;
    }
    __syncthreads();
    // O += P V: rows ty + 16 i, channels tx + 16 c
    for (int kk = 0; kk < TK32; ++kk) {
      float pv[RI], vv[CPT];
#pragma unroll
      for (int i = 0; i < RI; ++i) pv[i] = Ps[(ty + 16 * i) * KP + kk];
#pragma unroll
      for (int c = 0; c < CPT; ++c) vv[c] = Vs[kk * D + tx + 16 * c];
#pragma unroll
      for (int i = 0; i < RI; ++i)
#pragma unroll
        for (int c = 0; c < CPT; ++c) acc[i][c] = __builtin_fmaf(pv[i], vv[c], acc[i][c]);
    }
  }
#pragma unroll
  for (int i = 0; i < RI; ++i) {
    const int qi = q0 + ty + 16 * i;
    if (qi >= p.L || qi >= (I + 1) * p.bm) continue;
    const int orow = p.q_index != nullptr ? p.q_index[qi] : qi;
    if ((unsigned)orow >= (unsigned)p.L) continue;
    const float l_safe = fmaxf(l_run[i], 1e-8f);
    const float inv = 1.0f / l_safe;
    float* op = p.o + b * p.o_sb + h * p.o_sh + (int64_t)orow * p.o_sl;
#pragma unroll
    for (int c = 0; c < CPT; ++c) op[tx + 16 * c] = acc[i][c] * inv;
    if (p.lse != nullptr && tx == 0) p.lse[((int64_t)b * p.Hq + h) * p.L + orow] = (m_run[i] + fast_log2(l_safe)) * 0.6931471805599453f;
  }
}

template <int D, int RI>
int launch_f32(const F32Params& p, hipStream_t stream) {
  constexpr int QR = 16 * RI;
  const size_t shmem = (size_t)(QR * (D + 1) + D * (TK32 + 1) + TK32 * D + QR * (TK32 + 1)) * 4 + TK32 * 4 + (size_t)p.max_tiles * 8 +
                       (size_t)p.Nk * 2 + 16;
  if (shmem > 160 * 1024) return PSA_ERR_UNSUPPORTED;
  if (hipFuncSetAttribute((const void*)psa_fwd_f32_kernel<D, RI>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess)
    return PSA_ERR_LAUNCH;
  const int64_t units = (int64_t)p.B * p.Hq * p.Mq * p.halves;
  hipLaunchKernelGGL((psa_fwd_f32_kernel<D, RI>), dim3((unsigned)units), dim3(256), shmem, stream, p);
  return PSA_OK;
}

}  // namespace

int psa_fwd_f32(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool, const void* map, int map_elem_bytes,
                psa_tensor4 out, float* lse, int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, float sm_scale, int causal,
                psa_stream_t stream, const int32_t* q_index) {
  PSA_REQUIRE(q.ptr && k.ptr && v.ptr && out.ptr, PSA_ERR_ARG, "psa_fwd: null pointer");
  PSA_REQUIRE(map == nullptr || (k_pool && v_pool), PSA_ERR_ARG, "psa_fwd: pooled K/V required with a level map");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_fwd: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(Hq % Hkv == 0, PSA_ERR_ARG, "psa_fwd: Hq=%d must be a multiple of Hkv=%d", Hq, Hkv);
  PSA_REQUIRE(sm_scale > 0.f, PSA_ERR_ARG, "psa_fwd: sm_scale must be positive");
  PSA_REQUIRE(D == 64 || D == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: head dim %d not in {64, 128}", D);
  PSA_REQUIRE(block_m == 64 || block_m == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: block_m=%d not in {64, 128}", block_m);
  PSA_REQUIRE(block_n == 32 || block_n == 64 || block_n == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: block_n=%d not in {32, 64, 128}", block_n);
  const psa_tensor4* ts[4] = {&q, &k, &v, &out};
  for (int i = 0; i < 4; ++i)
    PSA_REQUIRE(((uintptr_t)ts[i]->ptr % 16 == 0) && ts[i]->stride_b % 4 == 0 && ts[i]->stride_h % 4 == 0 && ts[i]->stride_l % 4 == 0,
                PSA_ERR_UNSUPPORTED, "psa_fwd: fp32 tensors must be 16-byte aligned with strides that are multiples of 4 elements");
  const int Mq = (L + block_m - 1) / block_m, Nk = (L + block_n - 1) / block_n;
  PSA_REQUIRE(Nk <= 65535, PSA_ERR_UNSUPPORTED, "psa_fwd: more than 65535 kv-blocks");
  PSA_REQUIRE((int64_t)B * Hq * Mq * 8 < (1ll << 31), PSA_ERR_UNSUPPORTED, "psa_fwd: too many workgroups");
  F32Params p;
  p.q = (const float*)q.ptr; p.k = (const float*)k.ptr; p.v = (const float*)v.ptr; p.o = (float*)out.ptr;
  p.kp = (const float*)k_pool; p.vp = (const float*)v_pool;
  p.lse = lse; p.map = map; p.map_elem = map_elem_bytes;
  p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sl = q.stride_l;
  p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sl = k.stride_l;
  p.v_sb = v.stride_b; p.v_sh = v.stride_h; p.v_sl = v.stride_l;
  p.o_sb = out.stride_b; p.o_sh = out.stride_h; p.o_sl = out.stride_l;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.L = L; p.Mq = Mq; p.Nk = Nk;
  // rows per workgroup: 64, or 32 / 16 while the launch would have fewer than two workgroups per CU
  int ri = 4;
  while (ri > 1 && (int64_t)B * Hq * Mq * (block_m / (16 * ri)) < 512) ri >>= 1;
  p.bn_log2 = psa_ilog2(block_n); p.bm = block_m; p.halves = block_m / (16 * ri);
  p.npad = (int64_t)Nk * block_n;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  p.causal = causal ? 1 : 0;
  p.max_tiles = (block_n >= 64 ? Nk * (block_n / 64) : (Nk * block_n + 63) / 64) + 4;
  p.q_index = q_index;
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (D == 128) rc = ri == 4 ? launch_f32<128, 4>(p, st) : ri == 2 ? launch_f32<128, 2>(p, st) : launch_f32<128, 1>(p, st);
  else rc = ri == 4 ? launch_f32<64, 4>(p, st) : ri == 2 ? launch_f32<64, 2>(p, st) : launch_f32<64, 1>(p, st);
  PSA_REQUIRE(rc == PSA_OK, rc, "psa_fwd: sequence too long for the fp32 kernel's on-chip schedule (LDS)");
  return psa_check_launch("psa_fwd (fp32)");
}
