// Sampled block-importance estimator: a dense bf16 MFMA contraction of the sampled query rows with
// the sampled key rows, with the reference's max-pooling epilogue fused in, so neither the sampled
// tensors nor the per-row group maxima ever touch HBM.
//
//   R[r, j]  = max_{c in key group j} (q_r . k_c) * scale * log2(e)
//   m[r]     = max_j R[r, j]
//   Po[i, j] = max_{r in query group i} exp2(R[r, j] - m[r]);   Po[i, :] /= sum_j Po[i, j]
//
// One workgroup = NW waves x 32 sampled query rows; all waves share the K tile (64 sampled keys,
// gathered straight from the un-sampled K through the per-head offset table).  As in the forward
// kernel the transposed product S^T = K Q^T is computed, so that a lane holds 16 keys of one query
// row and a key-group maximum is an in-lane reduction plus one half-wave exchange.  R for the
// workgroup's rows stays in LDS (fp32, [key group][33]) until the row maxima are final.
//
// Roofline: MFMA-bound (2 * Ms * Ns * D flops against ~(Ms + Ns) * D * 2 bytes).
#include "psa_common.h"

namespace {

constexpr int TK = 64;
constexpr int RST = 33;  // floats per key-group row of the R buffer (32 + 1 pad)

struct EstParams {
  const bf16_t *q, *k;
  int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl;
  const int32_t *off_q, *off_k;
  float* scores;
  int Hq, Hkv, Lq, Lk;
  int bm, bn, keep_m_log2, keep_n_log2;
  int Ms, Ns, Ns_pad;  // real sampled rows / keys, padded key count (multiple of 64)
  int n_d;             // key groups incl. padding groups
  int out_rows, out_cols;
  float qk_scale;
};

__device__ __forceinline__ int sampled_src(int r, int n_real, int keep_log2, int block, const int32_t* off, int L) {
  r = r < n_real ? r : n_real - 1;
  const int grp = r >> keep_log2, e = r & ((1 << keep_log2) - 1);
  const int src = grp * block + (off ? off[e] : e);
  return src < L ? src : L - 1;
}

template <int D, int NW>
__global__ __launch_bounds__(NW * 64) void psa_estimate_kernel(EstParams p) {
  constexpr int NT = NW * 64;
  constexpr int CH = D / 8;
  constexpr int UNITS = 16 * CH;
  constexpr int PER = (UNITS + NT - 1) / NT;
  constexpr int KK = D / 16;
  constexpr int KST = D * 2 + 16;

  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* Ks = smem;
  float* Rl = (float*)(smem + TK * KST);  // [NW][n_d][RST]
  float* ml = Rl + (size_t)NW * p.n_d * RST;  // [NW][32]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const int bh = blockIdx.y;
  const int h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);
  const int keep_m = 1 << p.keep_m_log2, keep_n = 1 << p.keep_n_log2;

  // Q fragments
  const int row0 = blockIdx.x * (NW * 32) + wave * 32;
  bf16x8 qf[KK];
  {
    const int32_t* oq = p.off_q ? p.off_q + (int64_t)bh * keep_m : nullptr;
    const int src = sampled_src(row0 + l32, p.Ms, p.keep_m_log2, p.bm, oq, p.Lq);
    const bf16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)src * p.q_sl + hh * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const bf16x8*)(qp + kk * 16);
  }

  const bf16_t* kb = p.k + b * p.k_sb + hk * p.k_sh;
  const int32_t* ok = p.off_k ? p.off_k + ((int64_t)b * p.Hkv + hk) * keep_n : nullptr;
  u32x4 kreg[PER][4];
  auto load_tile = [&](int t) {
#pragma unroll
    for (int u_ = 0; u_ < PER; ++u_) {
      const int u = tid + u_ * NT;
      if (UNITS % NT != 0 && u >= UNITS) break;
      const int r0 = (u / CH) * 4, ch = u % CH;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int src = sampled_src(t * TK + r0 + i, p.Ns, p.keep_n_log2, p.bn, ok, p.Lk);
        kreg[u_][i] = *(const u32x4*)(kb + (int64_t)src * p.k_sl + ch * 8);
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int u_ = 0; u_ < PER; ++u_) {
      const int u = tid + u_ * NT;
      if (UNITS % NT != 0 && u >= UNITS) break;
      const int r0 = (u / CH) * 4, ch = u % CH;
#pragma unroll
      for (int i = 0; i < 4; ++i) *(u32x4*)(Ks + (r0 + i) * KST + ch * 16) = kreg[u_][i];
    }
  };

  float* Rw = Rl + (size_t)wave * p.n_d * RST;
  float m_run = -INFINITY;
  const int T = p.Ns_pad / TK;
  const int gpc_log2 = 5 - p.keep_n_log2;  // key groups per 32-key chunk (1, 2 or 4)

  load_tile(0);
  for (int t = 0; t < T; ++t) {
    __syncthreads();
    store_tile();
    __syncthreads();
    if (t + 1 < T) load_tile(t + 1);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      f32x16 s;
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] = 0.f;
      const unsigned char* kr = Ks + (c * 32 + l32) * KST + hh * 16;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const bf16x8 a = *(const bf16x8*)(kr + kk * 32);
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[kk], s, 0, 0, 0);
      }
      // register i holds key (i/4)*8 + hh*4 + i%4 of this chunk: 8-key octets are registers 4o..4o+3
      float o4[4];
#pragma unroll
      for (int o = 0; o < 4; ++o) o4[o] = fmaxf(fmaxf(s[4 * o], s[4 * o + 1]), fmaxf(s[4 * o + 2], s[4 * o + 3]));
      const int jbase = (t * 2 + c) << gpc_log2;
      if (gpc_log2 == 0) {
        float v = fmaxf(fmaxf(o4[0], o4[1]), fmaxf(o4[2], o4[3]));
        v = fmaxf(v, shfl_xor32(v)) * p.qk_scale;
        m_run = fmaxf(m_run, v);
        if (hh == 0) Rw[jbase * RST + l32] = v;
      } else if (gpc_log2 == 1) {
        float v0 = fmaxf(o4[0], o4[1]), v1 = fmaxf(o4[2], o4[3]);
        v0 = fmaxf(v0, shfl_xor32(v0)) * p.qk_scale;
        v1 = fmaxf(v1, shfl_xor32(v1)) * p.qk_scale;
        m_run = fmaxf(m_run, fmaxf(v0, v1));
        if (hh == 0) {
          Rw[jbase * RST + l32] = v0;
          Rw[(jbase + 1) * RST + l32] = v1;
        }
      } else {
#pragma unroll
        for (int o = 0; o < 4; ++o) {
          const float v = fmaxf(o4[o], shfl_xor32(o4[o])) * p.qk_scale;
          m_run = fmaxf(m_run, v);
          if (hh == 0) Rw[(jbase + o) * RST + l32] = v;
        }
      }
    }
  }
  if (hh == 0) ml[wave * 32 + l32] = m_run;
  __syncthreads();

  // phase 2: per query group, Po[j] = exp2(max_r (R[r][j] - m[r])), normalised by the sum over ALL n_d
  const float* mw = ml + wave * 32;
  const int groups = 32 >> p.keep_m_log2;
  for (int g = 0; g < groups; ++g) {
    const int grow = ((row0 + g * keep_m) >> p.keep_m_log2);
    const int r_lo = g * keep_m;
    float part = 0.f;
    for (int j = lane; j < p.n_d; j += 64) {
      float v = -INFINITY;
      for (int r = 0; r < keep_m; ++r) v = fmaxf(v, Rw[j * RST + r_lo + r] - mw[r_lo + r]);
      const float e = fast_exp2(v);
      Rw[j * RST + r_lo] = e;
      part += e;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
    if (grow < p.out_rows) {
      float* dst = p.scores + ((int64_t)bh * p.out_rows + grow) * p.out_cols;
      for (int j = lane; j < p.out_cols; j += 64) dst[j] = Rw[j * RST + r_lo] / part;
    }
  }
}

template <int D, int NW>
int launch_est(const EstParams& p, int B, int q_rows_needed, hipStream_t stream) {
  size_t shmem = (size_t)TK * (D * 2 + 16) + ((size_t)NW * p.n_d * RST + NW * 32) * sizeof(float);
  if (shmem > 160 * 1024) return PSA_ERR_UNSUPPORTED;
  if (shmem > 48 * 1024) {
    if (hipFuncSetAttribute((const void*)psa_estimate_kernel<D, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess)
      return PSA_ERR_LAUNCH;
  }
  dim3 grid((unsigned)((q_rows_needed + NW * 32 - 1) / (NW * 32)), (unsigned)(B * p.Hq));
  hipLaunchKernelGGL((psa_estimate_kernel<D, NW>), grid, dim3(NW * 64), shmem, stream, p);
  return PSA_OK;
}

}  // namespace

extern "C" int psa_estimate_sampled(psa_tensor4 q, psa_tensor4 k, const int32_t* off_q, const int32_t* off_k, float* scores,
                                    int B, int Hq, int Hkv, int Lq, int Lk, int D, int block_m, int block_n, int keep_m,
                                    int keep_n, float sm_scale, int out_rows, int out_cols, psa_stream_t stream) {
  PSA_REQUIRE(q.ptr && k.ptr && scores, PSA_ERR_ARG, "psa_estimate_sampled: null pointer");
  PSA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Lq > 0 && Lk > 0, PSA_ERR_ARG, "psa_estimate_sampled: sizes must be positive");
  PSA_REQUIRE(Hq % Hkv == 0, PSA_ERR_ARG, "psa_estimate_sampled: Hq must be a multiple of Hkv");
  PSA_REQUIRE((int64_t)B * Hq <= 65535, PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: B*Hq too large");
  PSA_REQUIRE(D == 64 || D == 128, PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: head dim %d not in {64, 128}", D);
  PSA_REQUIRE(keep_m == 8 || keep_m == 16 || keep_m == 32, PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: keep_m=%d not in {8,16,32}", keep_m);
  PSA_REQUIRE(keep_n == 8 || keep_n == 16 || keep_n == 32, PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: keep_n=%d not in {8,16,32}", keep_n);
  PSA_REQUIRE(block_m >= keep_m && block_n >= keep_n, PSA_ERR_ARG, "psa_estimate_sampled: block smaller than keep");
  PSA_REQUIRE(((uintptr_t)q.ptr % 16 == 0) && ((uintptr_t)k.ptr % 16 == 0) && q.stride_l % 8 == 0 && k.stride_l % 8 == 0 &&
                  q.stride_h % 8 == 0 && k.stride_h % 8 == 0 && q.stride_b % 8 == 0 && k.stride_b % 8 == 0,
              PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: tensors must be 16-byte aligned with strides multiple of 8");
  EstParams p;
  p.q = (const bf16_t*)q.ptr; p.k = (const bf16_t*)k.ptr;
  p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sl = q.stride_l;
  p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sl = k.stride_l;
  p.off_q = off_q; p.off_k = off_k; p.scores = scores;
  p.Hq = Hq; p.Hkv = Hkv; p.Lq = Lq; p.Lk = Lk; p.bm = block_m; p.bn = block_n;
  p.keep_m_log2 = psa_ilog2(keep_m); p.keep_n_log2 = psa_ilog2(keep_n);
  const int Mq = (Lq + block_m - 1) / block_m, Nk = (Lk + block_n - 1) / block_n;
  p.Ms = Mq * keep_m; p.Ns = Nk * keep_n;
  const int Ms_pad = (p.Ms + 63) / 64 * 64;
  p.Ns_pad = (p.Ns + 63) / 64 * 64;
  p.n_d = p.Ns_pad / keep_n;
  const int m_d = Ms_pad / keep_m;
  PSA_REQUIRE(out_rows > 0 && out_rows <= m_d && out_cols > 0 && out_cols <= p.n_d, PSA_ERR_ARG,
              "psa_estimate_sampled: out_rows/out_cols exceed %d x %d", m_d, p.n_d);
  p.out_rows = out_rows; p.out_cols = out_cols;
  p.qk_scale = sm_scale * 1.44269504f;
  const int rows_needed = out_rows * keep_m;
  // waves per workgroup: as many as the R buffer lets fit in LDS
  const size_t kt = (size_t)TK * (D * 2 + 16);
  int nw = 4;
  while (nw > 1 && kt + ((size_t)nw * p.n_d * RST + nw * 32) * 4 > 160 * 1024) nw >>= 1;
  int rc;
  if (D == 128) rc = nw == 4 ? launch_est<128, 4>(p, B, rows_needed, (hipStream_t)stream)
                   : nw == 2 ? launch_est<128, 2>(p, B, rows_needed, (hipStream_t)stream)
                             : launch_est<128, 1>(p, B, rows_needed, (hipStream_t)stream);
  else rc = nw == 4 ? launch_est<64, 4>(p, B, rows_needed, (hipStream_t)stream)
            : nw == 2 ? launch_est<64, 2>(p, B, rows_needed, (hipStream_t)stream)
                      : launch_est<64, 1>(p, B, rows_needed, (hipStream_t)stream);
  PSA_REQUIRE(rc == PSA_OK, rc, "psa_estimate_sampled: %d key groups do not fit the on-chip score buffer", p.n_d);
  return psa_check_launch("psa_estimate_sampled");
}
