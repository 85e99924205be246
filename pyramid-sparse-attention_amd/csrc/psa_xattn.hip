// Antidiagonal ("xattn") block-importance estimator used by the causal Qwen2.5-VL path.
//
//   A[m, n]   = sum_{i < S} q[m S + S-1-i] . k[n S + i]                 (S = stride; m, n index groups of S tokens)
//   z[m, n]   = A[m, n] * log2(e) / (sqrt(D) * S);  causal: only n <= m + (Nr - Mr)
//   P[m, :]   = softmax_2(z[m, :])                                       (base-2 softmax over all strided keys)
//   Est[I, J] = sum_{m in I, n in J} P[m, n]                             (I, J: blocks of block/S strided rows)
//
// A is a plain NT GEMM of Q' [Mr, S*D] (the S rows of a group concatenated in reverse order) with
// K' [Nr, S*D] (K viewed with S rows per line), i.e. MFMA-bound: 2*Mr*Nr*S*D flops (half under causality).
// Kernel 1: 128 x 128 output tiles, 4 waves of 64 x 64, operands staged through double-buffered LDS in
// stages of 64 contraction elements; the transposed product (rows = n, lanes = m) makes the per-row
// reductions over n in-lane.  The epilogue reduces each (row m, key block J) to a pair
// (local max, sum of exp2(z - local max)) in an fp32 workspace laid out [J][m] - the logits never
// reach HBM.  Kernel 2 (HBM-bound): per row the global max and denominator from the pairs, then the
// block sums.  Rows / keys past the real length are zero vectors (zero padding to `chunk` tokens); padded
// keys are not masked (logit 0), padded query rows contribute 0.
#include "psa_common.h"

namespace {

constexpr int TM = 128, TN = 128, KC = 64;  // output tile and contraction chunk
constexpr int RST = KC * 2 + 16;            // LDS row stride (bytes)
constexpr int TILE_BYTES = 128 * RST;

struct XParams {
  const bf16_t *q, *k;
  int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl;
  float* ws;      // [B*Hq][NB][Mr][2]
  float* est;     // [B*Hq][out_rows][out_cols]
  int Hq, Hkv, Lq, Lk, D, S_log2, rb_log2;
  int Mr, Nr, NB;  // strided rows / keys (padded), key blocks
  int off;         // causal offset in strided units (Nr - Mr)
  int causal;
  int real_rows;   // strided query rows with real data
  int out_rows, out_cols;
  float scale2;
};

template <int RBL>  // log2 of the strided keys per block
__global__ __launch_bounds__(256, 2) void psa_xattn_gemm_kernel(XParams p) {
  extern __shared__ __align__(16) unsigned char smem[];  // 4 tiles: A (keys) and B (queries), double-buffered
  const int tn = blockIdx.x, tm = blockIdx.y, bh = blockIdx.z;
  const int m0 = tm * TM, n0 = tn * TN;
  if (p.causal && n0 > m0 + TM - 1 + p.off) return;  // tile entirely above the diagonal
  const int h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const int wn = wave & 1, wm = wave >> 1;
  const int S = 1 << p.S_log2;

  const bf16_t* qb = p.q + b * p.q_sb + h * p.q_sh;
  const bf16_t* kb = p.k + b * p.k_sb + hk * p.k_sh;
  const int stages = S * (p.D / KC);
  const int dchunks = p.D / KC;

  // each thread moves 4 x 16 bytes of each operand per stage: rows r = tid/8 + 32*j, 16-byte chunk tid%8
  u32x4 areg[4], breg[4];
  auto load_stage = [&](int st) __attribute__((always_inline)) {
    const int i = st / dchunks, dc = st % dchunks;
    const int c16 = tid & 7;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = (tid >> 3) + 32 * j;
      const int64_t krow = ((int64_t)(n0 + r) << p.S_log2) + i;
      const int64_t qrow = ((int64_t)(m0 + r) << p.S_log2) + (S - 1 - i);
      u32x4 z = {0u, 0u, 0u, 0u};
      areg[j] = krow < p.Lk ? *(const u32x4*)(kb + krow * p.k_sl + dc * KC + c16 * 8) : z;
      breg[j] = qrow < p.Lq ? *(const u32x4*)(qb + qrow * p.q_sl + dc * KC + c16 * 8) : z;
    }
  };
  auto store_stage = [&](int buf) __attribute__((always_inline)) {
    unsigned char* A = smem + buf * 2 * TILE_BYTES;
    unsigned char* Bm = A + TILE_BYTES;
    const int c16 = tid & 7;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = (tid >> 3) + 32 * j;
      *(u32x4*)(A + r * RST + c16 * 16) = areg[j];
      *(u32x4*)(Bm + r * RST + c16 * 16) = breg[j];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][c][i] = 0.f;

  load_stage(0);
  store_stage(0);
  if (stages > 1) load_stage(1);
  __syncthreads();
  for (int st = 0; st < stages; ++st) {
    if (st + 1 < stages) store_stage((st + 1) & 1);
    if (st + 2 < stages) load_stage(st + 2);
    const unsigned char* A = smem + (st & 1) * 2 * TILE_BYTES;
    const unsigned char* Bm = A + TILE_BYTES;
#pragma unroll
    for (int ks = 0; ks < KC / 16; ++ks) {
      bf16x8 af[2], bf[2];
#pragma unroll
      for (int a = 0; a < 2; ++a) af[a] = *(const bf16x8*)(A + (wn * 64 + a * 32 + l32) * RST + ks * 32 + hh * 16);
#pragma unroll
      for (int c = 0; c < 2; ++c) bf[c] = *(const bf16x8*)(Bm + (wm * 64 + c * 32 + l32) * RST + ks * 32 + hh * 16);
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int c = 0; c < 2; ++c) acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bf[c], acc[a][c], 0, 0, 0);
    }
    __syncthreads();
  }

  // epilogue: accumulator (a, c): rows n = n0 + wn*64 + a*32 + (i/4)*8 + hh*4 + i%4, column m = m0 + wm*64 + c*32 + l32
  constexpr int OPB = 1 << (RBL - 3);  // 8-key octets per block: 1, 2 or 4
  float* ws = p.ws + (int64_t)bh * p.NB * p.Mr * 2;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int m = m0 + wm * 64 + c * 32 + l32;
    const int nlim = p.causal ? m + p.off : 0x7fffffff;  // visible keys: n <= nlim
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int nb0 = n0 + wn * 64 + a * 32;
      float z[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int n = nb0 + (i >> 2) * 8 + hh * 4 + (i & 3);
        z[i] = n <= nlim ? acc[a][c][i] * p.scale2 : -INFINITY;
      }
      // an octet of 8 consecutive keys = registers 4o..4o+3 of both half-waves; OPB octets form a block
#pragma unroll
      for (int blk = 0; blk < 4 / OPB; ++blk) {
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4 * OPB; ++i) mx = fmaxf(mx, z[blk * 4 * OPB + i]);
        mx = half_wave_max(mx);
        const float ref = mx == -INFINITY ? 0.f : mx;
        float sm = 0.f;
#pragma unroll
        for (int i = 0; i < 4 * OPB; ++i) sm += fast_exp2(z[blk * 4 * OPB + i] - ref);
        sm = half_wave_sum(sm);
        if (hh == 0) {
          const int J = (nb0 + blk * 8 * OPB) >> RBL;
          f32x2 pr = {mx, sm};
          *(f32x2*)(ws + ((int64_t)J * p.Mr + m) * 2) = pr;
        }
      }
    }
  }
}

// one workgroup per (b, h, q-block): 256 threads; thread t handles key blocks t, t+256, ...
__global__ __launch_bounds__(256) void psa_xattn_reduce_kernel(XParams p) {
  __shared__ float s_M[32], s_inv[32];
  __shared__ float s_big[256];
  const int I = blockIdx.x, bh = blockIdx.y;
  const int tid = threadIdx.x;
  const int rb = 1 << p.rb_log2;
  const int m0 = I * rb;
  const float* ws = p.ws + (int64_t)bh * p.NB * p.Mr * 2;
  // pass 1: row max and denominator.  Thread (r = tid % rb, jl = tid / rb) strides over the key blocks
  // visible to row r (J <= (m + off) / rb under causality); partials are combined in a fixed order.
  const int r = tid & (rb - 1), jl = tid >> p.rb_log2, nj = 256 >> p.rb_log2;
  const int m = m0 + r;
  const int jmax = p.causal ? ((m + p.off) >> p.rb_log2) + 1 : p.NB;
  const int jend = jmax < p.NB ? jmax : p.NB;
  float M = -INFINITY;
  for (int J = jl; J < jend; J += nj) M = fmaxf(M, ws[((int64_t)J * p.Mr + m) * 2]);
  s_big[jl * rb + r] = M;
  __syncthreads();
  if (tid < rb) {
    float mm = -INFINITY;
    for (int j = 0; j < nj; ++j) mm = fmaxf(mm, s_big[j * rb + tid]);
    s_M[tid] = mm;
  }
  __syncthreads();
  const float Mref = s_M[r] == -INFINITY ? 0.f : s_M[r];
  float l = 0.f;
  for (int J = jl; J < jend; J += nj) {
    const f32x2 pr = *(const f32x2*)(ws + ((int64_t)J * p.Mr + m) * 2);
    l += pr[1] * fast_exp2(pr[0] - Mref);  // pr = (-inf, 0) for fully masked pairs: 0 * exp2(-inf) = 0
  }
  __syncthreads();
  s_big[jl * rb + r] = l;
  __syncthreads();
  if (tid < rb) {
    float ll = 0.f;
    for (int j = 0; j < nj; ++j) ll += s_big[j * rb + tid];
    const bool real = (m0 + tid) < p.real_rows;
    s_inv[tid] = (real && ll > 0.f) ? 1.0f / ll : 0.f;  // padded query rows contribute nothing
  }
  __syncthreads();
  // pass 2: Est[I, J] = sum_r sum[r, J] * exp2(max[r, J] - M_r) / l_r
  float* dst = p.est + ((int64_t)bh * p.out_rows + I) * p.out_cols;
  for (int J = tid; J < p.out_cols; J += 256) {
    float e = 0.f;
    for (int rr = 0; rr < rb; ++rr) {
      const int mm = m0 + rr;
      const int jm = p.causal ? ((mm + p.off) >> p.rb_log2) + 1 : p.NB;
      if (J < jm) {
        const f32x2 pr = *(const f32x2*)(ws + ((int64_t)J * p.Mr + mm) * 2);
        const float Mx = s_M[rr] == -INFINITY ? 0.f : s_M[rr];
        e += pr[1] * fast_exp2(pr[0] - Mx) * s_inv[rr];
      }
    }
    dst[J] = e;
  }
}

struct XGeom {
  int Lq_pad, Lk_pad, Mr, Nr, NB, MB;
};
XGeom xgeom(int Lq, int Lk, int block, int stride, int chunk) {
  XGeom g;
  g.Lq_pad = (Lq + chunk - 1) / chunk * chunk;
  g.Lk_pad = (Lk + chunk - 1) / chunk * chunk;
  g.Mr = g.Lq_pad / stride;
  g.Nr = g.Lk_pad / stride;
  g.NB = g.Lk_pad / block;
  g.MB = g.Lq_pad / block;
  return g;
}

}  // namespace

extern "C" int64_t psa_estimate_xattn_workspace_bytes(int B, int Hq, int Lq, int Lk, int block_size, int stride, int chunk_size) {
  if (B <= 0 || Hq <= 0 || Lq <= 0 || Lk <= 0 || block_size <= 0 || stride <= 0 || chunk_size <= 0) return 0;
  const XGeom g = xgeom(Lq, Lk, block_size, stride, chunk_size);
  return (int64_t)B * Hq * g.NB * g.Mr * 2 * (int64_t)sizeof(float);
}

extern "C" int psa_estimate_xattn(psa_tensor4 q, psa_tensor4 k, float* est, void* workspace, int B, int Hq, int Hkv, int Lq,
                                  int Lk, int D, int block_size, int stride, int chunk_size, int causal, psa_stream_t stream) {
  PSA_REQUIRE(q.ptr && k.ptr && est && workspace, PSA_ERR_ARG, "psa_estimate_xattn: null pointer");
  PSA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Lq > 0 && Lk > 0, PSA_ERR_ARG, "psa_estimate_xattn: sizes must be positive");
  PSA_REQUIRE(Hq % Hkv == 0, PSA_ERR_ARG, "psa_estimate_xattn: Hq must be a multiple of Hkv");
  PSA_REQUIRE(D == 64 || D == 128, PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: head dim %d not in {64, 128}", D);
  PSA_REQUIRE(psa_is_pow2(stride) && stride <= 16, PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: stride=%d must be a power of two <= 16", stride);
  PSA_REQUIRE(psa_is_pow2(block_size) && block_size % stride == 0, PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: bad block_size");
  const int rb = block_size / stride;
  PSA_REQUIRE(rb == 8 || rb == 16 || rb == 32, PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: block_size/stride=%d not in {8,16,32}", rb);
  PSA_REQUIRE(chunk_size % (128 * stride) == 0, PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: chunk_size must be a multiple of 128*stride");
  PSA_REQUIRE(Lk >= Lq, PSA_ERR_ARG, "psa_estimate_xattn: Lk must not be shorter than Lq");
  PSA_REQUIRE(((uintptr_t)q.ptr % 16 == 0) && ((uintptr_t)k.ptr % 16 == 0) && q.stride_l % 8 == 0 && k.stride_l % 8 == 0 &&
                  q.stride_h % 8 == 0 && k.stride_h % 8 == 0 && q.stride_b % 8 == 0 && k.stride_b % 8 == 0,
              PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: tensors must be 16-byte aligned with strides multiple of 8");
  PSA_REQUIRE((int64_t)B * Hq <= 65535, PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: B*Hq too large");
  const XGeom g = xgeom(Lq, Lk, block_size, stride, chunk_size);
  XParams p;
  p.q = (const bf16_t*)q.ptr; p.k = (const bf16_t*)k.ptr;
  p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sl = q.stride_l;
  p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sl = k.stride_l;
  p.ws = (float*)workspace; p.est = est;
  p.Hq = Hq; p.Hkv = Hkv; p.Lq = Lq; p.Lk = Lk; p.D = D;
  p.S_log2 = psa_ilog2(stride); p.rb_log2 = psa_ilog2(rb);
  p.Mr = g.Mr; p.Nr = g.Nr; p.NB = g.NB;
  p.off = g.Nr - g.Mr;
  p.causal = causal ? 1 : 0;
  // the reference zeroes rows at or past (real key length)/stride in the key-aligned numbering
  p.real_rows = (Lk + stride - 1) / stride - p.off;
  p.out_rows = (Lq + block_size - 1) / block_size;
  p.out_cols = (Lk + block_size - 1) / block_size;
  p.scale2 = 1.4426950408889634f / sqrtf((float)D) / (float)stride;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)(g.Nr / TN), (unsigned)(g.Mr / TM), (unsigned)(B * Hq));
  const size_t shmem = 4 * (size_t)TILE_BYTES;
  auto launch = [&](auto kern) -> int {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess) return PSA_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, grid, dim3(256), shmem, st, p);
    return PSA_OK;
  };
  int rc = rb == 8 ? launch(psa_xattn_gemm_kernel<3>) : rb == 16 ? launch(psa_xattn_gemm_kernel<4>) : launch(psa_xattn_gemm_kernel<5>);
  PSA_REQUIRE(rc == PSA_OK, rc, "psa_estimate_xattn: cannot reserve LDS");
  rc = psa_check_launch("psa_estimate_xattn (contraction)");
  if (rc != PSA_OK) return rc;
  hipLaunchKernelGGL(psa_xattn_reduce_kernel, dim3((unsigned)p.out_rows, (unsigned)(B * Hq)), dim3(256), 0, st, p);
  return psa_check_launch("psa_estimate_xattn (reduction)");
}
