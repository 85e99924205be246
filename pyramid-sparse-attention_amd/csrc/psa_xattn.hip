// Antidiagonal ("xattn") block-importance estimator used by the causal Qwen2.5-VL path.
//
//   A[m, n]   = sum_{i < S} q[m S + S-1-i] . k[n S + i]                 (S = stride; m, n index groups of S tokens)
//   z[m, n]   = A[m, n] * log2(e) / (sqrt(D) * S);  causal: only n <= m + (Nr - Mr)
//   P[m, :]   = softmax_2(z[m, :])                                       (base-2 softmax over all strided keys)
//   Est[I, J] = sum_{m in I, n in J} P[m, n]                             (I, J: blocks of block/S strided rows)
//
// A is a plain NT GEMM of Q' [Mr, S*D] (the S rows of a group concatenated in reverse order) with
// K' [Nr, S*D] (K viewed with S rows per line), i.e. MFMA-bound: 2*Mr*Nr*S*D flops (half under causality).
// Kernel 1: 256 (m) x 256 (n) output tiles, 8 waves of 64 (m) x 128 (n); both operands go from global memory
// straight into double-buffered LDS (global_load_lds_dwordx4, the padded + swizzled 64-row tile layout of
// psa_tiles.h) in stages of 64 contraction elements, i.e. half a head-dim row of one of the S interleaved
// tokens; the transposed product (rows = n, lanes = m) makes the per-row reductions over n in-lane.  The tile
// size is set by the copy path and LDS: a 256 x 256 tile needs 32 bytes of copies per CU cycle at the full MFMA
// rate (the path delivers 64; a 128 x 128 tile would need all of it) and 0.75 LDS operand reads per MFMA.
// The epilogue reduces each (row m, key block J) to a pair
// (local max, sum of exp2(z - local max)) in an fp32 workspace laid out [J][m] - the logits never
// reach HBM.  Kernel 2 (HBM-bound): per row the global max and denominator from the pairs, then the
// block sums.  Rows / keys past the real length are zero vectors (zero padding to `chunk` tokens); padded
// keys are not masked (logit 0), padded query rows contribute 0.
#include "psa_common.h"
#include "psa_tiles.h"

namespace {

constexpr int TM = 256, TN = 256, KC = 64;  // output tile and contraction chunk
using XG = psa_tiles::LtGeom<KC>;            // LDS tiles: 64 rows of KC values
constexpr int X_TILE = XG::TILE, X_ISTR = psa_tiles::LT_ISTR;
constexpr int X_QT = TM / 64, X_KT = TN / 64;             // Q and K tiles per stage
constexpr int X_STAGE = (X_QT + X_KT) * X_TILE;           // bytes per stage
constexpr int X_GROUPS = (X_QT + X_KT) * 4;               // 16-row groups per stage
constexpr int X_WAVES = 8, X_GPW = X_GROUPS / X_WAVES;    // groups copied per wave
static_assert(X_GROUPS % X_WAVES == 0, "groups divide over the waves");
constexpr int X_BUFS = 2;                                 // stages in LDS
constexpr int X_NA = TN / 2 / 32, X_NC = TM / 4 / 32;     // 32 x 32 accumulators per wave: X_NA along n, X_NC along m

// rows past the end of Q / K are zero vectors: their copies read this page
__device__ __align__(256) const unsigned char x_zero_page[256] = {};

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
  int tiles_m, tiles_n, act_per_bh, n_active, per_xcd;  // output tiles; those with visible keys per (batch, head) / in all / per XCD
};

// output tiles of tile row tm that contain visible keys
__host__ __device__ inline int tiles_in_row(int tm, int tiles_n, int causal, int off) {
  if (!causal) return tiles_n;
  const int last_n = (tm + 1) * TM - 1 + off;  // last visible strided key of the row's last query
  const int n = last_n / TN + 1;
  return n < tiles_n ? n : tiles_n;
}

template <int RBL>  // log2 of the strided keys per block
__global__ __launch_bounds__(X_WAVES * 64, 1) void psa_xattn_gemm_kernel(XParams p) {
  extern __shared__ __align__(16) unsigned char smem[];  // X_BUFS stages of [Q tiles | K tiles]
  // Workgroup ids go round-robin over the 8 XCDs and every XCD runs its ids in order.  The output tiles with
  // visible keys are listed (batch-head, tile row, tile column) and the list is cut into 8 contiguous shares, one
  // per XCD: all tiles cost the same, so the XCDs finish together, and the ~32 tiles an XCD works on at a time
  // are neighbours that find each other's Q and K rows in its L2.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int idx = xcd * p.per_xcd + slot;
  if (idx >= p.n_active) return;
  const int bh = idx / p.act_per_bh;
  int tn = idx % p.act_per_bh, tm = 0;
  for (;; ++tm) {
    const int row_n = tiles_in_row(tm, p.tiles_n, p.causal, p.off);
    if (tn < row_n) break;
    tn -= row_n;
  }
  const int m0 = tm * TM, n0 = tn * TN;
  const int h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;
  const int wn = wave & 1, wm = wave >> 1;  // wave tile: rows m0 + 64 * wm .., keys n0 + 128 * wn ..
  const int S = 1 << p.S_log2;

  const char* qb = (const char*)(p.q + b * p.q_sb + h * p.q_sh);
  const char* kb = (const char*)(p.k + b * p.k_sb + hk * p.k_sh);
  const uint32_t q_strb = (uint32_t)p.q_sl * 2u, k_strb = (uint32_t)p.k_sl * 2u;
  const int dc_log2 = p.D == 2 * KC ? 1 : 0;  // 64-channel chunks per row: 1 (D = 64) or 2 (D = 128)
  const int stages = S << dc_log2;

  // copies: wave w moves the 16-row groups w*X_GPW .. of a stage (group g: tile g/4, rows 16*(g%4)..), a lane
  // the RPL consecutive rows frow.. of each group; a row is one strided index (S tokens apart in memory)
  constexpr int RPL = XG::RPL;
  const uint32_t f_chunk = psa_tiles::lt_fetch_chunk<KC>(lane);
  const int frow = psa_tiles::lt_fetch_row<KC>(lane);
  int g_idx[X_GPW];       // strided index (m or n) of the lane's first row of each group
  uint32_t g_off[X_GPW];  // its byte offset inside the (batch, head) slice, token 0 of the S, contraction chunk 0
  bool edge = false;      // some row of this tile reaches past the real length: take the checked path
#pragma unroll
  for (int j = 0; j < X_GPW; ++j) {
    const int g = wave * X_GPW + j, tile = g >> 2;
    const bool is_q = tile < X_QT;
    const int idx = (is_q ? m0 + tile * 64 : n0 + (tile - X_QT) * 64) + (g & 3) * 16 + frow;
    g_idx[j] = idx;
    g_off[j] = ((uint32_t)idx << p.S_log2) * (is_q ? q_strb : k_strb) + f_chunk;
  }
  edge = ((int64_t)(m0 + TM) << p.S_log2) > p.Lq || ((int64_t)(n0 + TN) << p.S_log2) > p.Lk;  // (covers tiles that stick out of Mr / Nr)
  // copy instruction `piece` (0 .. X_GPW * RPL - 1) of stage st
  auto issue_piece = [&](int st, int piece) __attribute__((always_inline)) {
    const int j = piece / RPL, n = piece % RPL;
    const int i = st >> dc_log2, dc = st & ((1 << dc_log2) - 1);  // (shifts: a division here would run on the vector unit and take the base pointers with it)
    unsigned char* dst = smem + (st & 1) * X_STAGE;
    const int g = wave * X_GPW + j, tile = g >> 2;
    const bool is_q = tile < X_QT;
    // token S-1-i of every query group, token i of every key group
    const char* base = is_q ? qb + (uint64_t)(S - 1 - i) * q_strb + dc * (KC * 2) : kb + (uint64_t)i * k_strb + dc * (KC * 2);
    const uint32_t rstr = (is_q ? q_strb : k_strb) << p.S_log2;
    const uint32_t lds = psa_tiles::lds_addr_of(dst + tile * X_TILE + ((g & 3) * RPL + n) * X_ISTR);
    if (!edge) {
      psa_tiles::lds_copy16(base, g_off[j] + n * rstr, lds);
    } else {
      const int64_t tok = ((int64_t)(g_idx[j] + n) << p.S_log2) + (is_q ? S - 1 - i : i);
      const bool real = tok < (is_q ? p.Lq : p.Lk);
      const char* src = real ? base + (g_off[j] + n * rstr) : (const char*)x_zero_page + f_chunk;
      psa_tiles::lds_copy16_addr(src, lds);
    }
  };
  auto issue_stage = [&](int st) __attribute__((always_inline)) {
#pragma unroll
    for (int piece = 0; piece < X_GPW * RPL; ++piece) issue_piece(st, piece);
  };
  // operands: K rows (A) of tile wn, Q rows (B) of tile wm; rows l32 and l32 + 32; k-step ks: off[ks & 1] + 64 * (ks >> 1)
  uint32_t r_off[2];
  psa_tiles::lt_row_operand<KC>(l32, hh, r_off);

  f32x16 acc[X_NA][X_NC];
#pragma unroll
  for (int a = 0; a < X_NA; ++a)
#pragma unroll
    for (int c = 0; c < X_NC; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][c][i] = 0.f;

  issue_stage(0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  for (int st = 0; st < stages; ++st) {
    // invariant: buffer st&1 holds stage st and every wave is done with the other buffer
    if (st + 1 < stages) issue_stage(st + 1);
    PSA_LDS(const unsigned char) Qs = (PSA_LDS(const unsigned char))(smem) + (st & 1) * X_STAGE + wm * X_TILE;
    PSA_LDS(const unsigned char) Ks = (PSA_LDS(const unsigned char))(smem) + (st & 1) * X_STAGE + (X_QT + wn * (X_NA / 2)) * X_TILE;
#pragma unroll
    for (int ks = 0; ks < KC / 16; ++ks) {
      bf16x8 af[X_NA], bf[X_NC];
      const uint32_t o = r_off[ks & 1] + (ks >> 1) * 64;
#pragma unroll
      for (int a = 0; a < X_NA; ++a) af[a] = *(PSA_LDS(const bf16x8))(Ks + o + (a >> 1) * X_TILE + (a & 1) * XG::HALF);
#pragma unroll
      for (int c = 0; c < X_NC; ++c) bf[c] = *(PSA_LDS(const bf16x8))(Qs + o + c * XG::HALF);
#pragma unroll
      for (int a = 0; a < X_NA; ++a)
#pragma unroll
        for (int c = 0; c < X_NC; ++c) acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bf[c], acc[a][c], 0, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // the copies of stage st+1 were issued a stage ago
    __syncthreads();
  }

  // epilogue: accumulator (a, c): rows n = n0 + wn*128 + a*32 + (i/4)*8 + hh*4 + i%4, column m = m0 + wm*64 + c*32 + l32
  constexpr int OPB = 1 << (RBL - 3);  // 8-key octets per block: 1, 2 or 4
  float* ws = p.ws + (int64_t)bh * p.NB * p.Mr * 2;
#pragma unroll
  for (int c = 0; c < X_NC; ++c) {
    const int m = m0 + wm * 64 + c * 32 + l32;
    const int nlim = p.causal ? m + p.off : 0x7fffffff;  // visible keys: n <= nlim
#pragma unroll
    for (int a = 0; a < X_NA; ++a) {
      const int nb0 = n0 + wn * (TN / 2) + a * 32;
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
        if (hh == 0 && m < p.Mr && nb0 < p.Nr) {
          const int J = (nb0 + blk * 8 * OPB) >> RBL;
          f32x2 pr = {mx, sm};
          *(f32x2*)(ws + ((int64_t)J * p.Mr + m) * 2) = pr;
        }
      }
    }
  }
}

// one workgroup per (b, h, q-block): 256 threads; thread t handles key blocks t, t+256, ...
// cached != 0: the (maximum, sum) pairs of the workgroup's rows are read from the workspace once into dynamic LDS
// ([key block][row], NB * rb pairs) and the three passes below run on that copy instead of on memory.
__global__ __launch_bounds__(256) void psa_xattn_reduce_kernel(XParams p, int cached) {
  extern __shared__ __align__(16) unsigned char s_cache[];
  __shared__ float s_M[32], s_inv[32];
  __shared__ float s_big[256];
  const int I = blockIdx.x, bh = blockIdx.y;
  const int tid = threadIdx.x;
  const int rb = 1 << p.rb_log2;
  const int m0 = I * rb;
  const float* ws = p.ws + (int64_t)bh * p.NB * p.Mr * 2;
  int64_t row_stride = p.Mr;  // pairs between consecutive key blocks of one row
  int m_sub = 0;
  if (cached) {
    // a key block's rb pairs of this q-block are contiguous in the workspace: rb * 8 bytes per key block
    f32x2* c = (f32x2*)s_cache;
    const int jlim = p.causal ? (((m0 + rb - 1 + p.off) >> p.rb_log2) + 1) : p.NB;  // key blocks any row of the q-block sees
    const int jn = jlim < p.NB ? jlim : p.NB;
    for (int u = tid; u < jn * rb; u += 256) {
      const int J = u >> p.rb_log2, rr = u & (rb - 1);
      c[u] = *(const f32x2*)(ws + ((int64_t)J * p.Mr + m0 + rr) * 2);
    }
    __syncthreads();
    ws = (const float*)s_cache;
    row_stride = rb;
    m_sub = m0;  // the copy starts at row m0: index (J * rb + (m - m0)) (never form a pointer below the array)
  }
  // pass 1: row max and denominator.  Thread (r = tid % rb, jl = tid / rb) strides over the key blocks
  // visible to row r (J <= (m + off) / rb under causality); partials are combined in a fixed order.
  const int r = tid & (rb - 1), jl = tid >> p.rb_log2, nj = 256 >> p.rb_log2;
  const int m = m0 + r;
  const int jmax = p.causal ? ((m + p.off) >> p.rb_log2) + 1 : p.NB;
  const int jend = jmax < p.NB ? jmax : p.NB;
  float M = -INFINITY;
  for (int J = jl; J < jend; J += nj) M = fmaxf(M, ws[((int64_t)J * row_stride + (m - m_sub)) * 2]);
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
    const f32x2 pr = *(const f32x2*)(ws + ((int64_t)J * row_stride + (m - m_sub)) * 2);
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
        const f32x2 pr = *(const f32x2*)(ws + ((int64_t)J * row_stride + (mm - m_sub)) * 2);
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
  PSA_REQUIRE(((int64_t)Lq + chunk_size) * q.stride_l * 2 < (1ll << 32) && ((int64_t)Lk + chunk_size) * k.stride_l * 2 < (1ll << 32),
              PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: one (batch, head) slice of Q/K must span less than 4 GiB");
  PSA_REQUIRE(Lk >= Lq, PSA_ERR_ARG, "psa_estimate_xattn: Lk must not be shorter than Lq");
  PSA_REQUIRE(((uintptr_t)q.ptr % 16 == 0) && ((uintptr_t)k.ptr % 16 == 0) && q.stride_l % 8 == 0 && k.stride_l % 8 == 0 &&
                  q.stride_h % 8 == 0 && k.stride_h % 8 == 0 && q.stride_b % 8 == 0 && k.stride_b % 8 == 0,
              PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: tensors must be 16-byte aligned with strides multiple of 8");
  PSA_REQUIRE((int64_t)B * Hq <= 65535, PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: B*Hq too large");
  PSA_REQUIRE(q.dtype == PSA_DTYPE_BF16 && k.dtype == PSA_DTYPE_BF16, PSA_ERR_UNSUPPORTED,
              "psa_estimate_xattn: bf16 tensors only (element type %d / %d)", q.dtype, k.dtype);
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
  p.tiles_m = (g.Mr + TM - 1) / TM;
  p.tiles_n = (g.Nr + TN - 1) / TN;
  p.act_per_bh = 0;
  for (int tm = 0; tm < p.tiles_m; ++tm) p.act_per_bh += tiles_in_row(tm, p.tiles_n, p.causal, p.off);
  const int64_t n_active = (int64_t)B * Hq * p.act_per_bh;
  PSA_REQUIRE(n_active < (1ll << 28), PSA_ERR_UNSUPPORTED, "psa_estimate_xattn: too many output tiles");
  p.n_active = (int)n_active;
  p.per_xcd = (int)((n_active + 7) / 8);
  dim3 grid((unsigned)(p.per_xcd * 8));
  const size_t shmem = X_BUFS * (size_t)X_STAGE;
  auto launch = [&](auto kern) -> int {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess) return PSA_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, grid, dim3(X_WAVES * 64), shmem, st, p);
    return PSA_OK;
  };
  int rc = rb == 8 ? launch(psa_xattn_gemm_kernel<3>) : rb == 16 ? launch(psa_xattn_gemm_kernel<4>) : launch(psa_xattn_gemm_kernel<5>);
  PSA_REQUIRE(rc == PSA_OK, rc, "psa_estimate_xattn: cannot reserve LDS");
  rc = psa_check_launch("psa_estimate_xattn (contraction)");
  if (rc != PSA_OK) return rc;
  // the pairs of one q-block: NB * rb * 8 bytes; cached in LDS when that leaves room for several workgroups per CU
  const size_t cache_bytes = (size_t)p.NB * ((size_t)1 << p.rb_log2) * 8;
  const int cached = cache_bytes <= 48 * 1024 ? 1 : 0;
  hipLaunchKernelGGL(psa_xattn_reduce_kernel, dim3((unsigned)p.out_rows, (unsigned)(B * Hq)), dim3(256), cached ? cache_bytes : 0, st, p, cached);
  return psa_check_launch("psa_estimate_xattn (reduction)");
}
