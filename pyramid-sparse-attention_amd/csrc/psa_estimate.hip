// Sampled block-importance estimator.
//
//   R[r, j]  = max_{c in key group j} (q_r . k_c) * scale * log2(e)
//   m[r]     = max_j R[r, j]
//   Po[i, j] = max_{r in query group i} exp2(R[r, j] - m[r]);   Po[i, :] /= sum_j Po[i, j]
//
// Kernel 1 (MFMA-bound, 2*Ms*Ns*D flops): a dense bf16 / fp16 contraction of the sampled query rows with the
// sampled key rows, both gathered straight from the un-sampled Q / K through the per-head offset
// tables.  One workgroup = 4 waves x 64 sampled query rows (two B-operand sets per wave share every K
// operand read from LDS); the waves share K tiles of 64 sampled keys, copied by global_load_lds into
// double-buffered LDS (one barrier per tile).  The key range is cut into 1, 2 or 4 shares (grid z) so that
// the launch fills the chip; the row maxima of the shares are combined by kernel 2.  As in the forward
// kernel the transposed product S^T = K Q^T is computed, so a lane holds 16 keys of one query row and a
// key-group maximum is an in-lane v_max3 chain plus a half-wave exchange shared by two key groups.  The group
// maxima go to an fp32 workspace laid out [key group][query row] (coalesced stores, issued one tile late).
// Kernel 2 (HBM-bound, reads the workspace once): per (query group, key group) the maximum over the
// group's rows of R - m, exp2, row sum in a fixed order, normalisation.
#include "psa_common.h"
#include "psa_level_map_row.h"
#include "psa_tiles.h"

namespace {

constexpr int TK = 64;
constexpr int EST_MAX_KSPLIT = 4;

struct EstParams {
  const uint16_t *q, *k;  // bf16 or fp16 (the kernel's element trait says which)
  int dtype;
  int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl;
  const int32_t *off_q, *off_k;
  const int32_t* q_index;  // optional: the sampled query position i is source row q_index[i] (token re-ordering)
  float* rt;   // workspace: R^T [B*Hq][n_d][Ms_pad]
  float* mrow; // workspace: m [B*Hq][ksplit][Ms_pad]: row maxima over each share of the keys
  int ksplit;  // the key range is cut into ksplit shares (grid z) to even out the load
  float* scores;
  int Hq, Hkv, Lq, Lk;
  int bm, bn, keep_m_log2, keep_n_log2;
  int Ms, Ns, Ms_pad, Ns_pad;  // real sampled rows / keys, padded counts (multiples of 64)
  int n_d;                     // key groups incl. padding groups
  int out_rows, out_cols;
  float qk_scale;
};

__device__ __forceinline__ int sampled_src(int r, int n_real, int keep_log2, int block, const int32_t* off, int L) {
  r = r < n_real ? r : n_real - 1;
  const int grp = r >> keep_log2, e = r & ((1 << keep_log2) - 1);
  const int src = grp * block + (off ? off[e] : e);
  return src < L ? src : L - 1;
}

// 64 sampled query rows per wave (two B-operand sets share every K operand fetched from LDS) and K tiles
// copied from global memory straight into LDS, double buffered, in the padded + swizzled tile layout of
// psa_tiles.h (shared with the attention kernels): the 128-bit operand reads are bank-conflict free and their
// addresses are lane base + immediate.
//
// Three waves share a SIMD, and whatever a wave executes outside its MFMA stream (copy addresses, the group
// maxima, store addresses) advances slowly while the other two stream MFMAs: that part is kept to a few dozen
// vector instructions per tile.  The copy and store addresses are a per-tile scalar base plus a lane offset
// computed once; the two 32-key chunks of a tile are multiplied one after the other, so that the maxima of
// the first chunk are taken in the shadow of the second chunk's MFMAs; and one half-wave exchange serves two
// key groups (lanes 0-31 keep the maximum of the even group, lanes 32-63 that of the odd one).
constexpr int E_STAGES = 2;

// piece k (0..7) of the in-lane maxima of one 32-key chunk: NV = 1 << GPC values, 8 instructions in all.
// Register i of the chunk holds key (i / 4) * 8 + 4 * (lane / 32) + i % 4, so the keys of an 8-key octet are
// registers 4o..4o+3 of both half-waves.
template <int GPC>
__device__ __forceinline__ void chunk_max_piece(const f32x16& sc, float (&val)[1 << GPC], float (&tmp)[3], int k) {
  if constexpr (GPC == 0) {
    if (k == 0) val[0] = max3f(sc[0], sc[1], sc[2]);
    else if (k < 7) val[0] = max3f(val[0], sc[2 * k + 1], sc[2 * k + 2]);
    else val[0] = fmaxf(val[0], sc[15]);
  } else if constexpr (GPC == 1) {
    const int o = k >> 2, j = k & 3;
    if (j == 0) tmp[0] = max3f(sc[8 * o], sc[8 * o + 1], sc[8 * o + 2]);
    else if (j == 1) tmp[1] = max3f(sc[8 * o + 3], sc[8 * o + 4], sc[8 * o + 5]);
    else if (j == 2) tmp[2] = fmaxf(sc[8 * o + 6], sc[8 * o + 7]);
    else val[o] = max3f(tmp[0], tmp[1], tmp[2]);
  } else {
    const int o = k >> 1;
    if ((k & 1) == 0) tmp[0] = max3f(sc[4 * o], sc[4 * o + 1], sc[4 * o + 2]);
    else val[o] = fmaxf(tmp[0], sc[4 * o + 3]);
  }
}

template <int D, int GPC, class ET>
__global__ __launch_bounds__(256, 2) void psa_est_gemm_lds_kernel(EstParams p) {
  using x8 = typename ET::x8;
  using G = psa_tiles::LtGeom<D>;
  constexpr int KK = D / 16, RS = 2;  // RS sets of 32 query rows per wave
  constexpr int E_TILE = G::TILE, E_ISTR = psa_tiles::LT_ISTR, RPL = G::RPL;
  constexpr int NV = 1 << GPC;        // key groups per 32-key chunk = registers of group maxima per row set and tile
  constexpr int PPS = 8 / KK;         // pieces of the first chunk's maxima per k-step of the second chunk
  static_assert(8 % KK == 0 && PPS >= 1, "the maxima of a chunk are 8 pieces");
  __shared__ __align__(16) unsigned char smem[E_STAGES * E_TILE];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;
  const int bh = blockIdx.y;
  const int h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);
  const int keep_m = 1 << p.keep_m_log2;
  constexpr int kn_log2 = 5 - GPC, keep_n = 1 << kn_log2;

  // Q fragments: lane holds Q[row l32 of set rs][16*kk + 8*hh .. +8]
  const int row0 = blockIdx.x * (4 * 32 * RS) + wave * (32 * RS);
  x8 qf[RS][KK];
  {
    const int32_t* oq = p.off_q ? p.off_q + (int64_t)bh * keep_m : nullptr;
#pragma unroll
    for (int rs = 0; rs < RS; ++rs) {
      int src = sampled_src(row0 + rs * 32 + l32, p.Ms, p.keep_m_log2, p.bm, oq, p.Lq);
      if (p.q_index != nullptr) src = clamp_row(p.q_index[src], p.Lq);
      const uint16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)src * p.q_sl + hh * 8;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) qf[rs][kk] = *(const x8*)(qp + kk * 16);
    }
  }

  const char* kb = (const char*)(p.k + b * p.k_sb + hk * p.k_sh);
  const uint32_t kstrb = (uint32_t)p.k_sl * 2u;
  const int32_t* ok = p.off_k ? p.off_k + ((int64_t)b * p.Hkv + hk) * keep_n : nullptr;
  const int Ns = p.Ns, Lk = p.Lk, bn = p.bn;

  // fetch: wave w copies the 16-row group w of a tile, one block per instruction.  A tile of 64 sampled keys
  // spans 64 / keep_n whole key groups, so the source row of a tile slot is t * (64 / keep_n) * block_n plus a
  // per-lane constant: the copies of a tile inside the sequence cost no vector arithmetic.
  const uint32_t f_chunk = psa_tiles::lt_fetch_chunk<D>(lane);
  const int slot0 = wave * 16 + psa_tiles::lt_fetch_row<D>(lane);  // first of this lane's consecutive tile slots
  int my_off[RPL];
  uint32_t c_off[RPL];
#pragma unroll
  for (int n = 0; n < RPL; ++n) {
    const int e = (slot0 + n) & (keep_n - 1);
    my_off[n] = ok ? ok[e] : e;
    c_off[n] = (uint32_t)((slot0 >> kn_log2) * bn + my_off[n]) * kstrb + f_chunk;
  }
  const int last_off = ok ? ok[keep_n - 1] : keep_n - 1;
  const uint64_t tile_step = (uint64_t)((TK >> kn_log2) * bn) * kstrb;  // bytes between the key groups of consecutive tiles
  auto issue_tile = [&](int t, int stage) __attribute__((always_inline)) {
    const bool inside = (t + 1) * TK <= Ns && ((((t + 1) * TK - 1) >> kn_log2) + 1) * bn <= Lk;  // uniform
    if (inside) {
      const char* tb = kb + (uint64_t)t * tile_step;
#pragma unroll
      for (int n = 0; n < RPL; ++n)
        psa_tiles::lds_copy16(tb, c_off[n], psa_tiles::lds_addr_of(smem + stage * E_TILE + (wave * RPL + n) * E_ISTR));
    } else {
      // padding keys replicate the last sampled key (Ns is a multiple of keep_n, so that is entry keep_n - 1 of
      // the offset table: looked up once, before the loop - a global load in here would make the compiler wait
      // for every copy in flight before each copy); rows past the sequence end clamp to its last row
      const int r0 = t * TK + slot0;
      const int grp_row = (r0 >> kn_log2) * bn;
#pragma unroll
      for (int n = 0; n < RPL; ++n) {
        int src = grp_row + my_off[n];
        if (r0 + n >= Ns) src = ((Ns - 1) >> kn_log2) * bn + last_off;
        src = src < Lk ? src : Lk - 1;
        psa_tiles::lds_copy16(kb, (uint32_t)src * kstrb + f_chunk, psa_tiles::lds_addr_of(smem + stage * E_TILE + (wave * RPL + n) * E_ISTR));
      }
    }
  };
  // K operand of k-step kk for tile slots l32 and l32 + 32: k_off[kk & 1] + 64 * (kk >> 1) (+ G::HALF)
  uint32_t k_off[2];
  psa_tiles::lt_row_operand<D>(l32, hh, k_off);

  const int T = p.Ns_pad / TK;
  // workspace rows of this wave: uniform base + lane offset (lanes 32-63 store for the odd key group of a pair)
  const int64_t rts = p.Ms_pad;
  float* const rt_u = p.rt + (int64_t)bh * p.n_d * rts + row0;
  const uint32_t st_off = (uint32_t)hh * (uint32_t)rts + (uint32_t)l32;
  float m_run[RS];
#pragma unroll
  for (int rs = 0; rs < RS; ++rs) m_run[rs] = -INFINITY;
  const float qk_scale = p.qk_scale;

  // group maxima of the previous tile, written one tile late so that the stores' latency hides behind the MFMAs:
  // register pr of a row set holds key groups 2 * pr (lanes 0-31) and 2 * pr + 1 (lanes 32-63) of the tile
  float pend[RS][NV];
  auto flush = [&](int tp) __attribute__((always_inline)) {
    float* const tb = rt_u + (int64_t)tp * (2 * NV) * rts;
#pragma unroll
    for (int rs = 0; rs < RS; ++rs)
#pragma unroll
      for (int pr = 0; pr < NV; ++pr) (tb + (int64_t)(2 * pr) * rts + rs * 32)[st_off] = pend[rs][pr];
  };

  // this workgroup's share of the key tiles
  const int ks = blockIdx.z;
  const int t_begin = (int)((int64_t)T * ks / p.ksplit), t_end = (int)((int64_t)T * (ks + 1) / p.ksplit);
  issue_tile(t_begin, t_begin & 1);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int t = t_begin; t < t_end; ++t) {
    // invariant: stage t&1 holds tile t and every wave is done with the other stage
    if (t + 1 < t_end) issue_tile(t + 1, (t + 1) & 1);
    if (t > t_begin) flush(t - 1);

    PSA_LDS(unsigned char) Ks = (PSA_LDS(unsigned char))(smem) + (t & 1) * E_TILE;
    // step i = chunk c * KK + k-step kk; its operand is requested two steps (four MFMAs) ahead
    auto kread = [&](int i) __attribute__((always_inline)) {
      const int c = i / KK, kk = i % KK;
      return *(PSA_LDS(const x8))(Ks + k_off[kk & 1] + (kk >> 1) * 64 + c * G::HALF);
    };
    f32x16 s[RS][2];
    float val[RS][2][NV], tmp[RS][3];
    x8 ka[3];
    ka[0] = kread(0);
    ka[1] = kread(1);
#pragma unroll
    for (int i = 0; i < 2 * KK; ++i) {
      const int c = i / KK, kk = i % KK;
      if (i + 2 < 2 * KK) ka[(i + 2) % 3] = kread(i + 2);
#pragma unroll
      for (int rs = 0; rs < RS; ++rs) s[rs][c] = ET::mfma(ka[i % 3], qf[rs][kk], kk == 0 ? zero16 : s[rs][c]);
      if (c == 1) {
        __builtin_amdgcn_sched_barrier(0);  // after this step's MFMAs: the first piece waits for chunk 0's last results
#pragma unroll
        for (int k = kk * PPS; k < (kk + 1) * PPS; ++k)
#pragma unroll
          for (int rs = 0; rs < RS; ++rs) chunk_max_piece<GPC>(s[rs][0], val[rs][0], tmp[rs], k);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
#pragma unroll
      for (int rs = 0; rs < RS; ++rs) chunk_max_piece<GPC>(s[rs][1], val[rs][1], tmp[rs], k);
#pragma unroll
    for (int rs = 0; rs < RS; ++rs)
#pragma unroll
      for (int pr = 0; pr < NV; ++pr) {
        // the tile's 2 * NV key groups in order: chunk 0's, then chunk 1's
        const int e0 = 2 * pr, e1 = 2 * pr + 1;
        const float v = half_wave_max_pair(val[rs][e0 / NV][e0 % NV], val[rs][e1 / NV][e1 % NV]) * qk_scale;
        m_run[rs] = fmaxf(m_run[rs], v);
        pend[rs][pr] = v;
      }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // the copies of tile t+1 (and the stores of tile t-1) were issued a tile ago
    __syncthreads();
  }
  if (t_end > t_begin) flush(t_end - 1);
#pragma unroll
  for (int rs = 0; rs < RS; ++rs) {
    const float m = half_wave_max(m_run[rs]);  // the halves saw different key groups
    if (hh == 0) p.mrow[((int64_t)bh * p.ksplit + ks) * p.Ms_pad + row0 + rs * 32 + l32] = m;
  }
}

// one workgroup per (b, h, query group): Po[i, :] from R^T and m.
// A lane reads 4 consecutive rows (16 bytes) of one key group, keep_m/4 neighbouring lanes cover the group's
// rows (one contiguous run of the workspace), a wave 256/keep_m key groups per load; the maximum over the
// group's rows is an in-lane maximum plus a butterfly over those lanes.
// Leaves the un-normalised row in s_e[0 .. n_d) and returns its sum (fixed summation order); 256 threads.
// The contraction for fp32 tensors: fp32 operands and arithmetic (vector FMAs), the same workspace contents as the
// MFMA kernel (group maxima R^T [key group][query row] in log2 units, row maxima; one share of the keys).  One
// workgroup per 64 sampled query rows; key tiles of 64 sampled keys go to LDS channel-major; thread (t / 16, t % 16)
// owns rows ty + 16 i and keys tx + 16 j of a tile, the tile's logits pass through LDS for the group maxima.
template <int D, int RI>
__global__ __launch_bounds__(256) void psa_est_gemm_f32_kernel(EstParams p) {
  constexpr int QR = 16 * RI;  // sampled query rows per workgroup
  constexpr int DP = D + 1, KP = TK + 1;
  extern __shared__ __align__(16) unsigned char smem_f32[];
  float* Qs = (float*)smem_f32;  // [QR][DP]
  float* Kt = Qs + QR * DP;      // [D][KP]
  float* Ss = Kt + D * KP;       // [QR][KP]
  const float* qg = (const float*)p.q;
  const float* kg = (const float*)p.k;
  const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
  const int bh = blockIdx.y, h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);
  const int row0 = blockIdx.x * QR;
  const int32_t* oq = p.off_q ? p.off_q + (int64_t)bh * (1 << p.keep_m_log2) : nullptr;
  const int32_t* ok = p.off_k ? p.off_k + ((int64_t)b * p.Hkv + hk) * (1 << p.keep_n_log2) : nullptr;
  for (int u = tid; u < QR * (D / 4); u += 256) {
    const int r = u / (D / 4), c4 = u % (D / 4);
    int src = sampled_src(row0 + r, p.Ms, p.keep_m_log2, p.bm, oq, p.Lq);
    if (p.q_index != nullptr) src = clamp_row(p.q_index[src], p.Lq);
    const f32x4 x = *(const f32x4*)(qg + b * p.q_sb + h * p.q_sh + (int64_t)src * p.q_sl + c4 * 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) Qs[r * DP + c4 * 4 + e] = x[e];
  }
  const int keep_n = 1 << p.keep_n_log2, gpt = TK >> p.keep_n_log2;  // key groups per tile
  float m_run = -INFINITY;  // of row (tid / 4) for the threads that write group maxima, see below
  float* rt = p.rt + (int64_t)bh * p.n_d * p.Ms_pad + row0;
  const float* kb = kg + b * p.k_sb + hk * p.k_sh;
  for (int t0 = 0; t0 < p.Ns_pad; t0 += TK) {
    __syncthreads();
    for (int u = tid; u < TK * (D / 4); u += 256) {
      const int r = u / (D / 4), c4 = u % (D / 4);
      const int src = sampled_src(t0 + r, p.Ns, p.keep_n_log2, p.bn, ok, p.Lk);
      const f32x4 x = *(const f32x4*)(kb + (int64_t)src * p.k_sl + c4 * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) Kt[(c4 * 4 + e) * KP + r] = x[e];
    }
    __syncthreads();
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
#pragma unroll
    for (int i = 0; i < RI; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) Ss[(ty + 16 * i) * KP + tx + 16 * j] = s[i][j] * p.qk_scale;
    __syncthreads();
    // group maxima: (row, group) pairs, row fastest so that the stores are coalesced
    for (int u = tid; u < QR * gpt; u += 256) {
      const int r = u % QR, g = u / QR;
      float mx = -INFINITY;
      for (int c = 0; c < keep_n; ++c) mx = fmaxf(mx, Ss[r * KP + g * keep_n + c]);
      rt[(int64_t)((t0 >> p.keep_n_log2) + g) * p.Ms_pad + r] = mx;
    }
    // row maxima: thread t < QR keeps the maximum of row t
    if (tid < QR) {
      float mx = m_run;
      for (int c = 0; c < TK; ++c) mx = fmaxf(mx, Ss[tid * KP + c]);
      m_run = mx;
    }
  }
  if (tid < QR) p.mrow[(int64_t)bh * p.Ms_pad + row0 + tid] = m_run;
}

__device__ __forceinline__ float est_reduce_row(const EstParams& p, float* s_e, float* s_part, int i, int bh) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lpg_log2 = p.keep_m_log2 - 2;            // lanes per key group
  const int quad = lane & ((1 << lpg_log2) - 1), sub = lane >> lpg_log2;
  const int per_iter = 64 >> lpg_log2;               // key groups per wave iteration
  const int r0 = (i << p.keep_m_log2) + quad * 4;
  f32x4 m = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
  for (int ks = 0; ks < p.ksplit; ++ks) {
    const f32x4 x = *(const f32x4*)(p.mrow + ((int64_t)bh * p.ksplit + ks) * p.Ms_pad + r0);
#pragma unroll
    for (int e = 0; e < 4; ++e) m[e] = fmaxf(m[e], x[e]);
  }
  const float* rt = p.rt + (int64_t)bh * p.n_d * p.Ms_pad + r0;
  for (int j0 = wave * per_iter; j0 < p.n_d; j0 += 4 * per_iter) {
    const int j = j0 + sub;
    float v = -INFINITY;
    if (j < p.n_d) {
      const f32x4 x = *(const f32x4*)(rt + (int64_t)j * p.Ms_pad);
      v = fmaxf(fmaxf(x[0] - m[0], x[1] - m[1]), fmaxf(x[2] - m[2], x[3] - m[3]));
    }
    for (int o = (1 << lpg_log2) >> 1; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    if (quad == 0 && j < p.n_d) s_e[j] = fast_exp2(v);
  }
  __syncthreads();
  // row sum in a fixed order: per-thread strided partials, wave butterfly, four wave partials
  float part = 0.f;
  for (int j = tid; j < p.n_d; j += 256) part += s_e[j];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
  if (lane == 0) s_part[wave] = part;
  __syncthreads();
  return (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
}

__global__ __launch_bounds__(256) void psa_est_reduce_kernel(EstParams p) {
  extern __shared__ float s_e[];  // [n_d] un-normalised Po row
  __shared__ float s_part[4];
  const int i = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x;
  const float total = est_reduce_row(p, s_e, s_part, i, bh);
  float* dst = p.scores + ((int64_t)bh * p.out_rows + i) * p.out_cols;
  for (int j = tid; j < p.out_cols; j += 256) dst[j] = s_e[j] / total;
}

// The same, followed by the level map of the row while its scores are still in LDS: the workspace pass (HBM) of
// one workgroup overlaps the sorting (VALU / LDS) of the others, and a launch and a round trip of the scores
// through memory go away.  LDS: [level-map scratch: lm_bytes][n_d floats].  p.scores may be null.
__global__ __launch_bounds__(256) void psa_est_reduce_map_kernel(EstParams p, LevelMapParams lp, int lm_bytes) {
  extern __shared__ __align__(16) unsigned char smem_rm[];
  __shared__ float s_part[4];
  __shared__ int s_cnt[PSA_MAX_LEVEL_ITEMS];
  __shared__ int s_iv[PSA_MAX_LEVEL_ITEMS][2];
  float* s_e = (float*)(smem_rm + lm_bytes);
  const int i = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x;
  const float total = est_reduce_row(p, s_e, s_part, i, bh);
  const int64_t row = (int64_t)bh * p.out_rows + i;
  for (int j = tid; j < p.out_cols; j += 256) {
    const float v = s_e[j] / total;
    s_e[j] = v;
    if (p.scores) p.scores[row * p.out_cols + j] = v;
  }
  __syncthreads();
  level_map_row(lp, s_e, row, smem_rm, s_cnt, s_iv, tid, 256);
}

template <int D>
int launch_est(EstParams& p, int B, hipStream_t stream, const LevelMapParams* lp, bool* map_done) {
  const int rows_needed = p.out_rows << p.keep_m_log2;
  dim3 grid((unsigned)((rows_needed + 255) / 256), (unsigned)(B * p.Hq));
  // 256-row workgroups: cut the key range until about 3 workgroups per CU exist (the kernel's occupancy),
  // keeping at least 8 key tiles per share
  p.ksplit = 1;
  const int64_t wgs = (int64_t)grid.x * B * p.Hq;
  const int tiles = p.Ns_pad / TK;
  while (p.ksplit < EST_MAX_KSPLIT && wgs * p.ksplit < 3 * 256 && tiles / (p.ksplit * 2) >= 8) p.ksplit *= 2;
  grid.z = (unsigned)p.ksplit;
  if (p.dtype == PSA_DTYPE_F32) {
    p.ksplit = 1;
    // 64 sampled rows per workgroup, or 32 / 16 while the launch would have fewer than two workgroups per CU
    auto go = [&](auto ri_c) -> int {
      constexpr int RI = decltype(ri_c)::value, QR = 16 * RI;
      const size_t shmem = (size_t)(QR * (D + 1) + D * (TK + 1) + QR * (TK + 1)) * sizeof(float);
      if (hipFuncSetAttribute((const void*)psa_est_gemm_f32_kernel<D, RI>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess)
        return PSA_ERR_LAUNCH;
      hipLaunchKernelGGL((psa_est_gemm_f32_kernel<D, RI>), dim3((unsigned)(p.Ms_pad / QR), (unsigned)(B * p.Hq)), dim3(256), shmem, stream, p);
      return PSA_OK;
    };
    int ri = 4;
    while (ri > 1 && (int64_t)(p.Ms_pad / (16 * ri)) * B * p.Hq < 512) ri >>= 1;
    const int rc32 = ri == 4 ? go(std::integral_constant<int, 4>{}) : ri == 2 ? go(std::integral_constant<int, 2>{}) : go(std::integral_constant<int, 1>{});
    if (rc32 != PSA_OK) return rc32;
  }
  psa_dispatch16(p.dtype, [&](auto et) {
    using ET = decltype(et);
    switch (p.keep_n_log2) {
      case 5: hipLaunchKernelGGL((psa_est_gemm_lds_kernel<D, 0, ET>), grid, dim3(256), 0, stream, p); break;
      case 4: hipLaunchKernelGGL((psa_est_gemm_lds_kernel<D, 1, ET>), grid, dim3(256), 0, stream, p); break;
      default: hipLaunchKernelGGL((psa_est_gemm_lds_kernel<D, 2, ET>), grid, dim3(256), 0, stream, p); break;
    }
  });
  const int rc = psa_check_launch("psa_estimate_sampled (contraction)");
  if (rc != PSA_OK) return rc;
  const dim3 rgrid((unsigned)p.out_rows, (unsigned)(B * p.Hq));
  if (lp == nullptr) {
    hipLaunchKernelGGL(psa_est_reduce_kernel, rgrid, dim3(256), (size_t)p.n_d * sizeof(float), stream, p);
    return psa_check_launch("psa_estimate_sampled (reduction)");
  }
  const size_t lm_bytes = (level_map_lds_bytes(lp->Nk) + 15) & ~(size_t)15;
  const size_t shmem = lm_bytes + (size_t)p.n_d * sizeof(float);
  if (shmem > 150 * 1024) {
    // very wide maps: the row of scores and the level-map scratch do not fit into LDS together - two kernels
    PSA_REQUIRE(p.scores != nullptr, PSA_ERR_ARG, "psa_estimate_sampled_map: maps of %d columns need the scores buffer", lp->Nk);
    hipLaunchKernelGGL(psa_est_reduce_kernel, rgrid, dim3(256), (size_t)p.n_d * sizeof(float), stream, p);
    *map_done = false;  // the caller finishes with psa_level_map on the scores
    return psa_check_launch("psa_estimate_sampled_map (reduction)");
  }
  if (shmem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)psa_est_reduce_map_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    PSA_REQUIRE(e == hipSuccess, PSA_ERR_LAUNCH, "psa_estimate_sampled_map: cannot reserve %zu bytes of LDS", shmem);
  }
  hipLaunchKernelGGL(psa_est_reduce_map_kernel, rgrid, dim3(256), shmem, stream, p, *lp, (int)lm_bytes);
  *map_done = true;
  return psa_check_launch("psa_estimate_sampled_map (reduction + level map)");
}

struct EstGeom {
  int Ms, Ns, Ms_pad, Ns_pad, m_d, n_d;
};
EstGeom est_geom(int Lq, int Lk, int block_m, int block_n, int keep_m, int keep_n) {
  EstGeom g;
  const int Mq = (Lq + block_m - 1) / block_m, Nk = (Lk + block_n - 1) / block_n;
  g.Ms = Mq * keep_m;
  g.Ns = Nk * keep_n;
  // the contraction kernels work on 128 or 256 query rows per workgroup; the reference pads to 64
  g.Ms_pad = (g.Ms + 255) / 256 * 256;
  g.Ns_pad = (g.Ns + 63) / 64 * 64;
  g.m_d = ((g.Ms + 63) / 64 * 64) / keep_m;
  g.n_d = g.Ns_pad / keep_n;
  return g;
}

}  // namespace

extern "C" int64_t psa_estimate_workspace_bytes(int B, int Hq, int Lq, int Lk, int block_m, int block_n, int keep_m, int keep_n) {
  if (B <= 0 || Hq <= 0 || Lq <= 0 || Lk <= 0 || block_m <= 0 || block_n <= 0 || keep_m <= 0 || keep_n <= 0) return 0;
  const EstGeom g = est_geom(Lq, Lk, block_m, block_n, keep_m, keep_n);
  return (int64_t)B * Hq * ((int64_t)g.n_d + EST_MAX_KSPLIT) * g.Ms_pad * (int64_t)sizeof(float);
}

namespace {
int est_run(psa_tensor4 q, psa_tensor4 k, const int32_t* off_q, const int32_t* off_k, const int32_t* q_index, float* scores,
            void* workspace, int B, int Hq,
            int Hkv, int Lq, int Lk, int D, int block_m, int block_n, int keep_m, int keep_n, float sm_scale, int out_rows,
            int out_cols, LevelMapParams* lp, bool* map_done, psa_stream_t stream) {
  PSA_REQUIRE(q.ptr && k.ptr && (scores || lp) && workspace, PSA_ERR_ARG, "psa_estimate_sampled: null pointer");
  PSA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Lq > 0 && Lk > 0, PSA_ERR_ARG, "psa_estimate_sampled: sizes must be positive");
  PSA_REQUIRE(Hq % Hkv == 0, PSA_ERR_ARG, "psa_estimate_sampled: Hq must be a multiple of Hkv");
  PSA_REQUIRE((int64_t)B * Hq <= 65535, PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: B*Hq too large");
  PSA_REQUIRE(q.dtype == k.dtype, PSA_ERR_ARG, "psa_estimate_sampled: q and k must share one element type");
  PSA_REQUIRE(q.dtype == PSA_DTYPE_BF16 || q.dtype == PSA_DTYPE_F16 || q.dtype == PSA_DTYPE_F32, PSA_ERR_ARG,
              "psa_estimate_sampled: unknown element type %d", q.dtype);
  PSA_REQUIRE(D == 64 || D == 128, PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: head dim %d not in {64, 128}", D);
  PSA_REQUIRE(keep_m == 8 || keep_m == 16 || keep_m == 32, PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: keep_m=%d not in {8,16,32}", keep_m);
  PSA_REQUIRE(keep_n == 8 || keep_n == 16 || keep_n == 32, PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: keep_n=%d not in {8,16,32}", keep_n);
  PSA_REQUIRE(block_m >= keep_m && block_n >= keep_n, PSA_ERR_ARG, "psa_estimate_sampled: block smaller than keep");
  PSA_REQUIRE(((uintptr_t)q.ptr % 16 == 0) && ((uintptr_t)k.ptr % 16 == 0) && q.stride_l % 8 == 0 && k.stride_l % 8 == 0 &&
                  q.stride_h % 8 == 0 && k.stride_h % 8 == 0 && q.stride_b % 8 == 0 && k.stride_b % 8 == 0,
              PSA_ERR_UNSUPPORTED, "psa_estimate_sampled: tensors must be 16-byte aligned with strides multiple of 8");
  PSA_REQUIRE((int64_t)Lk * k.stride_l * 2 < (1ll << 32), PSA_ERR_UNSUPPORTED,
              "psa_estimate_sampled: one (batch, head) slice of K must span less than 4 GiB");
  const EstGeom g = est_geom(Lq, Lk, block_m, block_n, keep_m, keep_n);
  EstParams p;
  p.q = (const uint16_t*)q.ptr; p.k = (const uint16_t*)k.ptr; p.dtype = q.dtype;
  p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sl = q.stride_l;
  p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sl = k.stride_l;
  p.off_q = off_q; p.off_k = off_k; p.q_index = q_index; p.scores = scores;
  p.Hq = Hq; p.Hkv = Hkv; p.Lq = Lq; p.Lk = Lk; p.bm = block_m; p.bn = block_n;
  p.keep_m_log2 = psa_ilog2(keep_m); p.keep_n_log2 = psa_ilog2(keep_n);
  p.Ms = g.Ms; p.Ns = g.Ns; p.Ms_pad = g.Ms_pad; p.Ns_pad = g.Ns_pad; p.n_d = g.n_d;
  PSA_REQUIRE(out_rows > 0 && out_rows <= g.m_d && out_cols > 0 && out_cols <= g.n_d, PSA_ERR_ARG,
              "psa_estimate_sampled: out_rows/out_cols exceed %d x %d", g.m_d, g.n_d);
  p.out_rows = out_rows; p.out_cols = out_cols;
  p.qk_scale = sm_scale * 1.44269504f;
  p.rt = (float*)workspace;
  p.mrow = p.rt + (int64_t)B * Hq * g.n_d * g.Ms_pad;
  if (lp != nullptr) {
    PSA_REQUIRE(lp->Nk == out_cols, PSA_ERR_ARG, "psa_estimate_sampled_map: the map has %d columns, the scores %d", lp->Nk, out_cols);
    lp->scores = nullptr;
  }
  return D == 128 ? launch_est<128>(p, B, (hipStream_t)stream, lp, map_done) : launch_est<64>(p, B, (hipStream_t)stream, lp, map_done);
}
}  // namespace

extern "C" int psa_estimate_sampled(psa_tensor4 q, psa_tensor4 k, const int32_t* off_q, const int32_t* off_k, float* scores,
                                    void* workspace, int B, int Hq, int Hkv, int Lq, int Lk, int D, int block_m, int block_n,
                                    int keep_m, int keep_n, float sm_scale, int out_rows, int out_cols, psa_stream_t stream) {
  PSA_REQUIRE(scores, PSA_ERR_ARG, "psa_estimate_sampled: null pointer");
  bool unused = false;
  return est_run(q, k, off_q, off_k, nullptr, scores, workspace, B, Hq, Hkv, Lq, Lk, D, block_m, block_n, keep_m, keep_n, sm_scale,
                 out_rows, out_cols, nullptr, &unused, stream);
}

extern "C" int psa_estimate_sampled_indexed(psa_tensor4 q, const int32_t* q_index, psa_tensor4 k, const int32_t* off_q,
                                            const int32_t* off_k, float* scores, void* workspace, int B, int Hq, int Hkv, int Lq,
                                            int Lk, int D, int block_m, int block_n, int keep_m, int keep_n, float sm_scale,
                                            int out_rows, int out_cols, psa_stream_t stream) {
  PSA_REQUIRE(scores && q_index, PSA_ERR_ARG, "psa_estimate_sampled_indexed: null pointer");
  bool unused = false;
  return est_run(q, k, off_q, off_k, q_index, scores, workspace, B, Hq, Hkv, Lq, Lk, D, block_m, block_n, keep_m, keep_n, sm_scale,
                 out_rows, out_cols, nullptr, &unused, stream);
}

static int est_map_run(psa_tensor4 q, psa_tensor4 k, const int32_t* off_q, const int32_t* off_k, const int32_t* q_index, float* scores,
                       void* workspace, int B, int Hq, int Hkv, int Lq, int Lk, int D, int block_m, int block_n,
                       int keep_m, int keep_n, float sm_scale, int out_rows, int out_cols, void* map_out,
                       int map_elem_bytes, int mode, int n_items, const int32_t* item_level, const double* item_hi,
                       int align_div, int text_blocks, double min_full_attn_ratio, psa_stream_t stream) {
  PSA_REQUIRE(map_out, PSA_ERR_ARG, "psa_estimate_sampled_map: null pointer");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_estimate_sampled_map: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(out_cols > 0, PSA_ERR_ARG, "psa_estimate_sampled_map: out_cols must be positive");
  LevelMapParams lp;
  const int rc = level_map_fill_params(lp, out_cols, mode, n_items, item_level, item_hi, align_div, text_blocks, min_full_attn_ratio);
  if (rc != PSA_OK) return rc;
  lp.map_out = map_out; lp.map_elem = map_elem_bytes;
  bool map_done = false;
  const int rc2 = est_run(q, k, off_q, off_k, q_index, scores, workspace, B, Hq, Hkv, Lq, Lk, D, block_m, block_n, keep_m, keep_n,
                          sm_scale, out_rows, out_cols, &lp, &map_done, stream);
  if (rc2 != PSA_OK || map_done) return rc2;
  return psa_level_map(scores, map_out, map_elem_bytes, nullptr, (int64_t)B * Hq * out_rows, out_cols, mode, n_items, item_level, item_hi,
                       align_div, text_blocks, min_full_attn_ratio, stream);
}

extern "C" int psa_estimate_sampled_map(psa_tensor4 q, psa_tensor4 k, const int32_t* off_q, const int32_t* off_k, float* scores,
                                        void* workspace, int B, int Hq, int Hkv, int Lq, int Lk, int D, int block_m, int block_n,
                                        int keep_m, int keep_n, float sm_scale, int out_rows, int out_cols, void* map_out,
                                        int map_elem_bytes, int mode, int n_items, const int32_t* item_level, const double* item_hi,
                                        int align_div, int text_blocks, double min_full_attn_ratio, psa_stream_t stream) {
  return est_map_run(q, k, off_q, off_k, nullptr, scores, workspace, B, Hq, Hkv, Lq, Lk, D, block_m, block_n, keep_m, keep_n, sm_scale,
                     out_rows, out_cols, map_out, map_elem_bytes, mode, n_items, item_level, item_hi, align_div, text_blocks,
                     min_full_attn_ratio, stream);
}

extern "C" int psa_estimate_sampled_map_indexed(psa_tensor4 q, const int32_t* q_index, psa_tensor4 k, const int32_t* off_q,
                                                const int32_t* off_k, float* scores, void* workspace, int B, int Hq, int Hkv, int Lq,
                                                int Lk, int D, int block_m, int block_n, int keep_m, int keep_n, float sm_scale,
                                                int out_rows, int out_cols, void* map_out, int map_elem_bytes, int mode, int n_items,
                                                const int32_t* item_level, const double* item_hi, int align_div, int text_blocks,
                                                double min_full_attn_ratio, psa_stream_t stream) {
  PSA_REQUIRE(q_index != nullptr, PSA_ERR_ARG, "psa_estimate_sampled_map_indexed: null index");
  return est_map_run(q, k, off_q, off_k, q_index, scores, workspace, B, Hq, Hkv, Lq, Lk, D, block_m, block_n, keep_m, keep_n, sm_scale,
                     out_rows, out_cols, map_out, map_elem_bytes, mode, n_items, item_level, item_hi, align_div, text_blocks,
                     min_full_attn_ratio, stream);
}
