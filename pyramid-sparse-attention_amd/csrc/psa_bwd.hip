// Backward of the pyramid sparse attention w.r.t. Q, K, V.
//
//   delta_i = sum_d O_id dO_id
//   p_it    = exp2(scale*log2e * q_i.K_l[t] + log2(l) - lse_i*log2e)     (one value per retained pooled key)
//   dV_l[t] += sum_i p_it dO_i          dP_it = dO_i . V_l[t]          dS_it = p_it (dP_it - delta_i)
//   dQ_i    += scale sum_t dS_it K_l[t]                                dK_l[t] += scale sum_i dS_it q_i
//   dK[n]    = dK_1[n] + sum_{l=2,4,8} dK_l[n/l] / l, the part of replicate-pad rows n >= L added to row L-1
//
// Four kernels:
//   psa_bwd_delta_kernel   HBM-bound: delta and lse in log2 units (rows without keys get +inf so p = 0)
//   psa_bwd_dq_lds_kernel  MFMA-bound row walk: the forward's tile schedule; per tile S^T = K Q^T,
//                          dP^T = V dO^T, dQ^T += K^T dS^T on bf16 / fp16 MFMA, operands pooled K/V read directly
//   psa_bwd_dkdv_lds_kernel MFMA-bound column walk: one workgroup per (kv head, kv-block, level slot) keeps its
//                          <= 64 pooled keys in registers and streams the q-blocks that retain this block at
//                          this level; dK_l, dV_l go to an fp32 workspace (every row written exactly once)
//   psa_bwd_unpool_kernel  HBM-bound: sums the levels, spreads pooled gradients, folds the pad tail, -> the tensors' type
#include <type_traits>

#include "psa_tiles.h"
#include "psa_order.h"

namespace {

using namespace psa_tiles;

struct BwdParams {
  const bf16_t *q, *k, *v, *o, *dout;
  int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, o_sb, o_sh, o_sl, do_sb, do_sh, do_sl;
  bf16_t *dq, *dk, *dv;
  int64_t dq_sb, dq_sh, dq_sl, dk_sb, dk_sh, dk_sl, dv_sb, dv_sh, dv_sl;
  const bf16_t *kp, *vp;
  const void* map;
  int map_elem;
  const float* lse;
  float *delta, *lse2;  // workspace [B*Hq*L] each
  float *wk, *wv;       // workspace: per-level fp32 dK / dV, levels back to back: [BHkv, npad >> lv, D]
  int B, Hq, Hkv, L, Mq, Nk, bn_log2, bm;
  int64_t npad;
  float scale, scale_log2;
  int causal;
  int max_tiles;
};

// ------------------------------------------------------------------------------------------------------
// delta and log2-domain lse
// ------------------------------------------------------------------------------------------------------
template <int D, class ET>
__global__ __launch_bounds__(256) void psa_bwd_delta_kernel(BwdParams p) {
  constexpr int LPR = D / 8;  // lanes per row
  const int bh = blockIdx.y, b = bh / p.Hq, h = bh % p.Hq;
  const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
  const int c = threadIdx.x % LPR;
  float acc = 0.f;
  if (row < p.L) {
    const u32x4 ow = *(const u32x4*)(p.o + b * p.o_sb + h * p.o_sh + row * p.o_sl + c * 8);
    const u32x4 dw = *(const u32x4*)(p.dout + b * p.do_sb + h * p.do_sh + row * p.do_sl + c * 8);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc += ET::from_bits(ow[j] & 0xffffu) * ET::from_bits(dw[j] & 0xffffu);
      acc += ET::from_bits(ow[j] >> 16) * ET::from_bits(dw[j] >> 16);
    }
  }
#pragma unroll
  for (int o = LPR / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (c == 0 && row < p.L) {
    const float l = p.lse[(int64_t)bh * p.L + row];
    p.delta[(int64_t)bh * p.L + row] = acc;
    // rows that saw no key have lse = -inf and zero gradient: +inf makes every p vanish
    p.lse2[(int64_t)bh * p.L + row] = (l == -INFINITY) ? INFINITY : l * 1.4426950408889634f;
  }
}

// ------------------------------------------------------------------------------------------------------
// dQ row walk, head dim 128: the forward's data path.  K and V tiles are copied from global memory straight
// into double-buffered LDS tiles (layout: psa_tiles.h), one barrier per tile; S^T = K Q^T and dP^T = V dO^T
// read them row-wise (128-bit reads), dQ^T += K^T dS^T reads the K tile through the transposing LDS load.
// ------------------------------------------------------------------------------------------------------
template <int D, int NW, class ET>
__global__ __launch_bounds__(NW * 64, 2) void psa_bwd_dq_lds_kernel(BwdParams p, int chunk, const int32_t* order) {
  using G = LtGeom<D>;
  using x8 = typename ET::x8;
  constexpr int LT_TILE = G::TILE;
  constexpr int NT = NW * 64, BM = NW * 32, CH = D / 8, KK = D / 16, DB = D / 32;
  constexpr int G16 = 4 / NW;
  constexpr int OST = D * 2 + 16;
  static_assert(BM * OST <= 4 * LT_TILE, "dQ staging must fit the tile buffers");

  extern __shared__ __align__(16) unsigned char smem[];
  // K tiles at 0 and LT_TILE, V tiles at 2*LT_TILE and 3*LT_TILE
  u32x2* tdesc = (u32x2*)(smem + 4 * LT_TILE);
  uint16_t* ids = (uint16_t*)(tdesc + p.max_tiles);
  __shared__ int s_cnt[4], s_ioff[4], s_toff[5], s_wcnt[4 * NW];

  // the workgroup's row (b, h, q-block): shares of rows per XCD, longest rows first (see psa_order.h)
  int row = psa_order::dealt_entry((int)blockIdx.x, chunk);
  if (order != nullptr) row = order[row];
  if (row < 0 || row >= p.B * p.Hq * p.Mq) return;
  const int I = row % p.Mq;
  const int bh = row / p.Mq;
  const int h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;
  const int L = p.L, bn_log2 = p.bn_log2, causal = p.causal;
  const float scale_log2 = p.scale_log2;

  int jmax = p.Nk;
  if (causal) {
    const int ce = (int)((((int64_t)(I + 1) * p.bm) + (1 << bn_log2) - 1) >> bn_log2);
    jmax = ce < jmax ? ce : jmax;
  }
  // Q and dO fragments of this wave's 32 rows (B operands), per-row delta and lse
  const int q_idx = I * BM + wave * 32 + l32;
  const int qr = q_idx < L ? q_idx : L - 1;
  x8 qf[KK], dof[KK];
  {
    const bf16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)qr * p.q_sl + hh * 8;
    const bf16_t* dp_ = p.dout + b * p.do_sb + h * p.do_sh + (int64_t)qr * p.do_sl + hh * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      qf[kk] = *(const x8*)(qp + kk * 16);
      dof[kk] = *(const x8*)(dp_ + kk * 16);
    }
  }
  const float delta = q_idx < L ? p.delta[(int64_t)bh * L + q_idx] : 0.f;
  const float lse2 = q_idx < L ? p.lse2[(int64_t)bh * L + q_idx] : INFINITY;

  const int T = build_row_schedule<NT>(p.map, p.map_elem, ((int64_t)bh * p.Mq + I) * p.Nk, p.Nk, jmax, bn_log2, L, causal != 0,
                                       (int64_t)I * p.bm, ids, tdesc, s_cnt, s_ioff, s_toff, s_wcnt);

  KvSource kvs;
  kvs.k0 = (const char*)(p.k + b * p.k_sb + hk * p.k_sh);
  kvs.v0 = (const char*)(p.v + b * p.v_sb + hk * p.v_sh);
  kvs.kp = (const char*)p.kp; kvs.vp = (const char*)p.vp;
  kvs.k_strb = (uint32_t)p.k_sl * 2u; kvs.v_strb = (uint32_t)p.v_sl * 2u;
  kvs.BHkv = (int64_t)p.B * p.Hkv; kvs.bhk = (int64_t)b * p.Hkv + hk; kvs.npad = p.npad;
  kvs.bn_log2 = bn_log2; kvs.L = L;
  const uint32_t f_chunk = lt_fetch_chunk<D>(lane);
  uint32_t r_off[2], t_off[2];
  lt_row_operand<D>(l32, hh, r_off);  // tile rows l32 (+32): r_off[kk & 1] + 64 * (kk >> 1) (+ 8 blocks)
  lt_tr_operand<D>(lane, t_off);      // K^T: t_off[s] + 64 * db + 4 * LT_ISTR * (16-key group)

  auto issue_tile = [&](int t, int stage) __attribute__((always_inline)) {
    TileSrc<G16> ts;
    lt_tile_src<D, G16>(kvs, tdesc, ids, t, wave, lane, ts);
    lt_issue_rows<D, G16>(smem + stage * LT_TILE, ts.kbase, ts.kstr, ts.lim, ts.src0, wave, f_chunk);
    lt_issue_rows<D, G16>(smem + (2 + stage) * LT_TILE, ts.vbase, ts.vstr, ts.lim, ts.src0, wave, f_chunk);
  };

  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;

  auto compute_tile = [&](int t, auto stage_c) __attribute__((always_inline)) {
    constexpr int ST = decltype(stage_c)::value;
    const uint32_t d = __builtin_amdgcn_readfirstlane(tdesc[t][0]);
    const int lv = d & 3;
    PSA_LDS(unsigned char) Ks = (PSA_LDS(unsigned char))(smem) + ST * LT_TILE;
    PSA_LDS(unsigned char) Vs = (PSA_LDS(unsigned char))(smem) + (2 + ST) * LT_TILE;
    f32x16 s[2], dp[2];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s[c][i] = 0.f;
        dp[c][i] = 0.f;
      }
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const x8 ka = *(PSA_LDS(const x8))(Ks + r_off[kk & 1] + (kk >> 1) * 64 + c * G::HALF);
        s[c] = ET::mfma(ka, qf[kk], s[c]);
        const x8 va = *(PSA_LDS(const x8))(Vs + r_off[kk & 1] + (kk >> 1) * 64 + c * G::HALF);
        dp[c] = ET::mfma(va, dof[kk], dp[c]);
      }
    }
    if (d & 4) {
      // Partly empty tile and/or causal diagonal: valid slots are a prefix of the tile (nvalid); a pooled key of
      // level lv is visible to query i iff src < (i + 1) >> lv.  Each run of 4 slots keeps its first `keep`.
      const int nvalid = (int)((d >> 3) & 127);
      const int qlim = (q_idx + 1) >> lv;
      const uint32_t d1 = __builtin_amdgcn_readfirstlane(tdesc[t][1]);
      const int cnt = (int)(d1 >> 16), lt = (int)(d >> 10), sbs_log2 = bn_log2 - lv;
      const uint16_t* lids = ids + (d1 & 0xffff);
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int r0 = c * 32 + g * 8 + hh * 4;
          int keep = nvalid - r0;
          if (causal) {
            const int gpos = (lt << 6) + r0;
            int bi = gpos >> sbs_log2;
            bi = bi < cnt - 1 ? bi : cnt - 1;
            const int src0 = ((int)lids[bi] << sbs_log2) + (gpos & ((1 << sbs_log2) - 1));
            keep = keep < qlim - src0 ? keep : qlim - src0;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) s[c][g * 4 + e] = e < keep ? s[c][g * 4 + e] : -INFINITY;
        }
    }
    const float nb = (float)lv - lse2;
    uint32_t pk[2][8];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float p0 = fast_exp2(__builtin_fmaf(s[c][i], scale_log2, nb));
        const float p1 = fast_exp2(__builtin_fmaf(s[c][i + 1], scale_log2, nb));
        pk[c][i >> 1] = ET::pack2(p0 * (dp[c][i] - delta), p1 * (dp[c][i + 1] - delta));
      }
    // dQ^T += K^T dS^T
#pragma unroll
    for (int cg = 0; cg < 4; ++cg) {
      const int c = cg >> 1, g = cg & 1;
      u32x4 bw = {pk[c][g * 4 + 0], pk[c][g * 4 + 1], pk[c][g * 4 + 2], pk[c][g * 4 + 3]};
      const x8 bfrag = __builtin_bit_cast(x8, bw);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const u32x2 lo = ET::read_tr(Ks + t_off[0] + db * 64 + cg * G::GROUP);
        const u32x2 hi = ET::read_tr(Ks + t_off[1] + db * 64 + cg * G::GROUP);
        u32x4 aw = {lo[0], lo[1], hi[0], hi[1]};
        acc[db] = ET::mfma(__builtin_bit_cast(x8, aw), bfrag, acc[db]);
      }
    }
  };

  if (T > 0) {
    // the Q / dO fragments must have arrived before the first copy is issued (a pending ordinary load would make
    // the compiler wait for all copies in flight inside the loop)
    __builtin_amdgcn_s_waitcnt(0x0f70);
    issue_tile(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    const std::integral_constant<int, 0> S0;
    const std::integral_constant<int, 1> S1;
    for (int t = 0; t < T; t += 2) {
      // invariant: stage t&1 holds tile t, the other stage is free
      if (t + 1 < T) issue_tile(t + 1, 1);
      compute_tile(t, S0);
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      if (t + 1 < T) {
        if (t + 2 < T) issue_tile(t + 2, 0);
        compute_tile(t + 1, S1);
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
      }
    }
  }

  __syncthreads();
  unsigned char* Os = smem;
  const float scale = p.scale;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w[0] = ET::pack2(acc[db][g * 4 + 0] * scale, acc[db][g * 4 + 1] * scale);
      w[1] = ET::pack2(acc[db][g * 4 + 2] * scale, acc[db][g * 4 + 3] * scale);
      *(u32x2*)(Os + (wave * 32 + l32) * OST + (db * 32 + g * 8 + hh * 4) * 2) = w;
    }
  __syncthreads();
  bf16_t* ob = p.dq + b * p.dq_sb + h * p.dq_sh;
  for (int u = tid; u < BM * CH; u += NT) {
    const int rr = u / CH, ch = u % CH;
    const int row = I * BM + rr;
    if (row < L) *(u32x4*)(ob + (int64_t)row * p.dq_sl + ch * 8) = *(const u32x4*)(Os + rr * OST + ch * 16);
  }
}

// slots of a kv-block in the dK/dV walk: one per level (a level-0 block of 128 keys is one slot of 128 keys)
constexpr int DKDV_SLOTS = 4;

// ------------------------------------------------------------------------------------------------------
// Longest-columns-first order for the dK/dV walk.  A workgroup's work is the number of q-blocks that retain its
// kv-block at its level, which varies a lot (a few key blocks are kept by every query block); issuing the
// workgroups by decreasing work removes the tail of the launch.  Results do not depend on the order.
// ------------------------------------------------------------------------------------------------------
constexpr int COL_BINS = psa_order::COST_BINS;

// one workgroup per (kv head, kv-block): per-level counts over the column -> cost of each of its slots.  The costs of
// the slots slot_lo .. of all blocks form one list per dK/dV launch: with a 128-key slot 0 that slot's list comes first
// (n_blocks entries), then the list of the slots 1 .. 3.
__global__ __launch_bounds__(256) void psa_bwd_colcost_kernel(BwdParams p, int wide0, int32_t* cost) {
  __shared__ int s_n[4];
  const int J = blockIdx.x, bhk = blockIdx.y, b = bhk / p.Hkv, hk = bhk % p.Hkv;
  const int n_rep = p.Hq / p.Hkv, Mq = p.Mq, bn_log2 = p.bn_log2;
  if (threadIdx.x < 4) s_n[threadIdx.x] = 0;
  __syncthreads();
  int n[4] = {0, 0, 0, 0};
  for (int e = threadIdx.x; e < n_rep * Mq; e += 256) {
    const int hl = e / Mq, I = e % Mq;
    const int h = hk * n_rep + hl;
    int level = load_map(p.map, (((int64_t)b * p.Hq + h) * Mq + I) * p.Nk + J, p.map_elem);
    if (p.causal) {
      const int ce = (int)((((int64_t)(I + 1) * p.bm) + (1 << bn_log2) - 1) >> bn_log2);
      if (J >= ce) level = 0;
    }
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) n[lv] += level == (1 << lv);
  }
#pragma unroll
  for (int lv = 0; lv < 4; ++lv)
    if (n[lv]) atomicAdd(&s_n[lv], n[lv]);
  __syncthreads();
  if ((int)threadIdx.x < DKDV_SLOTS) {
    const int lv = (int)threadIdx.x;
    const int c = s_n[lv] < COL_BINS - 1 ? s_n[lv] : COL_BINS - 1;
    const int64_t blk = (int64_t)bhk * p.Nk + J, n_blocks = (int64_t)gridDim.y * p.Nk;
    if (!wide0) cost[blk * DKDV_SLOTS + lv] = c;
    else if (lv == 0) cost[blk] = c;
    else cost[n_blocks + blk * (DKDV_SLOTS - 1) + (lv - 1)] = c;
  }
}

// ------------------------------------------------------------------------------------------------------
// dK/dV column walk, head dim 128: Q and dO rows are copied from global memory straight into LDS (double
// buffered, one barrier per step of 64 query rows) in the padded + swizzled row-major tile layout of the forward
// kernel; the row operands (S = Q K^T, dP = dO V^T) are 128-bit LDS reads and the transposed operands
// (dV^T += dO^T P, dK^T += Q^T dS) come from the same tiles through the transposing LDS load.
// The four waves of a workgroup split its keys and the 64 query rows of a step: 128 keys (level 0 of a 128-key
// block) = 4 key quarters, every wave takes both query halves one after the other ("wide": each Q / dO tile that is
// fetched feeds twice the arithmetic); <= 64 keys = 2 key halves x 2 query halves, combined through LDS at the end.
// ------------------------------------------------------------------------------------------------------
constexpr int B_ISTR = LT_ISTR;  // bytes between the blocks of a tile

// One instantiation per kind of slot (WIDE: the 128-key level-0 slot; else the slots slot_lo .. slot_lo + slot_cnt - 1 of
// every kv-block); workgroup id = ((b * Hkv + kv head) * Nk + kv-block) * slot_cnt + (slot - slot_lo), optionally
// re-ordered.
template <int D, bool WIDE, bool CAUSAL, class ET>
__global__ __launch_bounds__(256, 2) void psa_bwd_dkdv_lds_kernel(BwdParams p, int slot_lo, int slot_cnt, int n_wg, int chunk,
                                                                 const int32_t* order) {
  using G = LtGeom<D>;
  using x8 = typename ET::x8;
  constexpr int KK = D / 16, DB = D / 32, RPL = G::RPL;
  constexpr int B_TILE = G::TILE;
  extern __shared__ __align__(16) unsigned char smem[];
  // stage s: Q tile at 2*s*B_TILE, dO tile at (2*s + 1)*B_TILE
  float* s_lse = (float*)(smem + 4 * B_TILE);  // [2 stages][64]
  float* s_del = s_lse + 128;                  // [2 stages][64]
  uint32_t* qlist = (uint32_t*)(s_del + 128);  // [n_rep * Mq]  (head in group << 16 | q-block)
  __shared__ int s_nq;

  int wg = psa_order::dealt_entry((int)blockIdx.x, chunk);  // shares of slots per XCD, longest lists first (psa_order.h)
  if (order != nullptr) wg = order[wg];
  if (wg < 0 || wg >= n_wg) return;
  const int slot = slot_lo + wg % slot_cnt;
  const int J = (wg / slot_cnt) % p.Nk;
  const int bhk = wg / (slot_cnt * p.Nk), b = bhk / p.Hkv, hk = bhk % p.Hkv;
  const int n_rep = p.Hq / p.Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;
  const int L = p.L, bn_log2 = p.bn_log2, causal = p.causal, bm = p.bm, Mq = p.Mq;

  const int lv = slot;
  const int sbs = 1 << (bn_log2 - lv);            // pooled keys of this block at this level
  constexpr bool wide = WIDE;                     // 128 keys (the host launches this instantiation for such slots only)
  const int nkeys = sbs;
  const int64_t key_row0 = (int64_t)J << (bn_log2 - lv);  // first pooled row of this workgroup
  int key_valid = nkeys;                          // level 0: rows past L do not exist
  if (lv == 0) {
    const int64_t rem = (int64_t)L - key_row0;
    key_valid = rem < nkeys ? (rem > 0 ? (int)rem : 0) : nkeys;
  }
  // <= 64 keys: waves = 2 key halves x 2 query halves.  With at most 32 keys only one key half works: alternate
  // which pair of waves that is from workgroup to workgroup, so that all four SIMDs of a CU get work.
  // 128 keys: waves = 4 key quarters.
  const int flip = nkeys <= 32 ? (int)((blockIdx.x >> 3) & 1) : 0;
  const int kh = wide ? wave : ((wave & 1) ^ flip), qh = wide ? 0 : wave >> 1;
  const bool wave_active = key_valid > kh * 32;

  // ---- list of (head in group, q-block) that retain block J at this level -------------------------
  if (wave == 0) {
    int n = 0;
    const int total = n_rep * Mq;
    for (int e0 = 0; e0 < total; e0 += 64) {
      const int e = e0 + lane;
      bool on = false;
      if (e < total) {
        const int hl = e / Mq, I = e % Mq;
        const int h = hk * n_rep + hl;
        int level = p.map ? load_map(p.map, (((int64_t)b * p.Hq + h) * Mq + I) * p.Nk + J, p.map_elem) : 1;
        if (causal) {
          const int ce = (int)((((int64_t)(I + 1) * bm) + (1 << bn_log2) - 1) >> bn_log2);
          if (J >= ce) level = 0;
        }
        on = level == (1 << lv);
      }
      const uint64_t bal = __ballot(on);
      if (on) qlist[n + __popcll(bal & ((1ull << lane) - 1ull))] = ((uint32_t)(e / Mq) << 16) | (uint32_t)(e % Mq);
      n += __popcll(bal);
    }
    if (lane == 0) s_nq = n;
  }

  // ---- this wave's 32 keys: K and V fragments (B operands) --------------------------------------------
  const int key_local = kh * 32 + l32;
  x8 kf[KK], vf[KK];
  {
    int64_t row = key_row0 + (key_local < key_valid ? key_local : 0);
    if (key_valid == 0) row = 0;
    const bf16_t *kp_, *vp_;
    if (lv == 0 || p.kp == nullptr) {
      // without a level map there are no pooled buffers: the workgroups of the pooled levels have an empty
      // q-block list and only write zeros, whatever they load here
      kp_ = p.k + b * p.k_sb + hk * p.k_sh + (lv == 0 ? row : 0) * p.k_sl;
      vp_ = p.v + b * p.v_sb + hk * p.v_sh + (lv == 0 ? row : 0) * p.v_sl;
    } else {
      const int64_t off = (pool_row_offset(lv, (int64_t)p.B * p.Hkv, bhk, p.npad) + row) * D;
      kp_ = p.kp + off;
      vp_ = p.vp + off;
    }
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      kf[kk] = *(const x8*)(kp_ + kk * 16 + hh * 8);
      vf[kk] = *(const x8*)(vp_ + kk * 16 + hh * 8);
    }
  }
  const int key_up = (int)(((key_row0 + key_local + 1) << lv) - 1);  // last token the pooled key covers (< npad)
  __syncthreads();
  const int nq = s_nq;

  // ---- lane-invariant LDS addressing (tile layout: see the forward kernel) ---------------------------
  // copy: wave w fills the 16-row group w of both tiles; lane (fq = lane/16, pos = lane%16) of block n writes
  // row fq of that block, i.e. tile row 16w + 4fq + n, chunk pos ^ fq
  // (recomputed from the lane id at every use - see issue_step - instead of living in registers across the matrix work:
  // this kernel has no register to spare, and a spilled value comes back through a vmcnt wait that would also wait
  // for the tile copies in flight)
  uint32_t r_off[2], t_off[2];
  // (qh = 0 in a wide workgroup, whose passes add HALF * query half as an immediate)
  lt_row_operand<D>(qh * 32 + l32, hh, r_off);  // row operand of k-step kk: r_off[kk & 1] + 64 * (kk >> 1)
  lt_tr_operand<D>(lane, t_off);                // transposed operand: t_off[s] + 64 * db + GROUP * (16-row group)
#pragma unroll
  for (int i = 0; i < 2; ++i) t_off[i] += (uint32_t)(qh * G::HALF);

  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dk[db][i] = 0.f;
      dv[db][i] = 0.f;
    }
  const float scale_log2 = p.scale_log2;
  const float bias = (float)lv;
  const int spb_log2 = bm >> 7;      // steps of 64 query rows per q-block: 1 (block_m 64) or 2 (128)
  const int n_steps = key_valid > 0 ? nq << spb_log2 : 0;
  const uint32_t q_strb = (uint32_t)p.q_sl * 2u, do_strb = (uint32_t)p.do_sl * 2u;

  // step i -> (head, q-block, first query row)
  auto step_of = [&](int i, int& h, int& I, int& q0) __attribute__((always_inline)) {
    const uint32_t ent = qlist[i >> spb_log2];
    h = hk * n_rep + (int)(ent >> 16);
    I = (int)(ent & 0xffff);
    q0 = I * bm + (i & ((1 << spb_log2) - 1)) * 64;
  };
  // rows of step i -> stage; the per-row lse / delta values come back in registers and are put into LDS later
  float lse_next = 0.f, del_next = 0.f;

  auto issue_step = [&](int i, int stage) __attribute__((always_inline)) {
    int h, I, q0;
    step_of(i, h, I, q0);
    h = __builtin_amdgcn_readfirstlane(h);
    q0 = __builtin_amdgcn_readfirstlane(q0);
    if (tid < 64) {
      const int row = q0 + tid;
      const int64_t bh = (int64_t)b * p.Hq + h;
      // rows past L: p is forced to 0 through lse = +inf
      lse_next = row < L ? p.lse2[bh * L + row] : INFINITY;
      del_next = row < L ? p.delta[bh * L + row] : 0.f;
    }
    const char* qb = (const char*)(p.q + b * p.q_sb + h * p.q_sh);
    const char* ob = (const char*)(p.dout + b * p.do_sb + h * p.do_sh);
    int ln = lane;
    asm volatile("" : "+v"(ln));  // keeps the two values below out of the loop-invariant registers
    const uint32_t f_chunk = lt_fetch_chunk<D>(ln);
    const int f_row = wave * 16 + lt_fetch_row<D>(ln);
    const int r0 = q0 + f_row;
    if (q0 + 64 <= L) {
      const uint32_t qo = (uint32_t)r0 * q_strb + f_chunk, oo = (uint32_t)r0 * do_strb + f_chunk;
#pragma unroll
      for (int n = 0; n < RPL; ++n) {
        psa_tiles::lds_copy16(qb + (uint64_t)(n * q_strb), qo, psa_tiles::lds_addr_of(smem + 2 * stage * B_TILE + (wave * RPL + n) * B_ISTR));
        psa_tiles::lds_copy16(ob + (uint64_t)(n * do_strb), oo, psa_tiles::lds_addr_of(smem + (2 * stage + 1) * B_TILE + (wave * RPL + n) * B_ISTR));
      }
    } else {
#pragma unroll
      for (int n = 0; n < RPL; ++n) {
        int row = r0 + n;
        row = row < L ? row : L - 1;
        row = row > 0 ? row : 0;
        psa_tiles::lds_copy16(qb, (uint32_t)row * q_strb + f_chunk, psa_tiles::lds_addr_of(smem + 2 * stage * B_TILE + (wave * RPL + n) * B_ISTR));
        psa_tiles::lds_copy16(ob, (uint32_t)row * do_strb + f_chunk, psa_tiles::lds_addr_of(smem + (2 * stage + 1) * B_TILE + (wave * RPL + n) * B_ISTR));
      }
    }
  };
  // (the level's bias goes in with the row's lse: one subtraction per row here instead of one per logit later)
  auto publish_rows = [&](int stage) __attribute__((always_inline)) {
    if (tid < 64) {
      s_lse[stage * 64 + tid] = bias - lse_next;
      s_del[stage * 64 + tid] = del_next;
    }
  };

  PSA_LDS(const float) rows_base0 = (PSA_LDS(const float))(smem + 4 * B_TILE) + (qh * 32 + hh * 4);
  auto compute_step = [&](int i, auto stage_c) __attribute__((always_inline)) {
    constexpr int ST = decltype(stage_c)::value;
    int h, I, q0;
    step_of(i, h, I, q0);
    I = __builtin_amdgcn_readfirstlane(I);
    q0 = __builtin_amdgcn_readfirstlane(q0);
    const bool diag = causal && ((((int64_t)J + 1) << bn_log2) - 1 > (int64_t)I * bm);
#pragma unroll
    for (int qi = 0; qi < (WIDE ? 2 : 1); ++qi) {
    const int qhv = WIDE ? qi : qh;  // the query half of this pass (the lane offsets already hold qh)
    PSA_LDS(unsigned char) Qs = (PSA_LDS(unsigned char))(smem) + 2 * ST * B_TILE + (WIDE ? qi * G::HALF : 0);
    PSA_LDS(unsigned char) Os = (PSA_LDS(unsigned char))(smem) + (2 * ST + 1) * B_TILE + (WIDE ? qi * G::HALF : 0);
    PSA_LDS(const float) rows_base = rows_base0 + (WIDE ? qi * 32 : 0);
    // S = Q K^T and dP = dO V^T for this wave's (32 q) x (32 keys): lane = key column, registers = q rows
    f32x16 s, dp;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      s[j] = 0.f;
      dp[j] = 0.f;
    }
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const x8 qa = *(PSA_LDS(const x8))(Qs + r_off[kk & 1] + (kk >> 1) * 64);
      const x8 oa = *(PSA_LDS(const x8))(Os + r_off[kk & 1] + (kk >> 1) * 64);
      s = ET::mfma(qa, kf[kk], s);
      dp = ET::mfma(oa, vf[kk], dp);
    }
    uint32_t pk[8], dsk[8];
    // p = exp2(scale * s + bias - lse), dS = p (dP - delta).  Lanes whose key does not exist (the ragged end of the
    // sequence at level 0; lanes beyond the 16 keys of a level-8 block) work on a copy of the block's first key: the
    // columns of dK^T / dV^T are independent of each other and those lanes' columns are never read.  Only the causal
    // diagonal needs a mask: keys behind the query get p = 0 (thr: first query row of this pass, relative to the
    // lane's rows, that sees the lane's key).
    int thr = 0;
    if (CAUSAL) thr = diag ? key_up - (q0 + qhv * 32 + hh * 4) : -0x40000000;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      // one lane base + immediates (stage, group, bias - lse / delta array)
      const f32x4 l4 = *(PSA_LDS(const f32x4))(rows_base + ST * 64 + g * 8);
      const f32x4 d4 = *(PSA_LDS(const f32x4))(rows_base + 128 + ST * 64 + g * 8);
      float pv[4], dsv[4];
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2) {
        float pe = fast_exp2(__builtin_fmaf(s[g * 4 + e2], scale_log2, l4[e2]));
        if (CAUSAL) pe = thr <= g * 8 + e2 ? pe : 0.f;
        pv[e2] = pe;
        dsv[e2] = pe * (dp[g * 4 + e2] - d4[e2]);
      }
      pk[g * 2] = ET::pack2(pv[0], pv[1]);
      pk[g * 2 + 1] = ET::pack2(pv[2], pv[3]);
      dsk[g * 2] = ET::pack2(dsv[0], dsv[1]);
      dsk[g * 2 + 1] = ET::pack2(dsv[2], dsv[3]);
    }
    // dV^T += dO^T P,  dK^T += Q^T dS   (contraction over this wave's 32 query rows, 16 at a time)
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      u32x4 pw = {pk[g * 4 + 0], pk[g * 4 + 1], pk[g * 4 + 2], pk[g * 4 + 3]};
      u32x4 sw = {dsk[g * 4 + 0], dsk[g * 4 + 1], dsk[g * 4 + 2], dsk[g * 4 + 3]};
      const x8 pfrag = __builtin_bit_cast(x8, pw), sfrag = __builtin_bit_cast(x8, sw);
      const int grp = g * G::GROUP;  // (Qs, Os already point at this pass's query half = two 16-row groups)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const u32x2 olo = ET::read_tr(Os + t_off[0] + db * 64 + grp);
        const u32x2 ohi = ET::read_tr(Os + t_off[1] + db * 64 + grp);
        u32x4 oa = {olo[0], olo[1], ohi[0], ohi[1]};
        dv[db] = ET::mfma(__builtin_bit_cast(x8, oa), pfrag, dv[db]);
        const u32x2 qlo = ET::read_tr(Qs + t_off[0] + db * 64 + grp);
        const u32x2 qhi = ET::read_tr(Qs + t_off[1] + db * 64 + grp);
        u32x4 qa2 = {qlo[0], qlo[1], qhi[0], qhi[1]};
        dk[db] = ET::mfma(__builtin_bit_cast(x8, qa2), sfrag, dk[db]);
      }
    }
    if (WIDE) __builtin_amdgcn_sched_barrier(0);  // the second pass starts after the first: its operands do not fit beside it
    }
  };

  if (n_steps > 0) {
    issue_step(0, 0);
    publish_rows(0);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the rows have landed
    __syncthreads();
    const std::integral_constant<int, 0> S0;
    const std::integral_constant<int, 1> S1;
    for (int i = 0; i < n_steps; i += 2) {
      // invariant: stage i&1 holds step i, the other stage is free
      if (i + 1 < n_steps) issue_step(i + 1, 1);
      if (wave_active) compute_step(i, S0);
      if (i + 1 < n_steps) publish_rows(1);
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      if (i + 1 < n_steps) {
        if (i + 2 < n_steps) issue_step(i + 2, 0);
        if (wave_active) compute_step(i + 1, S1);
        if (i + 2 < n_steps) publish_rows(0);
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
      }
    }
  }

  // ---- 128-key level-0 slot: this workgroup owns 128 tokens of dK / dV outright.  The pooled levels' launch has
  // finished, so the tokens' shares of the pooled gradients (1/l of pooled row n >> level; for the last real token
  // also those of the replicate-pad tokens behind it) are added here and dK, dV leave in the tensors' 16-bit type: no fp32 level-0
  // buffer, no separate pass.  Same sums in the same order as psa_bwd_unpool_kernel.
  if constexpr (WIDE) {
    const int64_t n = key_row0 + key_local;
    if (n < L) {
      const int64_t BH = (int64_t)p.B * p.Hkv, npad = p.npad;
      const float* lk[3];
      const float* lvv[3];
#pragma unroll
      for (int l = 1; l < 4; ++l) {
        const int64_t rows = BH * npad + pool_row_offset(l, BH, bhk, npad);
        lk[l - 1] = p.wk + rows * D;
        lvv[l - 1] = p.wv + rows * D;
      }
      bf16_t* dkp = p.dk + b * p.dk_sb + hk * p.dk_sh + n * p.dk_sl;
      bf16_t* dvp = p.dv + b * p.dv_sb + hk * p.dv_sh + n * p.dv_sl;
      const float scale = p.scale;
      auto contrib = [&](const float* const (&w)[3], int64_t row, int col) __attribute__((always_inline)) {
        f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int l = 1; l < 4; ++l) {
          const f32x4 x = *(const f32x4*)(w[l - 1] + (row >> l) * D + col);
          const float inv = 1.0f / (float)(1 << l);
#pragma unroll
          for (int e = 0; e < 4; ++e) a[e] += x[e] * inv;
        }
        return a;
      };
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int col = db * 32 + g * 8 + hh * 4;
          f32x4 gk, gv;
#pragma unroll
          for (int e2 = 0; e2 < 4; ++e2) {
            gk[e2] = dk[db][g * 4 + e2] * scale;
            gv[e2] = dv[db][g * 4 + e2];
          }
          {
            const f32x4 ak = contrib(lk, n, col), av = contrib(lvv, n, col);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              gk[e] += ak[e];
              gv[e] += av[e];
            }
          }
          if (n == L - 1) {  // gradient of the replicate-pad rows lands on the last real token
            for (int64_t r = L; r < npad; ++r) {
              const f32x4 ak = contrib(lk, r, col), av = contrib(lvv, r, col);
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                gk[e] += ak[e];
                gv[e] += av[e];
              }
            }
          }
          u32x2 ok_, ov_;
          ok_[0] = ET::pack2(gk[0], gk[1]);
          ok_[1] = ET::pack2(gk[2], gk[3]);
          ov_[0] = ET::pack2(gv[0], gv[1]);
          ov_[1] = ET::pack2(gv[2], gv[3]);
          *(u32x2*)(dkp + col) = ok_;
          *(u32x2*)(dvp + col) = ov_;
        }
    }
    return;
  }
  // ---- combine the two query halves (<= 64 keys) and write this workgroup's rows of the level buffers ----
  __syncthreads();
  float* red = (float*)smem;  // [2 key halves][2 tensors][DB*16][64 lanes]
  if (!wide && qh == 1) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        red[((kh * 2 + 0) * DB * 16 + db * 16 + i) * 64 + lane] = dk[db][i];
        red[((kh * 2 + 1) * DB * 16 + db * 16 + i) * 64 + lane] = dv[db][i];
      }
  }
  __syncthreads();
  if (qh == 0 && key_local < nkeys) {
    const int64_t lvl_off = pool_row_offset(lv, (int64_t)p.B * p.Hkv, bhk, p.npad);
    // level buffers: level 0 first ([BHkv, npad, D]), then levels 1..3 like the pooled K/V buffers
    const int64_t base_rows = lv == 0 ? bhk * p.npad : (int64_t)p.B * p.Hkv * p.npad + lvl_off;
    float* wk = p.wk + (base_rows + key_row0 + key_local) * D;
    float* wv = p.wv + (base_rows + key_row0 + key_local) * D;
    const float scale = p.scale;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 a, c2;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          const int i = g * 4 + e2;
          a[e2] = (dk[db][i] + (wide ? 0.f : red[((kh * 2 + 0) * DB * 16 + db * 16 + i) * 64 + lane])) * scale;
          c2[e2] = dv[db][i] + (wide ? 0.f : red[((kh * 2 + 1) * DB * 16 + db * 16 + i) * 64 + lane]);
        }
        *(f32x4*)(wk + db * 32 + g * 8 + hh * 4) = a;
        *(f32x4*)(wv + db * 32 + g * 8 + hh * 4) = c2;
      }
  }
}

// ------------------------------------------------------------------------------------------------------
// un-pool: levels -> dK, dV (the tensors' 16-bit type)
// ------------------------------------------------------------------------------------------------------
template <class ET>
__global__ __launch_bounds__(256) void psa_bwd_unpool_kernel(BwdParams p, int D) {
  const int which = blockIdx.z;  // 0: dK, 1: dV
  const int bhk = blockIdx.y, b = bhk / p.Hkv, hk = bhk % p.Hkv;
  const int chunks = D >> 2;  // float4 chunks per row
  const int64_t unit = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t n = unit / chunks;
  const int c = (int)(unit % chunks);
  if (n >= p.L) return;
  const float* w = which == 0 ? p.wk : p.wv;
  const int64_t BH = (int64_t)p.B * p.Hkv, npad = p.npad;
  const float* w0 = w + (bhk * npad) * D;
  const float* wl[3];
#pragma unroll
  for (int lv = 1; lv < 4; ++lv) wl[lv - 1] = w + (BH * npad + pool_row_offset(lv, BH, bhk, npad)) * D;
  auto contrib = [&](int64_t row) {
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int lv = 1; lv < 4; ++lv) {
      const f32x4 x = *(const f32x4*)(wl[lv - 1] + (row >> lv) * D + c * 4);
      const float inv = 1.0f / (float)(1 << lv);
#pragma unroll
      for (int e = 0; e < 4; ++e) a[e] += x[e] * inv;
    }
    return a;
  };
  f32x4 g = *(const f32x4*)(w0 + n * D + c * 4);
  {
    const f32x4 a = contrib(n);
#pragma unroll
    for (int e = 0; e < 4; ++e) g[e] += a[e];
  }
  if (n == p.L - 1) {  // gradient of the replicate-pad rows lands on the last real token
    for (int64_t r = p.L; r < npad; ++r) {
      const f32x4 a = contrib(r);
#pragma unroll
      for (int e = 0; e < 4; ++e) g[e] += a[e];
    }
  }
  bf16_t* dst = which == 0 ? p.dk + b * p.dk_sb + hk * p.dk_sh + n * p.dk_sl : p.dv + b * p.dv_sb + hk * p.dv_sh + n * p.dv_sl;
  u32x2 o;
  o[0] = ET::pack2(g[0], g[1]);
  o[1] = ET::pack2(g[2], g[3]);
  *(u32x2*)(dst + c * 4) = o;
}


}  // namespace

extern "C" int64_t psa_bwd_workspace_bytes(int B, int Hq, int Hkv, int L, int D, int block_n) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || L <= 0 || D <= 0 || block_n <= 0) return 0;
  const int64_t npad = (int64_t)((L + block_n - 1) / block_n) * block_n;
  const int64_t levels = (int64_t)B * Hkv * D * (npad + npad / 2 + npad / 4 + npad / 8);
  // + cost and issue order of the dQ rows (block_m >= 64) and of the dK/dV slots (4 per kv-block), padded to whole shares
  const int64_t pad = 16 * psa_order::MAX_PHASES;
  const int64_t n_rows = (int64_t)B * Hq * ((L + 63) / 64), n_slots = (int64_t)B * Hkv * ((L + block_n - 1) / block_n) * DKDV_SLOTS;
  return (2 * levels + 2 * (int64_t)B * Hq * L + 2 * (n_rows + pad) + 2 * (n_slots + 2 * pad)) * (int64_t)sizeof(float);
}

extern "C" int psa_bwd(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool, const void* map,
                       int map_elem_bytes, psa_tensor4 out, psa_tensor4 dout, const float* lse, psa_tensor4 dq, psa_tensor4 dk,
                       psa_tensor4 dv, void* workspace, int B, int Hq, int Hkv, int L, int D, int block_m, int block_n,
                       float sm_scale, int causal, psa_stream_t stream) {
  PSA_REQUIRE(q.ptr && k.ptr && v.ptr && out.ptr && dout.ptr && lse && dq.ptr && dk.ptr && dv.ptr && workspace, PSA_ERR_ARG,
              "psa_bwd: null pointer");
  PSA_REQUIRE(map == nullptr || (k_pool && v_pool), PSA_ERR_ARG, "psa_bwd: pooled K/V required with a level map");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_bwd: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && L > 0, PSA_ERR_ARG, "psa_bwd: B, H, L must be positive");
  PSA_REQUIRE(Hq % Hkv == 0, PSA_ERR_ARG, "psa_bwd: Hq=%d must be a multiple of Hkv=%d", Hq, Hkv);
  PSA_REQUIRE(sm_scale > 0.f, PSA_ERR_ARG, "psa_bwd: sm_scale must be positive");
  PSA_REQUIRE(D == 64 || D == 128, PSA_ERR_UNSUPPORTED, "psa_bwd: head dim %d not in {64, 128}", D);
  PSA_REQUIRE(block_m == 64 || block_m == 128, PSA_ERR_UNSUPPORTED, "psa_bwd: block_m=%d not in {64, 128}", block_m);
  PSA_REQUIRE(block_n == 32 || block_n == 64 || block_n == 128, PSA_ERR_UNSUPPORTED, "psa_bwd: block_n=%d not in {32, 64, 128}", block_n);
  const psa_tensor4* ts[8] = {&q, &k, &v, &out, &dout, &dq, &dk, &dv};
  for (int i = 0; i < 8; ++i)
    PSA_REQUIRE(((uintptr_t)ts[i]->ptr % 16 == 0) && ts[i]->stride_b % 8 == 0 && ts[i]->stride_h % 8 == 0 && ts[i]->stride_l % 8 == 0,
                PSA_ERR_UNSUPPORTED, "psa_bwd: tensors must be 16-byte aligned with strides that are multiples of 8 elements");
  PSA_REQUIRE((int64_t)L * k.stride_l * 2 < (1ll << 32) && (int64_t)L * v.stride_l * 2 < (1ll << 32), PSA_ERR_UNSUPPORTED,
              "psa_bwd: one (batch, head) slice of K/V must span less than 4 GiB");
  PSA_REQUIRE((int64_t)L * q.stride_l * 2 < (1ll << 32) && (int64_t)L * dout.stride_l * 2 < (1ll << 32), PSA_ERR_UNSUPPORTED,
              "psa_bwd: one (batch, head) slice of q / dout must span less than 4 GiB");
  const int Mq = (L + block_m - 1) / block_m, Nk = (L + block_n - 1) / block_n;
  PSA_REQUIRE(Nk <= 65535 && Mq <= 65535, PSA_ERR_UNSUPPORTED, "psa_bwd: more than 65535 blocks");
  PSA_REQUIRE((int64_t)B * Hq <= 65535, PSA_ERR_UNSUPPORTED, "psa_bwd: B*Hq too large");
  for (int i = 1; i < 8; ++i)
    PSA_REQUIRE(ts[i]->dtype == q.dtype, PSA_ERR_ARG, "psa_bwd: q, k, v, out, dout, dq, dk, dv must share one element type");
  PSA_REQUIRE(q.dtype == PSA_DTYPE_BF16 || q.dtype == PSA_DTYPE_F16, PSA_ERR_UNSUPPORTED,
              "psa_bwd: element type must be bf16 or fp16 (the pooled buffers in the same type)");
  BwdParams p;
  p.q = (const bf16_t*)q.ptr; p.k = (const bf16_t*)k.ptr; p.v = (const bf16_t*)v.ptr;
  p.o = (const bf16_t*)out.ptr; p.dout = (const bf16_t*)dout.ptr;
  p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sl = q.stride_l;
  p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sl = k.stride_l;
  p.v_sb = v.stride_b; p.v_sh = v.stride_h; p.v_sl = v.stride_l;
  p.o_sb = out.stride_b; p.o_sh = out.stride_h; p.o_sl = out.stride_l;
  p.do_sb = dout.stride_b; p.do_sh = dout.stride_h; p.do_sl = dout.stride_l;
  p.dq = (bf16_t*)dq.ptr; p.dk = (bf16_t*)dk.ptr; p.dv = (bf16_t*)dv.ptr;
  p.dq_sb = dq.stride_b; p.dq_sh = dq.stride_h; p.dq_sl = dq.stride_l;
  p.dk_sb = dk.stride_b; p.dk_sh = dk.stride_h; p.dk_sl = dk.stride_l;
  p.dv_sb = dv.stride_b; p.dv_sh = dv.stride_h; p.dv_sl = dv.stride_l;
  p.kp = (const bf16_t*)k_pool; p.vp = (const bf16_t*)v_pool;
  p.map = map; p.map_elem = map_elem_bytes; p.lse = lse;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.L = L; p.Mq = Mq; p.Nk = Nk;
  p.bn_log2 = psa_ilog2(block_n); p.bm = block_m;
  p.npad = (int64_t)Nk * block_n;
  p.scale = sm_scale;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  p.causal = causal ? 1 : 0;
  p.max_tiles = psa_tiles::max_tiles(Nk, block_n);
  const int64_t levels = (int64_t)B * Hkv * D * (p.npad + p.npad / 2 + p.npad / 4 + p.npad / 8);
  p.wk = (float*)workspace;
  p.wv = p.wk + levels;
  p.delta = p.wv + levels;
  p.lse2 = p.delta + (int64_t)B * Hq * L;
  hipStream_t st = (hipStream_t)stream;

  auto run = [&](auto et) -> int {
  using ET = decltype(et);
  // 1. delta, lse2
  {
    const int rows_per_wg = 256 / (D / 8);
    dim3 grid((unsigned)((L + rows_per_wg - 1) / rows_per_wg), (unsigned)(B * Hq));
    if (D == 128) hipLaunchKernelGGL((psa_bwd_delta_kernel<128, ET>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((psa_bwd_delta_kernel<64, ET>), grid, dim3(256), 0, st, p);
    const int rc = psa_check_launch("psa_bwd (delta)");
    if (rc != PSA_OK) return rc;
  }
  // issue orders (costs and orders live behind lse2 in the workspace; every list is padded to whole shares)
  int32_t* ws_int = (int32_t*)(p.lse2 + (int64_t)B * Hq * L);
  // 2. dQ
  {
    const int64_t total = (int64_t)B * Hq * Mq;
    PSA_REQUIRE(total < (1ll << 28), PSA_ERR_UNSUPPORTED, "psa_bwd: too many workgroups");
    int chunk, groups;
    const double kv_bytes = 2.0 * B * Hkv * (double)p.npad * D * 2.0 * (map != nullptr ? 1.875 : 1.0);
    psa_order::deal(total, kv_bytes, B * Hkv, chunk, groups);
    const int32_t* order = nullptr;
    if (map != nullptr && total > 8 * 32) {
      int32_t* cost = ws_int;
      int32_t* ord = cost + total;
      hipLaunchKernelGGL(psa_order::psa_row_cost_kernel, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, st, map, map_elem_bytes, (int)total,
                         Mq, Nk, p.bn_log2, block_m, p.causal, cost);
      if (int e = psa_check_launch("psa_bwd (row cost)")) return e;
      hipLaunchKernelGGL(psa_order::psa_chunk_sort_kernel, dim3((unsigned)groups), dim3(256), 0, st, cost, (int)total, chunk, ord);
      if (int e = psa_check_launch("psa_bwd (row order)")) return e;
      order = ord;
    }
    ws_int += 2 * total + 16 * psa_order::MAX_PHASES;
    auto launch = [&](auto kern, size_t tile_bytes, int nw) -> int {
      const size_t shmem = tile_bytes + (size_t)p.max_tiles * 8 + (size_t)Nk * 2;
      if (shmem > 160 * 1024) return PSA_ERR_UNSUPPORTED;
      if (shmem > 48 * 1024 && hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess)
        return PSA_ERR_LAUNCH;
      hipLaunchKernelGGL(kern, dim3((unsigned)(chunk * groups)), dim3(nw * 64), shmem, st, p, chunk, order);
      return PSA_OK;
    };
    int rc;
    if (D == 128 && block_m == 128) rc = launch(psa_bwd_dq_lds_kernel<128, 4, ET>, (size_t)4 * LtGeom<128>::TILE, 4);
    else if (D == 128) rc = launch(psa_bwd_dq_lds_kernel<128, 2, ET>, (size_t)4 * LtGeom<128>::TILE, 2);
    else if (block_m == 128) rc = launch(psa_bwd_dq_lds_kernel<64, 4, ET>, (size_t)4 * LtGeom<64>::TILE, 4);
    else rc = launch(psa_bwd_dq_lds_kernel<64, 2, ET>, (size_t)4 * LtGeom<64>::TILE, 2);
    PSA_REQUIRE(rc == PSA_OK, rc, "psa_bwd: sequence too long for the on-chip schedule (LDS)");
    rc = psa_check_launch("psa_bwd (dQ)");
    if (rc != PSA_OK) return rc;
  }
  // 3. dK, dV per level: the 128-key level-0 slots (if block_n = 128) in one launch, the other slots in a second one
  {
    const int n_rep = Hq / Hkv;
    const bool wide0 = block_n > 64;
    const int64_t n_blocks = (int64_t)B * Hkv * Nk;
    const int64_t n_wide = wide0 ? n_blocks : 0, n_rest = n_blocks * (wide0 ? DKDV_SLOTS - 1 : DKDV_SLOTS);
    PSA_REQUIRE(n_wide + n_rest < (1ll << 28), PSA_ERR_UNSUPPORTED, "psa_bwd: too many workgroups");
    size_t shmem = (size_t)4 * (D == 128 ? LtGeom<128>::TILE : LtGeom<64>::TILE) + 256 * sizeof(float) + (size_t)n_rep * Mq * 4;
    const size_t red = (size_t)2 * 2 * (D / 32) * 16 * 64 * sizeof(float);
    if (shmem < red) shmem = red;
    PSA_REQUIRE(shmem <= 160 * 1024, PSA_ERR_UNSUPPORTED, "psa_bwd: too many q-blocks for the on-chip lists (LDS)");
    // shares by the Q / dO rows the walk streams
    const double qdo_bytes = 2.0 * B * Hq * (double)L * D * 2.0;
    int chunk_w = 1, groups_w = 8, chunk_r, groups_r;
    if (wide0) psa_order::deal(n_wide, qdo_bytes, B * Hkv, chunk_w, groups_w);
    psa_order::deal(n_rest, qdo_bytes, B * Hkv, chunk_r, groups_r);
    const int32_t *order_wide = nullptr, *order_rest = nullptr;
    if (map != nullptr && n_blocks > 8) {
      int32_t* cost = ws_int;
      int32_t* ord_w = cost + (n_wide + n_rest);
      int32_t* ord_r = ord_w + (wide0 ? (int64_t)chunk_w * groups_w : 0);
      hipLaunchKernelGGL(psa_bwd_colcost_kernel, dim3((unsigned)Nk, (unsigned)(B * Hkv)), dim3(256), 0, st, p, wide0 ? 1 : 0, cost);
      if (int e = psa_check_launch("psa_bwd (column cost)")) return e;
      if (wide0) {
        hipLaunchKernelGGL(psa_order::psa_chunk_sort_kernel, dim3((unsigned)groups_w), dim3(256), 0, st, cost, (int)n_wide, chunk_w, ord_w);
        order_wide = ord_w;
      }
      hipLaunchKernelGGL(psa_order::psa_chunk_sort_kernel, dim3((unsigned)groups_r), dim3(256), 0, st, cost + n_wide, (int)n_rest, chunk_r,
                         ord_r);
      order_rest = ord_r;
      if (int e = psa_check_launch("psa_bwd (column order)")) return e;
    }
    auto launch = [&](auto kern, int64_t n_wg, int chunk, int groups, int slot_lo, int slot_cnt, const int32_t* order) -> int {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess) return PSA_ERR_LAUNCH;
      hipLaunchKernelGGL(kern, dim3((unsigned)(chunk * groups)), dim3(256), shmem, st, p, slot_lo, slot_cnt, (int)n_wg, chunk, order);
      return PSA_OK;
    };
    // the pooled levels first: the 128-key level-0 launch adds their rows to its own and writes dK, dV
    const int lo = wide0 ? 1 : 0;
    int rl;
    if (causal)
      rl = D == 128 ? launch(psa_bwd_dkdv_lds_kernel<128, false, true, ET>, n_rest, chunk_r, groups_r, lo, DKDV_SLOTS - lo, order_rest)
                    : launch(psa_bwd_dkdv_lds_kernel<64, false, true, ET>, n_rest, chunk_r, groups_r, lo, DKDV_SLOTS - lo, order_rest);
    else
      rl = D == 128 ? launch(psa_bwd_dkdv_lds_kernel<128, false, false, ET>, n_rest, chunk_r, groups_r, lo, DKDV_SLOTS - lo, order_rest)
                    : launch(psa_bwd_dkdv_lds_kernel<64, false, false, ET>, n_rest, chunk_r, groups_r, lo, DKDV_SLOTS - lo, order_rest);
    PSA_REQUIRE(rl == PSA_OK, rl, "psa_bwd: cannot reserve %zu bytes of LDS", shmem);
    if (int e = psa_check_launch("psa_bwd (dK/dV)")) return e;
    if (wide0) {
      if (causal)
        rl = D == 128 ? launch(psa_bwd_dkdv_lds_kernel<128, true, true, ET>, n_wide, chunk_w, groups_w, 0, 1, order_wide)
                      : launch(psa_bwd_dkdv_lds_kernel<64, true, true, ET>, n_wide, chunk_w, groups_w, 0, 1, order_wide);
      else
        rl = D == 128 ? launch(psa_bwd_dkdv_lds_kernel<128, true, false, ET>, n_wide, chunk_w, groups_w, 0, 1, order_wide)
                      : launch(psa_bwd_dkdv_lds_kernel<64, true, false, ET>, n_wide, chunk_w, groups_w, 0, 1, order_wide);
      PSA_REQUIRE(rl == PSA_OK, rl, "psa_bwd: cannot reserve %zu bytes of LDS", shmem);
      return psa_check_launch("psa_bwd (dK/dV, 128-key slots)");
    }
  }
  // 4. un-pool (blocks of 64 or 32 keys: every level went to the fp32 buffers)
  {
    const int64_t units = (int64_t)L * (D / 4);
    dim3 grid((unsigned)((units + 255) / 256), (unsigned)(B * Hkv), 2);
    hipLaunchKernelGGL(psa_bwd_unpool_kernel<ET>, grid, dim3(256), 0, st, p, D);
  }
  return psa_check_launch("psa_bwd (un-pool)");
  };
  int rc = PSA_ERR_ARG;
  psa_dispatch16(q.dtype, [&](auto et) { rc = run(et); });
  return rc;
}
