// Pyramid sparse attention forward (non-causal and causal) on bf16 MFMA.
//
// One workgroup per (batch, head, q-block of BM = 32*NW rows); every wave owns 32 query rows; two workgroups
// per CU.
//
//  * The workgroup first compacts its row of the level map into four per-level lists of kv-block ids in LDS
//    (ballot + popcount, ascending block order - deterministic) and a list of tile descriptors.
//  * Work is a sequence of TILES of 64 pooled keys of one level: a level-l kv-block holds block_n/l pooled
//    keys, so one tile is half a 128-key block, one 64-key block, or 64/(block_n/l) small blocks of the same
//    level packed side by side.  All tiles therefore cost the same MFMA work whatever their level; only the
//    last tile of a level can be partly empty.
//  * K and V tiles go from global memory straight into LDS (global_load_lds_dwordx4: no staging registers, no
//    VALU work), both row-major, double buffered, in the padded + swizzled layout of psa_tiles.h.  K operands
//    are 128-bit LDS reads; V operands come through ds_read_b64_tr_b16, which hands every lane 4 keys of one
//    channel: exactly the A operand of O^T += V^T P^T, in the key order that the S^T accumulator layout gives
//    P^T.  All operand addresses are lane base + immediate (the tile loop is unrolled by two for that).
//  * The kernel computes the transposed problem  S^T = K Q^T  (32 keys x 32 queries per MFMA,
//    v_mfma_f32_32x32x16_bf16) and  O^T += V^T P^T.  In the MFMA accumulator layout a lane then holds 16 keys of
//    ONE query column: the softmax row max / row sum are in-lane reductions plus a single exchange between the
//    two half-waves (v_permlane32_swap), and P^T is already in B-operand layout.
//  * Online softmax in base 2: p = exp2(s*scale*log2e + log2(level) - m); the reference maximum is only raised
//    when it lags by more than 2^8 (lazy rescaling), so most tiles skip the accumulator rescale.  Row sums add
//    the bf16-ROUNDED probabilities (v_dot2_f32_bf16): numerator and denominator use the same values.
//  * One barrier per tile: copy of tile t+1 in flight | QK(t) | softmax(t) | PV(t) | barrier.
//  * Rows are issued in groups (group g on XCD g mod 8, a few heads per phase of 8 groups) and, with the
//    optional workspace, longest first inside a group.
//
// Roofline: MFMA-bound; 4*BM*64*D flops per tile.
#include <type_traits>

#include "psa_common.h"
#include "psa_tiles.h"

namespace {

constexpr int TK = 64;              // pooled keys per tile
constexpr float LAZY_THRESHOLD = 8.f;  // log2 units the running max may lag behind

struct FwdParams {
  const bf16_t *q, *k, *v;
  int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, o_sb, o_sh, o_sl;
  const bf16_t *kp, *vp;  // pooled levels 2,4,8 (may be null when map is null)
  const void* map;
  int map_elem;
  bf16_t* o;
  float* lse;
  int B, Hq, Hkv, L, Mq, Nk, bn_log2, bm;
  int64_t npad;
  float scale_log2;
  int causal;
  int total_wg, wg_chunk, wg_groups;  // rows are dealt in wg_groups groups of wg_chunk; group g runs on XCD g % 8
  int max_tiles;
  const int32_t* order;  // optional: logical workgroup id -> (b, h, q-block) row, longest rows first per XCD
};

constexpr int F_ISTR = psa_tiles::LT_ISTR;  // bytes between the blocks of a tile


#define TILE_SYNC()                         \
  do {                                      \
    __builtin_amdgcn_s_waitcnt(0x0f70);     \
    __syncthreads();                        \
  } while (0)

template <int D, int NW>
__global__ __launch_bounds__(NW * 64, 2) void psa_fwd_lds_kernel(FwdParams p) {
  using G = psa_tiles::LtGeom<D>;
  constexpr int F_TILE = G::TILE;  // bytes of one K or V tile
  constexpr int NT = NW * 64, BM = NW * 32, KK = D / 16, DB = D / 32, CH = D / 8;
  constexpr int G16 = 4 / NW;  // 16-row groups of a tile fetched by one wave
  constexpr int OST = D * 2 + 16;
  static_assert(NW == 4 || NW == 2 || NW == 1, "1, 2 or 4 waves");
  static_assert(BM * OST <= 4 * F_TILE, "O staging must fit the tile buffers");
  const auto P_L = p.L;
  const auto P_bn_log2 = p.bn_log2;
  const auto P_causal = p.causal;
  const auto P_scale_log2 = p.scale_log2;
  const auto P_npad = p.npad;
  const auto P_kp = p.kp;
  const auto P_vp = p.vp;
  const uint32_t P_k_strb = (uint32_t)p.k_sl * 2u, P_v_strb = (uint32_t)p.v_sl * 2u;

  extern __shared__ __align__(16) unsigned char smem[];
  // K buffers at 0 and F_TILE, V buffers at 2*F_TILE and 3*F_TILE
  u32x2* tdesc = (u32x2*)(smem + 4 * F_TILE);
  uint16_t* ids = (uint16_t*)(tdesc + p.max_tiles);
  __shared__ int s_cnt[4], s_ioff[4], s_toff[5], s_wcnt[4 * NW];

  const int bid = blockIdx.x;
  // workgroup ids go round-robin over the 8 XCDs; slot s of XCD x works on row (s % chunk) of group 8*(s / chunk) + x
  int logical = (((bid >> 3) / p.wg_chunk) * 8 + (bid & 7)) * p.wg_chunk + (bid >> 3) % p.wg_chunk;
  if (p.order != nullptr) logical = p.order[logical];
  if (logical < 0 || logical >= p.total_wg) return;
  const int I = logical % p.Mq;
  const int bh = logical / p.Mq;
  const int h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;

  int jmax = p.Nk;
  if (P_causal) {
    const int ce = (int)((((int64_t)(I + 1) * p.bm) + (1 << P_bn_log2) - 1) >> P_bn_log2);
    jmax = ce < jmax ? ce : jmax;
  }
  // Q fragments (B operand of S^T = K Q^T): lane holds Q[row l32][16*kk + 8*hh .. +8]
  const int q_row0 = I * BM + wave * 32;
  const int q_idx = q_row0 + l32;
  bf16x8 qf[KK];
  {
    const int qr = q_idx < P_L ? q_idx : P_L - 1;
    const bf16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)qr * p.q_sl + hh * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const bf16x8*)(qp + kk * 16);
  }
  const int T = psa_tiles::build_row_schedule<NT>(p.map, p.map_elem, ((int64_t)bh * p.Mq + I) * p.Nk, p.Nk, jmax, P_bn_log2,
                                                 P_L, P_causal != 0, (int64_t)I * p.bm, ids, tdesc, s_cnt, s_ioff, s_toff, s_wcnt);

  const char* kb0 = (const char*)(p.k + b * p.k_sb + hk * p.k_sh);
  const char* vb0 = (const char*)(p.v + b * p.v_sb + hk * p.v_sh);
  const int64_t BHkv = (int64_t)p.B * p.Hkv, bhk = (int64_t)b * p.Hkv + hk;

  // ---- lane-invariant addressing (tile layout: psa_tiles.h) -------------------------------------------
  const uint32_t f_chunk = psa_tiles::lt_fetch_chunk<D>(lane);
  uint32_t k_off[2], v_off[2];
  psa_tiles::lt_row_operand<D>(l32, hh, k_off);  // K rows l32 (+32): k_off[kk & 1] + 64 * (kk >> 1) (+ 8 blocks)
  psa_tiles::lt_tr_operand<D>(lane, v_off);      // V^T: v_off[s] + 64 * db + 4 * F_ISTR * cg

  psa_tiles::KvSource kvs;
  kvs.k0 = kb0; kvs.v0 = vb0; kvs.kp = (const char*)P_kp; kvs.vp = (const char*)P_vp;
  kvs.k_strb = P_k_strb; kvs.v_strb = P_v_strb;
  kvs.BHkv = BHkv; kvs.bhk = bhk; kvs.npad = P_npad; kvs.bn_log2 = P_bn_log2; kvs.L = P_L;
  using TileSrc = psa_tiles::TileSrc<G16>;
  auto tile_src = [&](int t, TileSrc& a) __attribute__((always_inline)) { psa_tiles::lt_tile_src<D, G16>(kvs, tdesc, ids, t, wave, lane, a); };
  auto issue_rows = [&](const char* base, uint32_t str, int lim, const int (&src0)[G16], int lds_byte) __attribute__((always_inline)) {
    psa_tiles::lt_issue_rows<D, G16>(smem + lds_byte, base, str, lim, src0, wave, f_chunk);
  };

  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
  float m_run = -INFINITY;  // running reference max (log2 domain), same in both half-waves
  float l_run = 0.f;        // this lane's partial row sum
  const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};

  // masks (if needed) and reduces the logits of tile t; returns the bias - reference max and the rescale factor
  auto softmax_head = [&](int t, f32x16 (&s_cur)[2], float& nb, float& alpha) __attribute__((always_inline)) {
    const uint32_t d = __builtin_amdgcn_readfirstlane(tdesc[t][0]);
    const int lv = d & 3;
    if (d & 4) {
      // Partly empty tile and/or causal diagonal.  Valid slots are a prefix of the tile (nvalid), and a
      // pooled key of level lv is visible to query i once its last token is: ((src + 1) << lv) - 1 <= i, i.e.
      // src < (i + 1) >> lv.  Both limits cut each run of 4 consecutive slots after its first `keep` elements.
      const int nvalid = (int)((d >> 3) & 127);
      const int qlim = (q_idx + 1) >> lv;
      const uint32_t d1 = __builtin_amdgcn_readfirstlane(tdesc[t][1]);
      const int cnt = (int)(d1 >> 16), lt = (int)(d >> 10), sbs_log2 = P_bn_log2 - lv;
      const uint16_t* lids = ids + (d1 & 0xffff);
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int r0 = c * 32 + g * 8 + hh * 4;
          int keep = nvalid - r0;
          if (P_causal) {
            const int gpos = (lt << 6) + r0;
            int bi = gpos >> sbs_log2;
            bi = bi < cnt - 1 ? bi : cnt - 1;
            const int src0 = ((int)lids[bi] << sbs_log2) + (gpos & ((1 << sbs_log2) - 1));
            keep = keep < qlim - src0 ? keep : qlim - src0;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) s_cur[c][g * 4 + e] = e < keep ? s_cur[c][g * 4 + e] : -INFINITY;
        }
    }
    float mx0 = s_cur[0][0], mx1 = s_cur[1][0];
#pragma unroll
    for (int i = 1; i < 15; i += 2) {
      mx0 = max3f(mx0, s_cur[0][i], s_cur[0][i + 1]);
      mx1 = max3f(mx1, s_cur[1][i], s_cur[1][i + 1]);
    }
    float mx = max3f(mx0, s_cur[0][15], fmaxf(mx1, s_cur[1][15]));
    mx = half_wave_max(mx);
    const float bias = (float)lv;
    const float m_cand = __builtin_fmaf(mx, P_scale_log2, bias);
    // raise the reference max only when it lags by more than the threshold (or is still -inf)
    float m_new = (m_cand - m_run > LAZY_THRESHOLD) ? m_cand : m_run;
    m_new = (m_run == -INFINITY) ? m_cand : m_new;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // rows that still see no key
    alpha = fast_exp2(m_run - m_use);
    nb = bias - m_use;
    m_run = m_new;
  };
  // probabilities of 4 logits: exp2, round to bf16, add the ROUNDED values (the ones that multiply V) to the row sum
  auto prob4 = [&](const f32x16& sc, int i, float nb, uint32_t* pk2, float& lsum) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 4; e += 2) {
      const float p0 = fast_exp2(__builtin_fmaf(sc[i + e], P_scale_log2, nb));
      const float p1 = fast_exp2(__builtin_fmaf(sc[i + e + 1], P_scale_log2, nb));
      pk2[e >> 1] = pack_bf16x2(p0, p1);
      lsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pk2[e >> 1]), ones, lsum, false);
    }
  };
  // exponentials of the 16 logits of one 32-key half (4 groups of 4)
  auto prob16 = [&](const f32x16& sc, float nb, uint32_t* pk8, float& lsum) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) prob4(sc, i * 4, nb, pk8 + i * 2, lsum);
  };
  // Both halves of S^T at once: two independent accumulation chains, operands fetched one k-step ahead.
  auto qk_full = [&](auto kb_c, f32x16 (&s2)[2]) __attribute__((always_inline)) {
    constexpr int KB = decltype(kb_c)::value;
    PSA_LDS(unsigned char) Ks = (PSA_LDS(unsigned char))(smem) + KB * F_TILE;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) s2[c][i] = 0.f;
    bf16x8 a0 = *(PSA_LDS(const bf16x8))(Ks + k_off[0]), a1 = *(PSA_LDS(const bf16x8))(Ks + k_off[0] + G::HALF);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      bf16x8 n0 = a0, n1 = a1;
      if (kk + 1 < KK) {
        n0 = *(PSA_LDS(const bf16x8))(Ks + k_off[(kk + 1) & 1] + ((kk + 1) >> 1) * 64);
        n1 = *(PSA_LDS(const bf16x8))(Ks + k_off[(kk + 1) & 1] + ((kk + 1) >> 1) * 64 + G::HALF);
      }
      s2[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, qf[kk], s2[0], 0, 0, 0);
      s2[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, qf[kk], s2[1], 0, 0, 0);
      a0 = n0;
      a1 = n1;
    }
  };
  // Half hf (32 keys) of O^T += V^T P^T from V buffer VB: per 16-key group cg, A = V^T[32 d][16 keys] (two
  // transposing reads), B = P^T.  8 MFMAs on 4 independent accumulators.
  auto pv_half = [&](auto vb_c, int hf, const uint32_t* pk8) __attribute__((always_inline)) {
    constexpr int VB = decltype(vb_c)::value;
    PSA_LDS(unsigned char) Vs = (PSA_LDS(unsigned char))(smem) + (2 + VB) * F_TILE + hf * G::HALF;
    // operand of MFMA step st = DB*g + db; reads run AHEAD steps in front of the MFMAs
    constexpr int AHEAD = 2, STEPS = 2 * DB;
    auto vread = [&](int st, int s) __attribute__((always_inline)) {
      return __builtin_bit_cast(
          u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((PSA_LDS(bf16x4))(Vs + v_off[s] + (st % DB) * 64 + (st / DB) * G::GROUP)));
    };
    u32x2 vlo[STEPS], vhi[STEPS];  // fully unrolled: every element is a short-lived register value
#pragma unroll
    for (int st = 0; st < AHEAD; ++st) {
      vlo[st] = vread(st, 0);
      vhi[st] = vread(st, 1);
    }
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      const int g = st / DB, db = st % DB;
      if (st + AHEAD < STEPS) {
        vlo[st + AHEAD] = vread(st + AHEAD, 0);
        vhi[st + AHEAD] = vread(st + AHEAD, 1);
      }
      u32x4 bw = {pk8[g * 4 + 0], pk8[g * 4 + 1], pk8[g * 4 + 2], pk8[g * 4 + 3]};
      u32x4 aw = {vlo[st][0], vlo[st][1], vhi[st][0], vhi[st][1]};
      acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, aw), __builtin_bit_cast(bf16x8, bw), acc[db], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);  // keep the reads AHEAD steps in front, not more
    }
  };
  auto rescale_acc = [&](float alpha) __attribute__((always_inline)) {
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][i] *= alpha;
    }
  };
  const std::integral_constant<int, 0> B0;
  const std::integral_constant<int, 1> B1;

  // Per tile: DMA tile t+1 | QK(t) | softmax(t) | PV(t) | barrier.  The MFMA phases of one workgroup overlap
  // the softmax of the other workgroup on the CU.  (Interleaving the exponentials of tile t with the MFMAs of
  // tiles t-1 / t+1 inside one wave was measured and is slower: it serialises the MFMA chains and costs registers.)
  if (T > 0) {
    TileSrc ts;
    f32x16 s[2];
    uint32_t pk[2][8];
    tile_src(0, ts);
    issue_rows(ts.kbase, ts.kstr, ts.lim, ts.src0, 0);
    issue_rows(ts.vbase, ts.vstr, ts.lim, ts.src0, 2 * F_TILE);
    TILE_SYNC();
    auto step = [&](int t, auto cur_c) __attribute__((always_inline)) {
      constexpr int CUR = decltype(cur_c)::value;
      if (t + 1 < T) {
        tile_src(t + 1, ts);
        issue_rows(ts.kbase, ts.kstr, ts.lim, ts.src0, (CUR ^ 1) * F_TILE);
        issue_rows(ts.vbase, ts.vstr, ts.lim, ts.src0, (2 + (CUR ^ 1)) * F_TILE);
      }
      float nb, alpha, lsum = 0.f;
      qk_full(cur_c, s);
      softmax_head(t, s, nb, alpha);
      prob16(s[0], nb, pk[0], lsum);
      prob16(s[1], nb, pk[1], lsum);
      l_run = l_run * alpha + lsum;
      rescale_acc(alpha);
      pv_half(cur_c, 0, pk[0]);
      pv_half(cur_c, 1, pk[1]);
      TILE_SYNC();
    };
    for (int t = 0; t < T; t += 2) {
      step(t, B0);
      if (t + 1 < T) step(t + 1, B1);
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------------------
  float l_tot = half_wave_sum(l_run);
  const float l_safe = fmaxf(l_tot, 1e-8f);
  const float inv = 1.0f / l_safe;
  if (p.lse != nullptr && hh == 0 && q_idx < P_L) {
    // natural-log domain: m*ln2 + ln(max(l, 1e-8))
    p.lse[((int64_t)b * p.Hq + h) * P_L + q_idx] = (m_run + fast_log2(l_safe)) * 0.6931471805599453f;
  }
  __syncthreads();  // everyone is done with the last K/V tile
  unsigned char* Os = smem;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w[0] = pack_bf16x2(acc[db][g * 4 + 0] * inv, acc[db][g * 4 + 1] * inv);
      w[1] = pack_bf16x2(acc[db][g * 4 + 2] * inv, acc[db][g * 4 + 3] * inv);
      *(u32x2*)(Os + (wave * 32 + l32) * OST + (db * 32 + g * 8 + hh * 4) * 2) = w;
    }
  __syncthreads();
  bf16_t* ob = p.o + b * p.o_sb + h * p.o_sh;
  for (int u = tid; u < BM * CH; u += NT) {
    const int r = u / CH, ch = u % CH;
    const int row = I * BM + r;
    if (row < P_L) *(u32x4*)(ob + (int64_t)row * p.o_sl + ch * 8) = *(const u32x4*)(Os + r * OST + ch * 16);
  }
}

// ---- longest-rows-first ordering ---------------------------------------------------------------------
// Rows of the level map differ in the number of tiles they retain.  Workgroup ids are dealt round-robin
// to the 8 XCDs and each XCD runs its ids in order, so sorting every XCD's share by decreasing tile count
// shortens the tail of the launch.  The order only changes WHEN a row is computed, never its result.
constexpr int COST_BINS = 2048;
constexpr int FWD_MAX_PHASES = 64;
constexpr int64_t FWD_PHASE_BYTES = 128ll << 20;  // K/V (+ pooled levels) in use at one time

__global__ __launch_bounds__(256) void psa_fwd_cost_kernel(const void* map, int map_elem, int total, int Mq, int Nk, int bn_log2,
                                                         int bm, int causal, int32_t* cost) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= total) return;
  const int I = row % Mq;
  int jmax = Nk;
  if (causal) {
    const int ce = (int)((((int64_t)(I + 1) * bm) + (1 << bn_log2) - 1) >> bn_log2);
    jmax = ce < jmax ? ce : jmax;
  }
  int cnt[4] = {0, 0, 0, 0};
  for (int j0 = 0; j0 < jmax; j0 += 64) {
    const int j = j0 + lane;
    const int lvl = j < jmax ? load_map(map, (int64_t)row * Nk + j, map_elem) : 0;
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) cnt[lv] += __popcll(__ballot(lvl == (1 << lv)));
  }
  if (lane == 0) {
    int tiles = 0;
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) tiles += ((cnt[lv] << (bn_log2 - lv)) + 63) >> 6;
    cost[row] = tiles < COST_BINS - 1 ? tiles : COST_BINS - 1;
  }
}

// one workgroup per group of rows: counting sort by decreasing cost
__global__ __launch_bounds__(256) void psa_fwd_sort_kernel(const int32_t* cost, int total, int chunk, int32_t* order) {
  __shared__ int hist[COST_BINS];
  const int x = blockIdx.x, tid = threadIdx.x;
  const int r0 = x * chunk;
  for (int i = tid; i < COST_BINS; i += 256) hist[i] = 0;
  __syncthreads();
  for (int i = tid; i < chunk; i += 256)
    if (r0 + i < total) atomicAdd(&hist[cost[r0 + i]], 1);
  __syncthreads();
  {  // start offset of every bin, highest cost first: thread i owns the 8 bins COST_BINS-1-8i .. COST_BINS-8-8i
    __shared__ int part[256];
    constexpr int PER = COST_BINS / 256;
    int c[PER], sum = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      c[j] = hist[COST_BINS - 1 - (tid * PER + j)];
      sum += c[j];
    }
    part[tid] = sum;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {  // inclusive scan over the threads
      const int add = tid >= d ? part[tid - d] : 0;
      __syncthreads();
      part[tid] += add;
      __syncthreads();
    }
    int run = part[tid] - sum;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      hist[COST_BINS - 1 - (tid * PER + j)] = run;
      run += c[j];
    }
  }
  __syncthreads();
  for (int i = tid; i < chunk; i += 256) {
    if (r0 + i < total) order[r0 + atomicAdd(&hist[cost[r0 + i]], 1)] = r0 + i;
  }
  // ids past the last row of the last share
  const int valid = total - r0 < chunk ? (total - r0 > 0 ? total - r0 : 0) : chunk;
  for (int i = valid + tid; i < chunk; i += 256) order[r0 + i] = -1;
}

template <int D, int NW>
int launch_fwd(const FwdParams& p, int Nk, hipStream_t stream) {
  size_t shmem = (size_t)4 * psa_tiles::LtGeom<D>::TILE + (size_t)p.max_tiles * 8 + (size_t)Nk * 2;
  if (shmem > 160 * 1024) return PSA_ERR_UNSUPPORTED;
  if (hipFuncSetAttribute((const void*)psa_fwd_lds_kernel<D, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess)
    return PSA_ERR_LAUNCH;
  hipLaunchKernelGGL((psa_fwd_lds_kernel<D, NW>), dim3((unsigned)(p.wg_chunk * p.wg_groups)), dim3(NW * 64), shmem, stream, p);
  return PSA_OK;
}

}  // namespace

extern "C" int64_t psa_fwd_workspace_bytes(int B, int Hq, int L, int block_m) {
  if (B <= 0 || Hq <= 0 || L <= 0 || block_m <= 0) return 0;
  const int64_t total = (int64_t)B * Hq * ((L + block_m - 1) / block_m);
  return 2 * (total + 8 * FWD_MAX_PHASES) * (int64_t)sizeof(int32_t);  // any grouping of the rows fits
}

extern "C" int psa_fwd(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool,
                       const void* map, int map_elem_bytes, psa_tensor4 out, float* lse, int B, int Hq, int Hkv, int L,
                       int D, int block_m, int block_n, float sm_scale, int causal, void* workspace, psa_stream_t stream) {
  PSA_REQUIRE(q.ptr && k.ptr && v.ptr && out.ptr, PSA_ERR_ARG, "psa_fwd: null pointer");
  PSA_REQUIRE(map == nullptr || (k_pool && v_pool), PSA_ERR_ARG, "psa_fwd: pooled K/V required with a level map");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_fwd: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && L > 0, PSA_ERR_ARG, "psa_fwd: B, H, L must be positive");
  PSA_REQUIRE(Hq % Hkv == 0, PSA_ERR_ARG, "psa_fwd: Hq=%d must be a multiple of Hkv=%d", Hq, Hkv);
  PSA_REQUIRE(sm_scale > 0.f, PSA_ERR_ARG, "psa_fwd: sm_scale must be positive");
  PSA_REQUIRE(D == 64 || D == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: head dim %d not in {64, 128}", D);
  PSA_REQUIRE(block_m == 64 || block_m == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: block_m=%d not in {64, 128}", block_m);
  PSA_REQUIRE(block_n == 32 || block_n == 64 || block_n == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: block_n=%d not in {32, 64, 128}", block_n);
  const psa_tensor4* ts[4] = {&q, &k, &v, &out};
  for (int i = 0; i < 4; ++i)
    PSA_REQUIRE(((uintptr_t)ts[i]->ptr % 16 == 0) && ts[i]->stride_b % 8 == 0 && ts[i]->stride_h % 8 == 0 && ts[i]->stride_l % 8 == 0,
                PSA_ERR_UNSUPPORTED, "psa_fwd: tensors must be 16-byte aligned with strides that are multiples of 8 elements");
  PSA_REQUIRE((int64_t)L * k.stride_l * 2 < (1ll << 32) && (int64_t)L * v.stride_l * 2 < (1ll << 32), PSA_ERR_UNSUPPORTED,
              "psa_fwd: one (batch, head) slice of K/V must span less than 4 GiB");
  const int Mq = (L + block_m - 1) / block_m, Nk = (L + block_n - 1) / block_n;
  PSA_REQUIRE(Nk <= 65535, PSA_ERR_UNSUPPORTED, "psa_fwd: more than 65535 kv-blocks");
  const int64_t total = (int64_t)B * Hq * Mq;
  PSA_REQUIRE(total < (1ll << 28), PSA_ERR_UNSUPPORTED, "psa_fwd: too many workgroups");
  FwdParams p;
  p.q = (const bf16_t*)q.ptr; p.k = (const bf16_t*)k.ptr; p.v = (const bf16_t*)v.ptr; p.o = (bf16_t*)out.ptr;
  p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sl = q.stride_l;
  p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sl = k.stride_l;
  p.v_sb = v.stride_b; p.v_sh = v.stride_h; p.v_sl = v.stride_l;
  p.o_sb = out.stride_b; p.o_sh = out.stride_h; p.o_sl = out.stride_l;
  p.kp = (const bf16_t*)k_pool; p.vp = (const bf16_t*)v_pool;
  p.map = map; p.map_elem = map_elem_bytes; p.lse = lse;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.L = L; p.Mq = Mq; p.Nk = Nk;
  p.bn_log2 = psa_ilog2(block_n); p.bm = block_m;
  p.npad = (int64_t)Nk * block_n;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  p.causal = causal ? 1 : 0;
  p.total_wg = (int)total;
  // Groups of rows run one after the other on each XCD.  With several phases (8 groups each) the K/V of only a
  // few heads is in use at a time, so that the part of it that misses L2 can stay in the last-level cache.
  int phases = 1;
  {
    const double kv_bytes = 2.0 * B * Hkv * ((double)Nk * block_n) * D * 2.0 * (map != nullptr ? 1.875 : 1.0);
    phases = (int)(kv_bytes / (double)FWD_PHASE_BYTES) + 1;
    const int max_phases = B * Hkv < FWD_MAX_PHASES ? B * Hkv : FWD_MAX_PHASES;
    phases = phases > max_phases ? max_phases : phases;
  }
  p.wg_groups = 8 * phases;
  p.wg_chunk = (int)((total + p.wg_groups - 1) / p.wg_groups);
  // worst case: every kv-block at level 1, plus one partly filled tile per pooled level
  p.max_tiles = (block_n >= 64 ? Nk * (block_n / 64) : (Nk * block_n + 63) / 64) + 4;
  p.order = nullptr;
  if (workspace != nullptr && map != nullptr && total > 8 * 32) {
    PSA_REQUIRE((uintptr_t)workspace % 4 == 0, PSA_ERR_ARG, "psa_fwd: workspace must be 4-byte aligned");
    int32_t* order = (int32_t*)workspace;
    int32_t* cost = order + (int64_t)p.wg_chunk * p.wg_groups;
    hipLaunchKernelGGL(psa_fwd_cost_kernel, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, (hipStream_t)stream, map, map_elem_bytes,
                       (int)total, Mq, Nk, p.bn_log2, block_m, p.causal, cost);
    if (int e = psa_check_launch("psa_fwd (row cost)")) return e;
    hipLaunchKernelGGL(psa_fwd_sort_kernel, dim3(p.wg_groups), dim3(256), 0, (hipStream_t)stream, cost, (int)total, p.wg_chunk, order);
    if (int e = psa_check_launch("psa_fwd (row order)")) return e;
    p.order = order;
  }
  int rc;
  if (D == 128 && block_m == 128) rc = launch_fwd<128, 4>(p, Nk, (hipStream_t)stream);
  else if (D == 128) rc = launch_fwd<128, 2>(p, Nk, (hipStream_t)stream);
  else if (block_m == 128) rc = launch_fwd<64, 4>(p, Nk, (hipStream_t)stream);
  else rc = launch_fwd<64, 2>(p, Nk, (hipStream_t)stream);
  PSA_REQUIRE(rc == PSA_OK, rc, "psa_fwd: sequence too long for the on-chip schedule (LDS)");
  return psa_check_launch("psa_fwd");
}
