// Pyramid sparse attention forward (non-causal and causal) on bf16 MFMA.
//
// psa_fwd_lds_kernel: one workgroup per (batch, head, q-block of BM = 32*NW rows); every wave owns 32 query rows;
// two workgroups per CU.  psa_fwd_pp_kernel (head dim 128, 128-row q-blocks, the usual case): two rows per
// workgroup of 8 waves, see there.  Both share the points below.
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
//    when it lags by more than 2^8 (lazy rescaling), so most tiles skip the accumulator rescale.  Row sums: the
//    one-row kernel adds the bf16-ROUNDED probabilities (v_dot2_f32_bf16: numerator and denominator use the same
//    values), the two-row kernel the unrounded ones with plain adds as the reference does (a dot-product
//    instruction runs on the matrix pipe and would queue behind the other group's MFMAs).
//  * One-row kernel: one barrier per tile: copy of tile t+1 in flight | QK(t) | softmax(t) | PV(t) | barrier.
//  * Rows are issued in groups (group g on XCD g mod 8, a few heads per phase of 8 groups) and, with the
//    optional workspace, longest first inside a group.
//
// Roofline: MFMA-bound; 4*BM*64*D flops per tile.
#include <type_traits>

#include "psa_common.h"
#include "psa_tiles.h"
#include "psa_order.h"
#include "psa_schedule.h"

// fp32 tensors: psa_f32.hip
int psa_fwd_f32(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool, const void* map, int map_elem_bytes,
                psa_tensor4 out, float* lse, int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, float sm_scale, int causal,
                psa_stream_t stream, const int32_t* q_index);

namespace {

#ifndef PSA_FWD_ONE_GROUP
#define PSA_FWD_ONE_GROUP 0
#endif
constexpr int TK = 64;              // pooled keys per tile
template <int V>
using IC = std::integral_constant<int, V>;
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(IC<Is>{}), ...);
}
// f(IC<0>{}), ..., f(IC<N-1>{}): a loop whose index is a compile-time constant in the body
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

constexpr float LAZY_THRESHOLD = 8.f;  // log2 units the running max may lag behind

struct FwdParams {
  const uint16_t *q, *k, *v;  // bf16 or fp16: the kernel's element trait says which
  int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, o_sb, o_sh, o_sl;
  const uint16_t *kp, *vp;  // pooled levels 2,4,8 (may be null when map is null)
  const void* map;
  int map_elem;
  uint16_t* o;
  float* lse;
  int B, Hq, Hkv, L, Mq, Nk, bn_log2, bm;
  int64_t npad;
  float scale_log2;
  int causal;
  int total_wg, wg_chunk, wg_groups;  // rows are dealt in wg_groups groups of wg_chunk; group g runs on XCD g % 8
  int max_tiles;
  int grp_bytes;  // two-group kernel: LDS bytes of one group (tile buffers + schedule)
  const int32_t* order;  // optional: logical workgroup id -> (b, h, q-block) row, longest rows first per XCD
  const int32_t* q_index;  // optional (token re-ordering): query / output position i lives in row q_index[i] of q, out, lse
  int dtype;               // PSA_DTYPE_BF16 / PSA_DTYPE_F16
  // prebuilt tile schedule (psa_schedule.h), scheduled kernel only: tiles per row and the rows' tile records
  const u32x4* sched_rec;
  const int32_t* sched_tiles;
  int rec_stride;
};

constexpr int F_ISTR = psa_tiles::LT_ISTR;  // bytes between the blocks of a tile


#define TILE_SYNC()                         \
  do {                                      \
    __builtin_amdgcn_s_waitcnt(0x0f70);     \
    __syncthreads();                        \
  } while (0)

// GS: the row's tiles come from a prebuilt schedule (psa_schedule.h) as in the two-group kernel below: one scalar word
// per wave and tile instead of a per-lane look-up, copies addressed from scalar registers.
template <int D, int NW, bool GS, class ET>
__global__ __launch_bounds__(NW * 64, 2) void psa_fwd_lds_kernel(FwdParams p) {
  using x8 = typename ET::x8;
  using G = psa_tiles::LtGeom<D>;
  constexpr int F_TILE = G::TILE;  // bytes of one K or V tile
  constexpr int NT = NW * 64, BM = NW * 32, KK = D / 16, DB = D / 32, CH = D / 8;
  constexpr int G16 = 4 / NW;  // 16-row groups of a tile fetched by one wave
  constexpr int OST = D * 2 + 16;
  static_assert(NW == 4 || NW == 2 || NW == 1, "1, 2 or 4 waves");
  static_assert(!GS || NW == 4, "schedules describe 128-row q-blocks: one 16-row quarter of a tile per wave");
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
  x8 qf[KK];
  {
    int qr = q_idx < P_L ? q_idx : P_L - 1;
    if (p.q_index != nullptr) qr = clamp_row(p.q_index[qr], P_L);
    const uint16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)qr * p.q_sl + hh * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const x8*)(qp + kk * 16);
  }
  using w_ptr = const __attribute__((address_space(4))) uint32_t*;
  using rec_ptr = const __attribute__((address_space(4))) u32x4*;
  rec_ptr recs = nullptr;
  int T;
  if constexpr (GS) {
    recs = (rec_ptr)(uintptr_t)(p.sched_rec + (int64_t)logical * p.rec_stride);
    T = __builtin_amdgcn_readfirstlane(p.sched_tiles[logical]);
  } else {
    T = psa_tiles::build_row_schedule<NT>(p.map, p.map_elem, ((int64_t)bh * p.Mq + I) * p.Nk, p.Nk, jmax, P_bn_log2, P_L,
                                          P_causal != 0, (int64_t)I * p.bm, ids, tdesc, s_cnt, s_ioff, s_toff, s_wcnt);
  }

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

  // masks (if needed) and reduces the logits of tile t; returns the bias - reference max and the rescale factor
  uint32_t w_cur = 0;  // GS: this wave's word of the record of the tile whose logits are being reduced
  auto softmax_head = [&](int t, f32x16 (&s_cur)[2], float& nb, float& alpha) __attribute__((always_inline)) {
    uint32_t d;
    if constexpr (GS) d = ((w_cur >> psa_sched::REC_CODE_SHIFT) & 3u) | ((w_cur >> (psa_sched::REC_MASKED_BIT - 2)) & 4u);  // level | masked << 2
    else d = __builtin_amdgcn_readfirstlane(tdesc[t][0]);
    const int lv = d & 3;
    if constexpr (GS) {
      if (d & 4) {
        const int nvalid = psa_sched::rec_nvalid(w_cur);
        const int qlim = (q_idx + 1) >> lv;
        u32x4 r4 = {0u, 0u, 0u, 0u};
        if (P_causal) r4 = recs[t];  // the source rows of all four quarters (rare path: fetched on demand)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int r0 = c * 32 + g * 8 + hh * 4;
            int keep = nvalid - r0;
            if (P_causal) {
              // slots r0 .. r0+3 lie in quarter 2c + g/2 of the tile, whose source rows are consecutive
              const int src0 = psa_sched::rec_src(r4[c * 2 + (g >> 1)]) + (g & 1) * 8 + hh * 4;
              keep = keep < qlim - src0 ? keep : qlim - src0;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) s_cur[c][g * 4 + e] = e < keep ? s_cur[c][g * 4 + e] : -INFINITY;
          }
      }
    } else if (d & 4) {
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
      pk2[e >> 1] = ET::pack2(p0, p1);
      lsum = ET::add_pair(pk2[e >> 1], lsum);
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
    x8 a0 = *(PSA_LDS(const x8))(Ks + k_off[0]), a1 = *(PSA_LDS(const x8))(Ks + k_off[0] + G::HALF);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      x8 n0 = a0, n1 = a1;
      if (kk + 1 < KK) {
        n0 = *(PSA_LDS(const x8))(Ks + k_off[(kk + 1) & 1] + ((kk + 1) >> 1) * 64);
        n1 = *(PSA_LDS(const x8))(Ks + k_off[(kk + 1) & 1] + ((kk + 1) >> 1) * 64 + G::HALF);
      }
      s2[0] = ET::mfma(a0, qf[kk], s2[0]);
      s2[1] = ET::mfma(a1, qf[kk], s2[1]);
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
      return ET::read_tr(Vs + v_off[s] + (st % DB) * 64 + (st / DB) * G::GROUP);
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
      acc[db] = ET::mfma(__builtin_bit_cast(x8, aw), __builtin_bit_cast(x8, bw), acc[db]);
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
  // GS: copies addressed from scalar registers (see the two-group kernel for the scheme)
  const int lane_row = psa_tiles::lt_fetch_row<D>(lane);
  const uint32_t voff_s = (uint32_t)lane_row * (uint32_t)(D * 2) + f_chunk;
  const uint32_t wave_lds = psa_tiles::lds_addr_of(smem) + (uint32_t)(wave * G::RPL * F_ISTR);
  auto pool_base = [&](const uint16_t* pool, int lv) __attribute__((always_inline)) {
    return (const char*)pool + (BHkv * (P_npad - (P_npad >> (lv - 1))) + bhk * (P_npad >> lv)) * (D * 2);
  };
  struct Stream {  // where one tensor's tiles currently come from: a level's rows (the level changes 3 times per row)
    const char* base;
    uint32_t code;
  };
  Stream st_k = {kb0, 0u}, st_v = {vb0, 0u};
  auto issue_tile = [&](Stream& st, bool is_k, uint32_t w, auto lds_byte) __attribute__((always_inline)) {
    const uint32_t code = psa_sched::rec_code(w);
    bool rag = false;
    if (code != st.code) {
      const int lv = (int)(code & 3u);
      st.code = code & 3u;  // (a ragged tile comes back here for every tile)
      const uint16_t* pool = is_k ? P_kp : P_vp;
      st.base = lv == 0 ? (is_k ? kb0 : vb0) : pool_base(pool, lv);
      rag = code == psa_sched::REC_CODE_RAGGED;
    }
    if (rag) {
      static_for<G::RPL>([&](auto n) __attribute__((always_inline)) {
        constexpr int N = decltype(n)::value, OFF = decltype(lds_byte)::value + N * F_ISTR;
        const int row = psa_sched::rec_src(w) + lane_row + N;
        psa_tiles::lds_copy16_row<OFF>(st.base, (uint32_t)(row < P_L - 1 ? row : P_L - 1), (uint32_t)(D * 2), f_chunk, wave_lds);
      });
    } else {
      const char* src = st.base + (uint64_t)((w & psa_sched::REC_SRC_MASK) * (uint32_t)(D * 2));
      static_for<G::RPL>([&](auto n) __attribute__((always_inline)) {
        constexpr int N = decltype(n)::value;
        psa_tiles::lds_copy16_imm<decltype(lds_byte)::value + N * F_ISTR, N * D * 2>(src, voff_s, wave_lds);
      });
    }
  };

  if (T > 0) {
    TileSrc ts;
    f32x16 s[2];
    uint32_t pk[2][8];
    w_ptr wp = nullptr;
    uint32_t w_next = 0, w_next2 = 0;  // GS: words of tiles t+1 and t+2 (records T .. T+2 repeat record T-1)
    if constexpr (GS) {
      wp = (w_ptr)(uintptr_t)((const uint32_t*)(p.sched_rec + (int64_t)logical * p.rec_stride) + wave);
      w_cur = wp[0];
      w_next = wp[4];
      w_next2 = wp[8];
      wp += 12;
      issue_tile(st_k, true, w_cur, IC<0>{});
      issue_tile(st_v, false, w_cur, IC<2 * F_TILE>{});
    } else {
      tile_src(0, ts);
      issue_rows(ts.kbase, ts.kstr, ts.lim, ts.src0, 0);
      issue_rows(ts.vbase, ts.vstr, ts.lim, ts.src0, 2 * F_TILE);
    }
    TILE_SYNC();
    auto step = [&](int t, auto cur_c) __attribute__((always_inline)) {
      constexpr int CUR = decltype(cur_c)::value;
      if (t + 1 < T) {
        if constexpr (GS) {
          issue_tile(st_k, true, w_next, IC<(CUR ^ 1) * F_TILE>{});
          issue_tile(st_v, false, w_next, IC<(2 + (CUR ^ 1)) * F_TILE>{});
        } else {
          tile_src(t + 1, ts);
          issue_rows(ts.kbase, ts.kstr, ts.lim, ts.src0, (CUR ^ 1) * F_TILE);
          issue_rows(ts.vbase, ts.vstr, ts.lim, ts.src0, (2 + (CUR ^ 1)) * F_TILE);
        }
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
      if constexpr (GS) {
        w_cur = w_next;
        w_next = w_next2;
        w_next2 = *wp;  // the word of tile t+3 (one scalar load; the records are padded, so no bounds test)
        wp += 4;
      }
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
    const int lrow = p.q_index != nullptr ? p.q_index[q_idx] : q_idx;  // (a row outside 0 .. L-1 is not stored)
    if ((unsigned)lrow < (unsigned)P_L) p.lse[((int64_t)b * p.Hq + h) * P_L + lrow] = (m_run + fast_log2(l_safe)) * 0.6931471805599453f;
  }
  __syncthreads();  // everyone is done with the last K/V tile
  unsigned char* Os = smem;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w[0] = ET::pack2(acc[db][g * 4 + 0] * inv, acc[db][g * 4 + 1] * inv);
      w[1] = ET::pack2(acc[db][g * 4 + 2] * inv, acc[db][g * 4 + 3] * inv);
      *(u32x2*)(Os + (wave * 32 + l32) * OST + (db * 32 + g * 8 + hh * 4) * 2) = w;
    }
  __syncthreads();
  uint16_t* ob = p.o + b * p.o_sb + h * p.o_sh;
  for (int u = tid; u < BM * CH; u += NT) {
    const int r = u / CH, ch = u % CH;
    const int row = I * BM + r;
    if (row < P_L) {
      const int orow = p.q_index != nullptr ? p.q_index[row] : row;
      if ((unsigned)orow < (unsigned)P_L) *(u32x4*)(ob + (int64_t)orow * p.o_sl + ch * 8) = *(const u32x4*)(Os + r * OST + ch * 16);
    }
  }
}

// ---- two-group ("ping-pong") variant -------------------------------------------------------------------
// A SIMD overlaps the MFMAs of one wave with the VALU work of another only while the two are in different
// phases, and two independent workgroups on a CU drift into the same phase.  This kernel therefore puts TWO rows
// of the level map into one workgroup of 2*NW waves - group g = waves g*NW .. g*NW + NW - 1, wave i of either
// group on the same SIMD - and makes the groups alternate under workgroup barriers:
//     group 0:  M0 | V0 | M1 | V1 | ...       M_t = QK(t), then rescale + PV(t-1) with the row maximum of tile t
//     group 1:     | M0 | V0 | M1 | ...             riding along in the shadow of its MFMAs       (matrix pipe)
//                                             V_t = exponentials of tile t, copies of V(t+1) and K(t+2)  (VALU)
// so the matrix phase of one group always runs next to the vector phase of the other.  The groups are otherwise
// independent (own row, own tile buffers and schedule in LDS); rows are paired in issue order, i.e. with the
// longest-first order neighbours of similar length, and the shorter row idles at the barriers of the longer.
// Copies: the buffers of K(t) and V(t-1) were last read in M_t, so V(t+1) and K(t+2) are issued during V_t and
// awaited at the start of V_(t+1), one barrier before M_(t+2) / M_(t+2) read them.
// Only one wave per SIMD is in a given phase, so nothing else hides its latencies: the matrix phase requests its
// operands far ahead, both phases are free of branches, and the copy instructions are spread between the
// exponentials.
#define PP_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

// GS: the rows' tiles come from a prebuilt schedule in device memory (psa_schedule.h; 128-key blocks, K / V rows D
// elements apart) instead of being compacted from the map row here.  A wave fetches ONE word per tile (a scalar load,
// three tiles ahead): level, fill and the first source row of the 16-row quarter it copies.  A wave issues at most one
// instruction per 4 cycles whatever its kind, so what bounds the vector phase is its instruction COUNT: a copy here is
// two instructions (M0, then the load with the row step n * 256 as its immediate offset - which the hardware also adds
// on the LDS side, so M0 carries the difference), the base pointer of a tile's level is kept while the level stays the
// same (tiles of a row are sorted by level), and nothing is looked up per lane.
template <int D, int NW, bool GS, class ET>
__global__ __launch_bounds__(2 * NW * 64, 1) void psa_fwd_pp_kernel(FwdParams p) {
  using x8 = typename ET::x8;
  using G = psa_tiles::LtGeom<D>;
  constexpr int F_TILE = G::TILE;
  constexpr int NT = NW * 64, BM = NW * 32, KK = D / 16, DB = D / 32, CH = D / 8;
  constexpr int G16 = 4 / NW;
  constexpr int OST = D * 2 + 16;
  static_assert(NW == 4, "4 waves per group");
  static_assert(BM * OST <= 4 * F_TILE, "O staging must fit the tile buffers");
  const auto P_L = p.L;
  const auto P_bn_log2 = p.bn_log2;
  const auto P_causal = p.causal;
  const auto P_scale_log2 = p.scale_log2;
  const auto P_npad = p.npad;
  const auto P_kp = p.kp;
  const auto P_vp = p.vp;
  const uint32_t P_k_strb = (uint32_t)p.k_sl * 2u, P_v_strb = (uint32_t)p.v_sl * 2u;

  extern __shared__ __align__(16) unsigned char smem_all[];
  __shared__ int s_cnt[2][4], s_ioff[2][4], s_toff[2][5], s_wcnt[2][4 * NW], s_T[2];
  const int grp = __builtin_amdgcn_readfirstlane((int)threadIdx.x / NT);
  const int tid = (int)threadIdx.x - grp * NT, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hh = lane >> 5;
  const uint32_t grp_base = (uint32_t)grp * (uint32_t)p.grp_bytes;
  unsigned char* smem = smem_all + grp_base;  // this group's K buffers at 0 and F_TILE, V buffers at 2 and 3 F_TILE
  u32x2* tdesc = (u32x2*)(smem + 4 * F_TILE);
  uint16_t* ids = (uint16_t*)(tdesc + p.max_tiles);

  // pair slot of the workgroup (same dealing as the one-row kernel, in units of two rows), then this group's row
  const int bid = blockIdx.x, sc = p.wg_chunk >> 1;
  const int entry = ((((bid >> 3) / sc) * 8 + (bid & 7)) * sc + (bid >> 3) % sc) * 2 + grp;
  int logical = p.order != nullptr ? p.order[entry] : entry;
  logical = __builtin_amdgcn_readfirstlane(logical);
  const bool active = logical >= 0 && logical < p.total_wg;
  if (!active) logical = 0;
  const int I = logical % p.Mq;
  const int bh = logical / p.Mq;
  const int h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);

  int jmax = p.Nk;
  if (P_causal) {
    const int ce = (int)((((int64_t)(I + 1) * p.bm) + (1 << P_bn_log2) - 1) >> P_bn_log2);
    jmax = ce < jmax ? ce : jmax;
  }
  if (!active) jmax = 0;
  const int q_row0 = I * BM + wave * 32;
  const int q_idx = q_row0 + l32;
  x8 qf[KK];
  {
    int qr = q_idx < P_L ? q_idx : P_L - 1;
    if (p.q_index != nullptr) qr = clamp_row(p.q_index[qr], P_L);
    const uint16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)qr * p.q_sl + hh * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const x8*)(qp + kk * 16);
  }
  // the row's tile records (GS): read through the scalar cache; wp walks this wave's word of the records
  using w_ptr = const __attribute__((address_space(4))) uint32_t*;
  using rec_ptr = const __attribute__((address_space(4))) u32x4*;
  rec_ptr recs = nullptr;
  int T;
  if constexpr (GS) {
    recs = (rec_ptr)(uintptr_t)(p.sched_rec + (int64_t)logical * p.rec_stride);
    T = active ? __builtin_amdgcn_readfirstlane(p.sched_tiles[logical]) : 0;
  } else {
    // both groups run the builder's barriers together
    T = psa_tiles::build_row_schedule<NT>(p.map, p.map_elem, ((int64_t)bh * p.Mq + I) * p.Nk, p.Nk, jmax, P_bn_log2, P_L,
                                          P_causal != 0, (int64_t)I * p.bm, ids, tdesc, s_cnt[grp], s_ioff[grp], s_toff[grp],
                                          s_wcnt[grp], tid);
  }
  if (tid == 0) s_T[grp] = T;

  const char* kb0 = (const char*)(p.k + b * p.k_sb + hk * p.k_sh);
  const char* vb0 = (const char*)(p.v + b * p.v_sb + hk * p.v_sh);
  const int64_t BHkv = (int64_t)p.B * p.Hkv, bhk = (int64_t)b * p.Hkv + hk;

  const uint32_t f_chunk = psa_tiles::lt_fetch_chunk<D>(lane);
  uint32_t k_off[2], v_off[2];
  psa_tiles::lt_row_operand<D>(l32, hh, k_off);
  psa_tiles::lt_tr_operand<D>(lane, v_off);
#pragma unroll
  for (int i = 0; i < 2; ++i) {  // operand addresses: lane base (incl. the group's region) + immediate
    k_off[i] += grp_base;
    v_off[i] += grp_base;
  }

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
  float m_run = -INFINITY;
  float l_run = 0.f;

  // ---- softmax of tile t, in pieces --------------------------------------------------------------------
  // mask_tile: partly filled tiles and the causal diagonal (rare).  head_piece(i): piece i of the row maximum /
  // reference update, small enough to ride along with one MFMA of PV(t-1).  prob16: the exponentials.
  uint32_t d_cur = 0;  // descriptor word 0 of the tile whose logits are in s: level | masked << 2 | ...
  uint32_t w_cur = 0;  // GS: this wave's word of its record
  auto mask_tile_rec = [&](int t, f32x16 (&s_cur)[2]) __attribute__((always_inline)) {
    const int lv = psa_sched::rec_level(w_cur);
    const int nvalid = psa_sched::rec_nvalid(w_cur);
    const int qlim = (q_idx + 1) >> lv;
    u32x4 r4 = {0u, 0u, 0u, 0u};
    if (P_causal) r4 = recs[t];  // the source rows of all four quarters (rare path: fetched on demand)
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int r0 = c * 32 + g * 8 + hh * 4;
        int keep = nvalid - r0;
        if (P_causal) {
          // slots r0 .. r0+3 lie in quarter 2c + g/2 of the tile, whose source rows are consecutive
          const int src0 = psa_sched::rec_src(r4[c * 2 + (g >> 1)]) + (g & 1) * 8 + hh * 4;
          keep = keep < qlim - src0 ? keep : qlim - src0;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) s_cur[c][g * 4 + e] = e < keep ? s_cur[c][g * 4 + e] : -INFINITY;
      }
  };
  auto mask_tile = [&](int t, f32x16 (&s_cur)[2]) __attribute__((always_inline)) {
    const uint32_t d = d_cur;
    const int lv = d & 3;
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
  };
  constexpr int HEAD_PIECES = 12;
  float hx0, hx1, h_cand, h_new;  // state between the pieces
  float alpha = 1.0f, nb = 0.f;
  auto head_piece = [&](int i, const f32x16 (&s_cur)[2], bool real) __attribute__((always_inline)) {
    if (i == 0) {
      hx0 = s_cur[0][0];
      hx1 = s_cur[1][0];
    }
    if (i < 7) {
      hx0 = max3f(hx0, s_cur[0][1 + 2 * i], s_cur[0][2 + 2 * i]);
      hx1 = max3f(hx1, s_cur[1][1 + 2 * i], s_cur[1][2 + 2 * i]);
    } else if (i == 7) {
      hx0 = max3f(hx0, s_cur[0][15], fmaxf(hx1, s_cur[1][15]));
    } else if (i == 8) {
      hx0 = half_wave_max(hx0);
    } else if (i == 9) {
      h_cand = __builtin_fmaf(hx0, P_scale_log2, (float)(d_cur & 3));
    } else if (i == 10) {
      // raise the reference max only when it lags by more than the threshold (or is still -inf)
      h_new = (h_cand - m_run > LAZY_THRESHOLD) ? h_cand : m_run;
      h_new = (m_run == -INFINITY) ? h_cand : h_new;
    } else if (i == 11) {
      const float m_use = h_new == -INFINITY ? 0.f : h_new;  // rows that still see no key
      alpha = real ? fast_exp2(m_run - m_use) : 1.0f;
      nb = (float)(d_cur & 3) - m_use;
      m_run = real ? h_new : m_run;
    }
  };
  // probabilities of 4 logits: exp2, round to bf16 for P^T; the row sum adds the unrounded values with plain adds
  // (a dot-product instruction would queue behind the other group's MFMAs)
  // (x0: scale * sc[i] + nb_, where the caller already has it - it rides along with a copy in the scheduled walk)
  auto prob4x = [&](const f32x16& sc, int i, float nb_, uint32_t* pk2, float& lsum, float x0) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 4; e += 2) {
      const float p0 = fast_exp2(e == 0 ? x0 : __builtin_fmaf(sc[i + e], P_scale_log2, nb_));
      const float p1 = fast_exp2(__builtin_fmaf(sc[i + e + 1], P_scale_log2, nb_));
      pk2[e >> 1] = ET::pack2(p0, p1);
      lsum += p0 + p1;
    }
  };
  auto prob4 = [&](const f32x16& sc, int i, float nb_, uint32_t* pk2, float& lsum) __attribute__((always_inline)) {
    prob4x(sc, i, nb_, pk2, lsum, __builtin_fmaf(sc[i], P_scale_log2, nb_));
  };
  // Copy source of a tile for this lane: base pointers and row strides of its level (uniform), and the RPL
  // consecutive source rows of this wave's 16-row group (clamped where a partly filled tile runs past the end).
  struct CopySrc {
    const char *kbase, *vbase;
    uint32_t kstr, vstr;
    int row[G::RPL];
  };
  // base pointers of the pooled levels of this (batch, kv head); plain scalars, selected by compare chains
  auto pool_base = [&](const uint16_t* pool, int lv) __attribute__((always_inline)) {
    return (const char*)pool + (BHkv * (P_npad - (P_npad >> (lv - 1))) + bhk * (P_npad >> lv)) * (D * 2);
  };
  const char* const kb1 = pool_base(P_kp, 1);
  const char* const kb2 = pool_base(P_kp, 2);
  const char* const kb3 = pool_base(P_kp, 3);
  const char* const vb1 = pool_base(P_vp, 1);
  const char* const vb2 = pool_base(P_vp, 2);
  const char* const vb3 = pool_base(P_vp, 3);
  auto by_level = [&](int lv, const char* a0, const char* a1, const char* a2, const char* a3) __attribute__((always_inline)) {
    const char* r = a0;
    r = lv == 1 ? a1 : r;
    r = lv == 2 ? a2 : r;
    r = lv == 3 ? a3 : r;
    return r;
  };
  // One copy instruction: block n of this wave's 16-row group, into the tile buffer at byte lds_byte of the group
  // One copy instruction: block N of this wave's 16-row group, into the tile buffer at byte LDS_BYTE of the group
  // (the group's and the wave's part of the address as one integer: no null test per address derived from it)
  const uint32_t wave_lds = psa_tiles::lds_addr_of(smem) + (uint32_t)(wave * G::RPL * F_ISTR);
  auto issue_one = [&](const char* base, uint32_t str, int row, auto lds_byte, auto n) __attribute__((always_inline)) {
    psa_tiles::lds_copy16_row<decltype(lds_byte)::value + decltype(n)::value * F_ISTR>(base, (uint32_t)row, str, f_chunk, wave_lds);
  };
  // The matrix work of one phase: S^T = K Q^T (tile in K buffer KB) and then O^T += V^T P^T (tile in V buffer
  // 1 - KB, probabilities pk2).  Only one wave per SIMD is in its matrix phase, so nothing else hides the LDS
  // latency: all 2*KK K operands are requested up front, and the V^T operands follow into the registers that
  // the QK steps release (two PV steps per k-step), so that the MFMAs stream.  hook(st) runs after PV step st.
  static_assert(4 * DB == 2 * KK, "two PV steps per QK k-step");
  auto matrix_work = [&](auto kb_c, f32x16 (&s2)[2], const uint32_t (&pk2)[2][8], float a_prev, auto mid, auto hook) __attribute__((always_inline)) {
    constexpr int KB = decltype(kb_c)::value;
    constexpr int STEPS = 4 * DB;
    PSA_LDS(unsigned char) Ks = (PSA_LDS(unsigned char))(smem_all) + KB * F_TILE;
    PSA_LDS(unsigned char) Vs = (PSA_LDS(unsigned char))(smem_all) + (2 + (KB ^ 1)) * F_TILE;
    constexpr int K_UP = KK - 2;          // k-steps whose K operands are requested before the first MFMA
    constexpr int V_LATE = 2 * (KK - K_UP);  // PV steps whose operands are requested during PV
    x8 ka[2 * KK];
    auto kread = [&](int kk) __attribute__((always_inline)) {
      ka[2 * kk] = *(PSA_LDS(const x8))(Ks + k_off[kk & 1] + (kk >> 1) * 64);
      ka[2 * kk + 1] = *(PSA_LDS(const x8))(Ks + k_off[kk & 1] + (kk >> 1) * 64 + G::HALF);
    };
#pragma unroll
    for (int kk = 0; kk < K_UP; ++kk) kread(kk);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) s2[c][i] = 0.f;
    u32x2 vlo[STEPS], vhi[STEPS];
    auto vread = [&](int st) __attribute__((always_inline)) {
      const int cg = st / DB, db = st % DB;
      const int off = (cg >> 1) * G::HALF + db * 64 + (cg & 1) * G::GROUP;
      vlo[st] = ET::read_tr(Vs + v_off[0] + off);
      vhi[st] = ET::read_tr(Vs + v_off[1] + off);
    };
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      s2[0] = ET::mfma(ka[2 * kk], qf[kk], s2[0]);
      s2[1] = ET::mfma(ka[2 * kk + 1], qf[kk], s2[1]);
      if (kk + K_UP < KK) {
        kread(kk + K_UP);
      } else {
        vread(2 * (kk - (KK - K_UP)));
        vread(2 * (kk - (KK - K_UP)) + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    mid();
    if (__any(a_prev != 1.0f)) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][i] *= a_prev;
    }
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      const int cg = st / DB, db = st % DB;
      const uint32_t* pk8 = pk2[cg >> 1];
      const int g = cg & 1;
      u32x4 bw = {pk8[g * 4 + 0], pk8[g * 4 + 1], pk8[g * 4 + 2], pk8[g * 4 + 3]};
      u32x4 aw = {vlo[st][0], vlo[st][1], vhi[st][0], vhi[st][1]};
      acc[db] = ET::mfma(__builtin_bit_cast(x8, aw), __builtin_bit_cast(x8, bw), acc[db]);
      if (st < V_LATE) vread(STEPS - V_LATE + st);
      hook(st);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  const std::integral_constant<int, 0> B0;
  const std::integral_constant<int, 1> B1;

  CopySrc ts, ts2;
  f32x16 s[2];
  uint32_t pk[2][8];
  auto to_copy_src = [&](const TileSrc& a, CopySrc& c) __attribute__((always_inline)) {
    c.kbase = a.kbase; c.vbase = a.vbase; c.kstr = a.kstr; c.vstr = a.vstr;
#pragma unroll
    for (int n = 0; n < G::RPL; ++n) c.row[n] = a.src0[0] + n < a.lim ? a.src0[0] + n : a.lim;
  };
  // ---- GS: copies addressed from scalar registers ------------------------------------------------------------
  // A lane fetches rows 4 * (lane / 16) + n of its wave's quarter, n = 0..3; all rows are D * 2 bytes apart.
  const int lane_row = psa_tiles::lt_fetch_row<D>(lane);
  const uint32_t voff_s = (uint32_t)lane_row * (uint32_t)(D * 2) + f_chunk;
  struct Stream {  // where one tensor's tiles currently come from: a level's rows (the level changes 3 times per row)
    const char* base;
    uint32_t code;
  };
  Stream st_k = {kb0, 0u}, st_v = {vb0, 0u};
  // first source row of this wave's quarter of the tile with word w; rag: the tile is ragged (rows are clamped per lane)
  auto quarter_src = [&](Stream& st, bool is_k, uint32_t w, bool& rag) __attribute__((always_inline)) {
    const uint32_t code = psa_sched::rec_code(w);
    if (code != st.code) {
      st.code = code & 3u;  // (a ragged tile comes back here for every tile)
      st.base = is_k ? by_level((int)(code & 3u), kb0, kb1, kb2, kb3) : by_level((int)(code & 3u), vb0, vb1, vb2, vb3);
      rag = rag || code == psa_sched::REC_CODE_RAGGED;
    }
    return st.base + (uint64_t)((w & psa_sched::REC_SRC_MASK) * (uint32_t)(D * 2));
  };
  // copy instruction N of the wave's quarter (tile rows 4i + N of the quarter) into the tile buffer at LDS_BYTE
  auto issue_s = [&](const char* src, auto lds_byte, auto n) __attribute__((always_inline)) {
    constexpr int N = decltype(n)::value;
    psa_tiles::lds_copy16_imm<decltype(lds_byte)::value + N * F_ISTR, N * D * 2>(src, voff_s, wave_lds);
  };
  // the same with the first multiply-add of the exponentials that follow in the wait state between the write of M0 and
  // the copy (returns scale * x + y)
  auto issue_s_fma = [&](const char* src, auto lds_byte, auto n, float x, float y) __attribute__((always_inline)) {
    constexpr int N = decltype(n)::value;
    return psa_tiles::lds_copy16_imm_fma<decltype(lds_byte)::value + N * F_ISTR, N * D * 2>(src, voff_s, wave_lds, P_scale_log2, x, y);
  };
  // the same with a row index per lane, clamped to the last token (ragged tiles: the walk takes this form only in
  // phases that copy such a tile, so that the usual phase has no branch between its copies)
  auto issue_clamped = [&](const char* base0, uint32_t w, auto lds_byte, auto n) __attribute__((always_inline)) {
    constexpr int N = decltype(n)::value, OFF = decltype(lds_byte)::value + N * F_ISTR;
    const int lim = psa_sched::rec_code(w) == psa_sched::REC_CODE_RAGGED ? P_L - 1 : 0x7fffffff;
    const int row = psa_sched::rec_src(w) + lane_row + N;
    psa_tiles::lds_copy16_row<OFF>(base0, (uint32_t)(row < lim ? row : lim), (uint32_t)(D * 2), f_chunk, wave_lds);
  };
  auto issue_tile = [&](Stream& st, bool is_k, uint32_t w, auto lds_byte) __attribute__((always_inline)) {
    bool rag = false;
    const char* src = quarter_src(st, is_k, w, rag);
    if (rag) static_for<G::RPL>([&](auto n) __attribute__((always_inline)) { issue_clamped(st.base, w, lds_byte, n); });
    else static_for<G::RPL>([&](auto n) __attribute__((always_inline)) { issue_s(src, lds_byte, n); });
  };
  w_ptr wp = nullptr;                    // this wave's word of the record fetched next
  uint32_t w_v = 0, w_k = 0, w_next = 0;  // words of tiles t+1 (its V goes out next), t+2 (its K), of the next M phase
  const int T_last = T > 0 ? T - 1 : 0;
  // first copies: K(0), V(0), K(1); ts is left describing tile min(1, T-1) for the copy of V(1)
  if constexpr (GS) {
    if (T > 0) {
      wp = (w_ptr)(uintptr_t)((const uint32_t*)(p.sched_rec + (int64_t)logical * p.rec_stride) + wave);
      w_next = wp[0];  // (records T .. T+2 repeat record T-1)
      w_v = wp[4];
      w_k = wp[8];
      wp += 12;
      issue_tile(st_k, true, w_next, IC<0>{});
      issue_tile(st_v, false, w_next, IC<2 * F_TILE>{});
      if (T > 1) issue_tile(st_k, true, w_v, IC<F_TILE>{});
    }
  } else if (T > 0) {
    TileSrc a;
    tile_src(0, a);
    issue_rows(a.kbase, a.kstr, a.lim, a.src0, 0);
    issue_rows(a.vbase, a.vstr, a.lim, a.src0, 2 * F_TILE);
    if (T > 1) {
      tile_src(1, a);
      issue_rows(a.kbase, a.kstr, a.lim, a.src0, F_TILE);
    }
    to_copy_src(a, ts);
  } else {
    ts.kbase = kb0; ts.vbase = vb0; ts.kstr = 0; ts.vstr = 0;
#pragma unroll
    for (int n = 0; n < G::RPL; ++n) ts.row[n] = 0;
  }
  ts2 = ts;
  // M_0 multiplies V buffer 1 by zero probabilities: give it finite contents
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int i = 0; i < 8; ++i) pk[c][i] = 0u;
  for (int u = tid * 16; u < F_TILE; u += NT * 16) *(u32x4*)(smem + 3 * F_TILE + u) = u32x4{0u, 0u, 0u, 0u};
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();
  const int T_other = s_T[grp ^ 1];
  const int C = (T > T_other ? T : T_other) + 1;  // (M, V) phase pairs both groups step through

  // M_t: the matrix phase.  K(t) lives in K buffer t&1, V(t-1) in V buffer (t-1)&1.  QK(t) comes first so that
  // the row maximum of tile t can ride along with the MFMAs of PV(t-1), and so does the look-up of the source
  // rows of tile t+2 (two dependent LDS reads, spread over the phase).  At t == T only PV(T-1) counts: QK then
  // runs on stale data and its maximum is dropped; at t == 0 PV multiplies the zeroed V buffer by zeros.
  // Both phases are free of branches (tiles past the end are clamped to the last one and copied again into a
  // buffer nobody reads), so that the instruction order below is the order that runs.
  constexpr int HOOK0 = 2;  // first PV step that carries a piece of the maximum (QK's last results need that long)
  uint32_t d_next = 0u;  // descriptor of the tile of the next M phase
  if constexpr (!GS) d_next = T > 0 ? __builtin_amdgcn_readfirstlane(tdesc[0][0]) : 0u;
  auto mfma_phase = [&](int t, auto cur_c) __attribute__((always_inline)) {
    if (T > 0 && t <= T) {
      const bool real = t < T;
      if constexpr (GS) {
        w_cur = w_next;
        d_cur = real ? (((w_cur >> psa_sched::REC_CODE_SHIFT) & 3u) | ((w_cur >> (psa_sched::REC_MASKED_BIT - 2)) & 4u)) : 0u;  // level | masked << 2
      } else {
        d_cur = real ? d_next : 0u;
      }
      matrix_work(
          cur_c, s, pk, alpha,
          [&]() __attribute__((always_inline)) {
            if (d_cur & 4) {
              if constexpr (GS) mask_tile_rec(t, s);
              else mask_tile(t, s);
            }
          },
          [&](int st) __attribute__((always_inline)) {
            if (st >= HOOK0 && st - HOOK0 < HEAD_PIECES) head_piece(st - HOOK0, s, real);
          });
    }
  };
  // V_t: the vector phase.  K buffer t&1 and V buffer (t-1)&1 were last read in M_t: V(t+1) (described by ts) and
  // K(t+2) (ts2, looked up in the first half of this phase) go there, one copy instruction per 4 exponentials so
  // that the copy unit never makes the wave wait.
  auto valu_phase_map = [&](int t, auto cur_c) __attribute__((always_inline)) {
    constexpr int CUR = decltype(cur_c)::value;
    if (t < T) {
      const int tn = t + 2 < T ? t + 2 : T_last;
      const u32x2 dd2 = tdesc[tn];
      const uint32_t dn = tdesc[t + 1 < T ? t + 1 : T_last][0];
      __builtin_amdgcn_s_waitcnt(0x0f70);  // K(t+1), V(t) of this wave have landed (visible to the group after the next barrier)
      float lsum = 0.f;
      int n_lv = 0, n_sbs = 0, n_g = 0, n_lim = 0;
      uint16_t n_id = 0;
      static_for<8>([&](auto cc) __attribute__((always_inline)) {
        constexpr int c = decltype(cc)::value;
        if constexpr (c < 4) issue_one(ts.vbase, ts.vstr, ts.row[c], IC<(2 + (CUR ^ 1)) * F_TILE>{}, IC<c>{});
        else issue_one(ts2.kbase, ts2.kstr, ts2.row[c - 4], IC<CUR * F_TILE>{}, IC<c - 4>{});
        prob4(s[c >> 2], (c & 3) * 4, nb, pk[c >> 2] + (c & 3) * 2, lsum);
        if (c == 0) {
          const uint32_t d0 = __builtin_amdgcn_readfirstlane(dd2[0]), d1 = __builtin_amdgcn_readfirstlane(dd2[1]);
          d_next = __builtin_amdgcn_readfirstlane(dn);
          n_lv = d0 & 3;
          const int nvalid = (d0 >> 3) & 127, lt = d0 >> 10, cnt = d1 >> 16;
          n_sbs = P_bn_log2 - n_lv;
          n_lim = (nvalid < TK && n_lv == 0) ? P_L - 1 : 0x7fffffff;
          n_g = (lt << 6) + wave * 16 + psa_tiles::lt_fetch_row<D>(lane);
          int bi = n_g >> n_sbs;
          bi = bi < cnt - 1 ? bi : cnt - 1;  // (only matters in a partly filled tile)
          n_id = ids[(d1 & 0xffff) + bi];
        }
        if (c == 2) {
          ts2.kbase = by_level(n_lv, kb0, kb1, kb2, kb3);
          ts2.vbase = by_level(n_lv, vb0, vb1, vb2, vb3);
          ts2.kstr = n_lv == 0 ? P_k_strb : (uint32_t)(D * 2);
          ts2.vstr = n_lv == 0 ? P_v_strb : (uint32_t)(D * 2);
        }
        if (c == 3) {
          const int src0 = ((int)n_id << n_sbs) + (n_g & ((1 << n_sbs) - 1));
#pragma unroll
          for (int n = 0; n < G::RPL; ++n) ts2.row[n] = src0 + n < n_lim ? src0 + n : n_lim;
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      ts = ts2;
      l_run = l_run * alpha + lsum;
    }
  };
  // The same with a prebuilt schedule: V(t+1) is described by w_v, K(t+2) by w_k; the word of tile t+3 is fetched here
  // (one scalar load) and is complete before the phase ends.
  auto valu_phase_rec = [&](int t, auto cur_c) __attribute__((always_inline)) {
    constexpr int CUR = decltype(cur_c)::value;
    if (t < T) {
      const uint32_t w3 = *wp;
      wp += 4;
      bool rag = false;
      const char* src_v = quarter_src(st_v, false, w_v, rag);
      const char* src_k = quarter_src(st_k, true, w_k, rag);
      __builtin_amdgcn_s_waitcnt(0x0f70);  // K(t+1), V(t) of this wave have landed (visible to the group after the next barrier)
      float lsum = 0.f;
      if (!rag) {
        static_for<8>([&](auto cc) __attribute__((always_inline)) {
          constexpr int c = decltype(cc)::value;
          float x0;
          if constexpr (c < 4) x0 = issue_s_fma(src_v, IC<(2 + (CUR ^ 1)) * F_TILE>{}, IC<c>{}, s[c >> 2][(c & 3) * 4], nb);
          else x0 = issue_s_fma(src_k, IC<CUR * F_TILE>{}, IC<c - 4>{}, s[c >> 2][(c & 3) * 4], nb);
          prob4x(s[c >> 2], (c & 3) * 4, nb, pk[c >> 2] + (c & 3) * 2, lsum, x0);
          __builtin_amdgcn_sched_barrier(0);
        });
      } else {
        static_for<8>([&](auto cc) __attribute__((always_inline)) {
          constexpr int c = decltype(cc)::value;
          if constexpr (c < 4) issue_clamped(st_v.base, w_v, IC<(2 + (CUR ^ 1)) * F_TILE>{}, IC<c>{});
          else issue_clamped(st_k.base, w_k, IC<CUR * F_TILE>{}, IC<c - 4>{});
          prob4(s[c >> 2], (c & 3) * 4, nb, pk[c >> 2] + (c & 3) * 2, lsum);
          __builtin_amdgcn_sched_barrier(0);
        });
      }
      w_next = w_v;
      w_v = w_k;
      w_k = w3;
      // the scalar load is awaited here, inside the phase: none stays in flight across the barrier into a matrix phase,
      // whose staged waits on its LDS reads count on the same counter
      asm volatile("" ::"s"(w_k));
      l_run = l_run * alpha + lsum;
    }
  };
  auto valu_phase = [&](int t, auto cur_c) __attribute__((always_inline)) {
    if constexpr (GS) valu_phase_rec(t, cur_c);
    else valu_phase_map(t, cur_c);
  };
  if (grp == 1) PP_BARRIER();
  for (int t = 0; t < C; t += 2) {
    mfma_phase(t, B0);
    PP_BARRIER();
    valu_phase(t, B0);
    PP_BARRIER();
    mfma_phase(t + 1, B1);
    PP_BARRIER();
    valu_phase(t + 1, B1);
    PP_BARRIER();
  }
  if (grp == 0) PP_BARRIER();

  // ---- epilogue ---------------------------------------------------------------------------------------
  float l_tot = half_wave_sum(l_run);
  const float l_safe = fmaxf(l_tot, 1e-8f);
  const float inv = 1.0f / l_safe;
  if (active && p.lse != nullptr && hh == 0 && q_idx < P_L) {
    const int lrow = p.q_index != nullptr ? p.q_index[q_idx] : q_idx;  // (a row outside 0 .. L-1 is not stored)
    if ((unsigned)lrow < (unsigned)P_L) p.lse[((int64_t)b * p.Hq + h) * P_L + lrow] = (m_run + fast_log2(l_safe)) * 0.6931471805599453f;
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // the last (repeated) tile copies land in the buffers that now stage O
  __syncthreads();
  unsigned char* Os = smem;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w[0] = ET::pack2(acc[db][g * 4 + 0] * inv, acc[db][g * 4 + 1] * inv);
      w[1] = ET::pack2(acc[db][g * 4 + 2] * inv, acc[db][g * 4 + 3] * inv);
      *(u32x2*)(Os + (wave * 32 + l32) * OST + (db * 32 + g * 8 + hh * 4) * 2) = w;
    }
  __syncthreads();
  if (active) {
    uint16_t* ob = p.o + b * p.o_sb + h * p.o_sh;
    for (int u = tid; u < BM * CH; u += NT) {
      const int r = u / CH, ch = u % CH;
      const int row = I * BM + r;
      if (row < P_L) {
        const int orow = p.q_index != nullptr ? p.q_index[row] : row;
        if ((unsigned)orow < (unsigned)P_L) *(u32x4*)(ob + (int64_t)orow * p.o_sl + ch * 8) = *(const u32x4*)(Os + r * OST + ch * 16);
      }
    }
  }
}


template <int D, int NW, bool GS = false>
int launch_fwd(const FwdParams& p, int Nk, hipStream_t stream) {
  // with a prebuilt schedule the workgroup keeps nothing but its tile buffers in LDS
  size_t shmem = (size_t)4 * psa_tiles::LtGeom<D>::TILE + (GS ? 0 : (size_t)p.max_tiles * 8 + (size_t)Nk * 2);
  if (shmem > 160 * 1024) return PSA_ERR_UNSUPPORTED;
  int rc = PSA_OK;
  psa_dispatch16(p.dtype, [&](auto et) {
    using ET = decltype(et);
    if (hipFuncSetAttribute((const void*)psa_fwd_lds_kernel<D, NW, GS, ET>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess) {
      rc = PSA_ERR_LAUNCH;
      return;
    }
    hipLaunchKernelGGL((psa_fwd_lds_kernel<D, NW, GS, ET>), dim3((unsigned)(p.wg_chunk * p.wg_groups)), dim3(NW * 64), shmem, stream, p);
  });
  return rc;
}

template <int D, int NW, bool GS>
int launch_fwd_pp(FwdParams& p, int Nk, hipStream_t stream) {
  // with a prebuilt schedule the groups keep nothing but their tile buffers in LDS
  const size_t sched = GS ? 0 : ((((size_t)p.max_tiles * 8 + (size_t)Nk * 2) + 15) & ~(size_t)15);
  p.grp_bytes = (int)(4 * psa_tiles::LtGeom<D>::TILE + sched);
  const size_t shmem = 2 * (size_t)p.grp_bytes;
  int rc = PSA_OK;
  psa_dispatch16(p.dtype, [&](auto et) {
    using ET = decltype(et);
    if (hipFuncSetAttribute((const void*)psa_fwd_pp_kernel<D, NW, GS, ET>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess) {
      rc = PSA_ERR_LAUNCH;
      return;
    }
    hipLaunchKernelGGL((psa_fwd_pp_kernel<D, NW, GS, ET>), dim3((unsigned)((p.wg_chunk / 2) * p.wg_groups)), dim3(2 * NW * 64), shmem, stream, p);
  });
  return rc;
}
// LDS bytes the two-group kernel needs (tile buffers and schedule of both groups + its static tables)
template <int D>
size_t pp_lds_bytes(int max_tiles, int Nk) {
  const size_t sched = (((size_t)max_tiles * 8 + (size_t)Nk * 2) + 15) & ~(size_t)15;
  return 2 * (4 * (size_t)psa_tiles::LtGeom<D>::TILE + sched) + 512;
}

}  // namespace

extern "C" int64_t psa_fwd_workspace_bytes(int B, int Hq, int L, int block_m) {
  if (B <= 0 || Hq <= 0 || L <= 0 || block_m <= 0) return 0;
  const int64_t total = (int64_t)B * Hq * ((L + block_m - 1) / block_m);
  return 2 * (total + 16 * psa_order::MAX_PHASES) * (int64_t)sizeof(int32_t);  // any grouping of the rows fits
}

static int fwd_impl(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool,
                    const void* map, int map_elem_bytes, psa_tensor4 out, float* lse, int B, int Hq, int Hkv, int L,
                    int D, int block_m, int block_n, float sm_scale, int causal, void* workspace, psa_stream_t stream,
                    const int32_t* q_index = nullptr, const void* schedule = nullptr) {
  PSA_REQUIRE(q.ptr && k.ptr && v.ptr && out.ptr, PSA_ERR_ARG, "psa_fwd: null pointer");
  PSA_REQUIRE(map == nullptr || (k_pool && v_pool), PSA_ERR_ARG, "psa_fwd: pooled K/V required with a level map");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_fwd: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && L > 0, PSA_ERR_ARG, "psa_fwd: B, H, L must be positive");
  PSA_REQUIRE(q.dtype == k.dtype && q.dtype == v.dtype && q.dtype == out.dtype, PSA_ERR_ARG, "psa_fwd: q, k, v, out must share one element type");
  if (q.dtype == PSA_DTYPE_F32)
    return psa_fwd_f32(q, k, v, k_pool, v_pool, map, map_elem_bytes, out, lse, B, Hq, Hkv, L, D, block_m, block_n, sm_scale, causal, stream, q_index);
  PSA_REQUIRE(q.dtype == PSA_DTYPE_BF16 || q.dtype == PSA_DTYPE_F16, PSA_ERR_ARG, "psa_fwd: unknown element type %d", q.dtype);
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
  p.q = (const uint16_t*)q.ptr; p.k = (const uint16_t*)k.ptr; p.v = (const uint16_t*)v.ptr; p.o = (uint16_t*)out.ptr;
  p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sl = q.stride_l;
  p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sl = k.stride_l;
  p.v_sb = v.stride_b; p.v_sh = v.stride_h; p.v_sl = v.stride_l;
  p.o_sb = out.stride_b; p.o_sh = out.stride_h; p.o_sl = out.stride_l;
  p.kp = (const uint16_t*)k_pool; p.vp = (const uint16_t*)v_pool;
  p.map = map; p.map_elem = map_elem_bytes; p.lse = lse; p.dtype = q.dtype;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.L = L; p.Mq = Mq; p.Nk = Nk;
  p.bn_log2 = psa_ilog2(block_n); p.bm = block_m;
  p.npad = (int64_t)Nk * block_n;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  p.causal = causal ? 1 : 0;
  p.total_wg = (int)total;
  // Groups of rows run one after the other on each XCD.  With several phases (8 groups each) the K/V of only a
  // few heads is in use at a time, so that the part of it that misses L2 can stay in the last-level cache.
  {
    const double kv_bytes = 2.0 * B * Hkv * ((double)Nk * block_n) * D * 2.0 * (map != nullptr ? 1.875 : 1.0);
    psa_order::deal(total, kv_bytes, B * Hkv, p.wg_chunk, p.wg_groups);
  }
  // worst case: every kv-block at level 1, plus one partly filled tile per pooled level
  p.max_tiles = (block_n >= 64 ? Nk * (block_n / 64) : (Nk * block_n + 63) / 64) + 4;
  p.grp_bytes = 0;
  // two rows per workgroup when the head dim / block size have that kernel and both schedules fit into LDS
  // (that kernel forms its copy offsets with 24-bit multiplies: row index and row stride in bytes must fit)
  const bool two_group = D == 128 && block_m == 128 && total > 1 && pp_lds_bytes<128>(p.max_tiles, Nk) <= 160 * 1024 && !PSA_FWD_ONE_GROUP &&
                         (int64_t)Nk * block_n < (1 << 24) && k.stride_l * 2 < (1 << 24) && v.stride_l * 2 < (1 << 24);
  if (two_group) p.wg_chunk = (p.wg_chunk + 1) & ~1;  // pairs never straddle two groups of rows
  p.order = nullptr;
  p.q_index = q_index;
  p.sched_rec = nullptr; p.sched_tiles = nullptr; p.rec_stride = 0;
  if (schedule != nullptr) {
    // prebuilt schedule (psa_build_schedule with the same shape arguments): issue order, tiles per row, tile records
    psa_sched::Geometry g;
    PSA_REQUIRE(map != nullptr && psa_schedule_geometry(B, Hq, Hkv, L, D, block_m, block_n, g), PSA_ERR_UNSUPPORTED,
                "psa_fwd: no scheduled kernel for this shape");
    const char* base = (const char*)schedule;
    p.wg_chunk = g.wg_chunk; p.wg_groups = g.wg_groups;
    p.order = (const int32_t*)(base + g.lay.order_off);
    // the record walk assumes K / V rows D elements apart (the usual layout); other layouts walk the map in the
    // schedule's issue order
    int rc;
    if (k.stride_l == D && v.stride_l == D) {
      p.sched_rec = (const u32x4*)(base + g.lay.rec_off);
      p.sched_tiles = (const int32_t*)(base + g.lay.tiles_off);
      p.rec_stride = g.lay.rec_stride;
      rc = D == 128 ? launch_fwd_pp<128, 4, true>(p, Nk, (hipStream_t)stream) : launch_fwd<64, 4, true>(p, Nk, (hipStream_t)stream);
    } else if (two_group) {
      rc = launch_fwd_pp<128, 4, false>(p, Nk, (hipStream_t)stream);
    } else {
      rc = D == 128 ? launch_fwd<128, 4>(p, Nk, (hipStream_t)stream) : launch_fwd<64, 4>(p, Nk, (hipStream_t)stream);
    }
    PSA_REQUIRE(rc == PSA_OK, rc, "psa_fwd: sequence too long for the on-chip schedule (LDS)");
    return psa_check_launch("psa_fwd");
  }
  if (workspace != nullptr && map != nullptr && total > 8 * 32) {
    PSA_REQUIRE((uintptr_t)workspace % 4 == 0, PSA_ERR_ARG, "psa_fwd: workspace must be 4-byte aligned");
    int32_t* order = (int32_t*)workspace;
    int32_t* cost = order + (int64_t)p.wg_chunk * p.wg_groups;
    hipLaunchKernelGGL(psa_order::psa_row_cost_kernel, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, (hipStream_t)stream, map, map_elem_bytes,
                       (int)total, Mq, Nk, p.bn_log2, block_m, p.causal, cost);
    if (int e = psa_check_launch("psa_fwd (row cost)")) return e;
    hipLaunchKernelGGL(psa_order::psa_chunk_sort_kernel, dim3(p.wg_groups), dim3(256), 0, (hipStream_t)stream, cost, (int)total, p.wg_chunk, order);
    if (int e = psa_check_launch("psa_fwd (row order)")) return e;
    p.order = order;
  }
  int rc;
  if (two_group) rc = launch_fwd_pp<128, 4, false>(p, Nk, (hipStream_t)stream);
  else if (D == 128 && block_m == 128) rc = launch_fwd<128, 4>(p, Nk, (hipStream_t)stream);
  else if (D == 128) rc = launch_fwd<128, 2>(p, Nk, (hipStream_t)stream);
  else if (block_m == 128) rc = launch_fwd<64, 4>(p, Nk, (hipStream_t)stream);
  else rc = launch_fwd<64, 2>(p, Nk, (hipStream_t)stream);
  PSA_REQUIRE(rc == PSA_OK, rc, "psa_fwd: sequence too long for the on-chip schedule (LDS)");
  return psa_check_launch("psa_fwd");
}

extern "C" int psa_fwd(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool,
                       const void* map, int map_elem_bytes, psa_tensor4 out, float* lse, int B, int Hq, int Hkv, int L,
                       int D, int block_m, int block_n, float sm_scale, int causal, void* workspace, psa_stream_t stream) {
  return fwd_impl(q, k, v, k_pool, v_pool, map, map_elem_bytes, out, lse, B, Hq, Hkv, L, D, block_m, block_n, sm_scale, causal,
                  workspace, stream);
}

extern "C" int psa_fwd_indexed(psa_tensor4 q, const int32_t* q_index, psa_tensor4 k, psa_tensor4 v, const void* k_pool,
                               const void* v_pool, const void* map, int map_elem_bytes, psa_tensor4 out, float* lse, int B, int Hq,
                               int Hkv, int L, int D, int block_m, int block_n, float sm_scale, int causal, void* workspace,
                               psa_stream_t stream) {
  PSA_REQUIRE(q_index != nullptr, PSA_ERR_ARG, "psa_fwd_indexed: null index");
  return fwd_impl(q, k, v, k_pool, v_pool, map, map_elem_bytes, out, lse, B, Hq, Hkv, L, D, block_m, block_n, sm_scale, causal,
                  workspace, stream, q_index);
}

extern "C" int psa_fwd_scheduled(psa_tensor4 q, const int32_t* q_index, psa_tensor4 k, psa_tensor4 v, const void* k_pool,
                                 const void* v_pool, const void* map, int map_elem_bytes, const void* schedule, psa_tensor4 out,
                                 float* lse, int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, float sm_scale,
                                 int causal, psa_stream_t stream) {
  PSA_REQUIRE(schedule != nullptr && map != nullptr, PSA_ERR_ARG, "psa_fwd_scheduled: null schedule or map");
  PSA_REQUIRE((uintptr_t)schedule % 16 == 0, PSA_ERR_ARG, "psa_fwd_scheduled: schedule must be 16-byte aligned");
  return fwd_impl(q, k, v, k_pool, v_pool, map, map_elem_bytes, out, lse, B, Hq, Hkv, L, D, block_m, block_n, sm_scale, causal,
                  nullptr, stream, q_index, schedule);
}

// ---- the variant that allocates nothing ------------------------------------------------------------------
// The row-ordering scratch of psa_fwd (cost and issue order of the rows) lives in a file-scope device array
// instead of a caller-provided workspace.  Every GPU holds its own copy of the array at its own address; the
// address is looked up once per device, with that device current, and only that pointer is ever handed to
// kernels (the array's name is a host-side stand-in, not a device address).
#include <mutex>

namespace {
constexpr int64_t FWD_NOALLOC_MAX_ROWS = 1 << 16;  // B * Hq * ceil(L / block_m)
constexpr size_t FWD_NOALLOC_BYTES = 2 * (size_t)(FWD_NOALLOC_MAX_ROWS + 16 * psa_order::MAX_PHASES) * sizeof(int32_t);
constexpr int FWD_NOALLOC_MAX_DEVICES = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[FWD_NOALLOC_BYTES];
static void* g_scratch_ptr[FWD_NOALLOC_MAX_DEVICES];
static std::mutex g_scratch_mutex;

extern "C" int64_t psa_fwd_noalloc_max_rows(void) { return FWD_NOALLOC_MAX_ROWS; }

extern "C" int psa_fwd_noalloc(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool,
                               const void* map, int map_elem_bytes, psa_tensor4 out, float* lse, int B, int Hq, int Hkv,
                               int L, int D, int block_m, int block_n, float sm_scale, int causal, psa_stream_t stream) {
  PSA_REQUIRE(B > 0 && Hq > 0 && L > 0 && block_m > 0, PSA_ERR_ARG, "psa_fwd_noalloc: B, H, L, block_m must be positive");
  const int64_t rows = (int64_t)B * Hq * ((L + block_m - 1) / block_m);
  PSA_REQUIRE(rows <= FWD_NOALLOC_MAX_ROWS, PSA_ERR_UNSUPPORTED,
              "psa_fwd_noalloc: %lld rows of the level map (B * Hq * ceil(L / block_m)) exceed the built-in scratch of %lld rows; "
              "use psa_fwd with a workspace", (long long)rows, (long long)FWD_NOALLOC_MAX_ROWS);
  PSA_REQUIRE(psa_fwd_workspace_bytes(B, Hq, L, block_m) <= (int64_t)FWD_NOALLOC_BYTES, PSA_ERR_UNSUPPORTED,
              "psa_fwd_noalloc: scratch too small for this shape");
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= FWD_NOALLOC_MAX_DEVICES) {
    psa_set_error("psa_fwd_noalloc: cannot identify the current device");
    return PSA_ERR_LAUNCH;
  }
  void* ptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
      void* p = nullptr;
      const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || p == nullptr) {
        psa_set_error("psa_fwd_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        return PSA_ERR_LAUNCH;
      }
      g_scratch_ptr[dev] = p;
    }
    ptr = g_scratch_ptr[dev];
  }
  // every entry of the scratch that a launch reads is written earlier in the same call (row costs, then the issue
  // order incl. its padding), so nothing has to be cleared between calls
  return fwd_impl(q, k, v, k_pool, v_pool, map, map_elem_bytes, out, lse, B, Hq, Hkv, L, D, block_m, block_n, sm_scale, causal, ptr,
                  stream);
}
