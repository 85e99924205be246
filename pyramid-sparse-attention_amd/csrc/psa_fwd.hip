// Pyramid sparse attention forward (non-causal and causal) on bf16 MFMA.
//
// One workgroup per (batch, head, q-block of BM = 32*NW rows); every wave owns 32 query rows.
//
//  * The workgroup first compacts its row of the level map into four per-level lists of kv-block
//    ids in LDS (ballot + popcount, ascending block order - deterministic).
//  * Work is then a sequence of TILES of 64 pooled keys of one level: a level-l kv-block holds
//    block_n/l pooled keys, so one tile is half a 128-key block, one 64-key block, or 64/(block_n/l)
//    small blocks of the same level packed side by side.  All tiles therefore cost the same MFMA
//    work whatever their level; only the last tile of a level can be partly empty.
//  * K tile -> LDS as [key][d] (row pad 16 B), V tile -> LDS TRANSPOSED as [d][key] (row pad 8 B):
//    the 4x8 register transpose is done with v_perm while staging, so that both MFMA operands are
//    read from LDS with the contraction index contiguous.
//  * The kernel computes the transposed problem  S^T = K Q^T  (32 keys x 32 queries per MFMA,
//    v_mfma_f32_32x32x16_bf16) and  O^T += V^T P^T.  In the MFMA accumulator layout a lane then
//    holds 16 keys of ONE query column: the softmax row max / row sum are in-lane reductions plus a
//    single exchange between the two half-waves, and P^T is already in B-operand layout (the
//    key<->slot permutation it implies is applied to the V^T reads, which is free).
//  * Online softmax in base 2: p = exp2(s*scale*log2e + log2(level) - m).
//  * Global loads of tile t+1 are issued before the math of tile t (register prefetch).
//
// Roofline: MFMA-bound; 4*BM*64*D flops per tile.
#include "psa_common.h"

namespace {

constexpr int TK = 64;  // pooled keys per tile

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
  int total_wg, wg_chunk;
};

template <int D>
struct Smem {
  static constexpr int KST = D * 2 + 16;   // bytes per K row
  static constexpr int VST = TK * 2 + 8;   // bytes per V^T row
  static constexpr int K_BYTES = TK * KST;
  static constexpr int V_BYTES = D * VST;
  static constexpr int OST = D * 2 + 16;   // bytes per O staging row
  static constexpr int tile_region(int bm) {  // K/V tiles and the O staging area share this region
    return (K_BYTES + V_BYTES) > bm * OST ? (K_BYTES + V_BYTES) : bm * OST;
  }
};

// source row (in the level's own row numbering) of tile slot r; returns -1 when the slot is empty
__device__ __forceinline__ int slot_src(int lv, int lt, int r, int sbs_log2, int cnt, const uint16_t* ids, int L) {
  int src;
  if (sbs_log2 >= 6) {
    const int tpb_log2 = sbs_log2 - 6;
    const int bi = lt >> tpb_log2;
    const int part = lt & ((1 << tpb_log2) - 1);
    src = ((int)ids[bi] << sbs_log2) + (part << 6) + r;
  } else {
    const int bi = (lt << (6 - sbs_log2)) + (r >> sbs_log2);
    if (bi >= cnt) return -1;
    src = ((int)ids[bi] << sbs_log2) + (r & ((1 << sbs_log2) - 1));
  }
  if (lv == 0 && src >= L) return -1;
  return src;
}

template <int D, int NW>
__global__ __launch_bounds__(NW * 64, 2) void psa_fwd_kernel(FwdParams p) {
  constexpr int NT = NW * 64;
  constexpr int BM = NW * 32;
  constexpr int CH = D / 8;           // 16-byte chunks per row
  constexpr int UNITS = 16 * CH;      // (4 keys x 1 chunk) units per tile
  constexpr int PER = (UNITS + NT - 1) / NT;
  constexpr int KK = D / 16;          // MFMA k-steps for QK^T
  constexpr int DB = D / 32;          // 32-row blocks of O^T
  using SM = Smem<D>;

  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* Ks = smem;
  unsigned char* Vt = smem + SM::K_BYTES;
  uint16_t* ids = (uint16_t*)(smem + SM::tile_region(NW * 32));
  __shared__ int s_cnt[4];

  // XCD-aware decode: consecutive workgroup ids go round-robin over the 8 XCDs; give each XCD a
  // contiguous range of (b, h, q-block) so that one XCD's L2 sees few heads at a time.
  const int bid = blockIdx.x;
  const int logical = (bid & 7) * p.wg_chunk + (bid >> 3);
  if (logical >= p.total_wg) return;
  const int I = logical % p.Mq;
  const int bh = logical / p.Mq;
  const int h = bh % p.Hq, b = bh / p.Hq;
  const int hk = h / (p.Hq / p.Hkv);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;

  // ---- 1. compact the map row into per-level lists ------------------------------------
  int jmax = p.Nk;
  if (p.causal) {
    const int ce = (int)((((int64_t)(I + 1) * p.bm) + (1 << p.bn_log2) - 1) >> p.bn_log2);
    jmax = ce < jmax ? ce : jmax;
  }
  if (wave == 0) {
    int cnt[4] = {0, 0, 0, 0};
    const int64_t mrow = ((int64_t)bh * p.Mq + I) * p.Nk;
    if (p.map == nullptr) {
      cnt[0] = jmax;
      for (int j = lane; j < jmax; j += 64) ids[j] = (uint16_t)j;
    } else {
      for (int j0 = 0; j0 < jmax; j0 += 64) {
        const int j = j0 + lane;
        const int lvl = j < jmax ? load_map(p.map, mrow + j, p.map_elem) : 0;
#pragma unroll
        for (int lv = 0; lv < 4; ++lv) cnt[lv] += __popcll(__ballot(lvl == (1 << lv)));
      }
      int run[4];
      run[0] = 0; run[1] = cnt[0]; run[2] = cnt[0] + cnt[1]; run[3] = cnt[0] + cnt[1] + cnt[2];
      const uint64_t lt_mask = (1ull << lane) - 1ull;
      for (int j0 = 0; j0 < jmax; j0 += 64) {
        const int j = j0 + lane;
        const int lvl = j < jmax ? load_map(p.map, mrow + j, p.map_elem) : 0;
#pragma unroll
        for (int lv = 0; lv < 4; ++lv) {
          const uint64_t bal = __ballot(lvl == (1 << lv));
          if (lvl == (1 << lv)) ids[run[lv] + __popcll(bal & lt_mask)] = (uint16_t)j;
          run[lv] += __popcll(bal);
        }
      }
    }
    if (lane < 4) s_cnt[lane] = lane == 0 ? cnt[0] : lane == 1 ? cnt[1] : lane == 2 ? cnt[2] : cnt[3];
  }

  // ---- 2. Q fragments (B operand of S^T = K Q^T): lane holds Q[row l32][16*kk + 8*hh .. +8] ---
  const int q_row0 = I * BM + wave * 32;
  bf16x8 qf[KK];
  {
    int qr = q_row0 + l32;
    qr = qr < p.L ? qr : p.L - 1;
    const bf16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)qr * p.q_sl + hh * 8;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const bf16x8*)(qp + kk * 16);
  }
  __syncthreads();

  int cnt[4], toff[5], ioff[4];
  toff[0] = 0;
  {
    int io = 0;
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) {
      cnt[lv] = s_cnt[lv];
      ioff[lv] = io;
      io += cnt[lv];
      const int sbs_log2 = p.bn_log2 - lv;
      const int nt = sbs_log2 >= 6 ? (cnt[lv] << (sbs_log2 - 6)) : ((cnt[lv] << sbs_log2) + 63) >> 6;
      toff[lv + 1] = toff[lv] + nt;
    }
  }
  const int T = toff[4];

  // level bases
  const bf16_t* kbase[4];
  const bf16_t* vbase[4];
  int64_t kstr[4], vstr[4];
  kbase[0] = p.k + b * p.k_sb + hk * p.k_sh;
  vbase[0] = p.v + b * p.v_sb + hk * p.v_sh;
  kstr[0] = p.k_sl;
  vstr[0] = p.v_sl;
  {
    const int64_t BH = (int64_t)p.B * p.Hkv;
    const int64_t bhk = (int64_t)b * p.Hkv + hk;
    int64_t off = 0;
#pragma unroll
    for (int lv = 1; lv < 4; ++lv) {
      const int64_t n_l = p.npad >> lv;
      kbase[lv] = p.kp + off + bhk * n_l * D;
      vbase[lv] = p.vp + off + bhk * n_l * D;
      kstr[lv] = D;
      vstr[lv] = D;
      off += BH * n_l * D;
    }
  }

  auto tile_level = [&](int t) -> int { return t < toff[1] ? 0 : (t < toff[2] ? 1 : (t < toff[3] ? 2 : 3)); };

  u32x4 kreg[PER][4], vreg[PER][4];
  auto load_tile = [&](int t) {
    const int lv = tile_level(t);
    const int lt = t - toff[lv];
    const int sbs_log2 = p.bn_log2 - lv;
    const bf16_t* kb = lv == 0 ? kbase[0] : (lv == 1 ? kbase[1] : (lv == 2 ? kbase[2] : kbase[3]));
    const bf16_t* vb = lv == 0 ? vbase[0] : (lv == 1 ? vbase[1] : (lv == 2 ? vbase[2] : vbase[3]));
    const int64_t ks = lv == 0 ? kstr[0] : D;
    const int64_t vs = lv == 0 ? vstr[0] : D;
    const int c = lv == 0 ? cnt[0] : (lv == 1 ? cnt[1] : (lv == 2 ? cnt[2] : cnt[3]));
    const int io = lv == 0 ? ioff[0] : (lv == 1 ? ioff[1] : (lv == 2 ? ioff[2] : ioff[3]));
#pragma unroll
    for (int u_ = 0; u_ < PER; ++u_) {
      const int u = tid + u_ * NT;
      if (UNITS % NT != 0 && u >= UNITS) break;
      const int r0 = (u / CH) * 4, ch = u % CH;
      const int src0 = slot_src(lv, lt, r0, sbs_log2, c, ids + io, p.L);  // 4 rows share a sub-block
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int src = src0 + i;
        const bool ok = src0 >= 0 && (lv != 0 || src < p.L);
        u32x4 z = {0u, 0u, 0u, 0u};
        kreg[u_][i] = ok ? *(const u32x4*)(kb + (int64_t)src * ks + ch * 8) : z;
        vreg[u_][i] = ok ? *(const u32x4*)(vb + (int64_t)src * vs + ch * 8) : z;
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
      for (int i = 0; i < 4; ++i) *(u32x4*)(Ks + (r0 + i) * SM::KST + ch * 16) = kreg[u_][i];
      // transpose 4 keys x 8 channels -> 8 channels x 4 keys
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32x2 e0, e1;
        e0[0] = __builtin_amdgcn_perm(vreg[u_][1][j], vreg[u_][0][j], 0x05040100u);
        e0[1] = __builtin_amdgcn_perm(vreg[u_][3][j], vreg[u_][2][j], 0x05040100u);
        e1[0] = __builtin_amdgcn_perm(vreg[u_][1][j], vreg[u_][0][j], 0x07060302u);
        e1[1] = __builtin_amdgcn_perm(vreg[u_][3][j], vreg[u_][2][j], 0x07060302u);
        *(u32x2*)(Vt + (ch * 8 + 2 * j) * SM::VST + r0 * 2) = e0;
        *(u32x2*)(Vt + (ch * 8 + 2 * j + 1) * SM::VST + r0 * 2) = e1;
      }
    }
  };

  // ---- 3. main loop -------------------------------------------------------------------
  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
  float m_run = -INFINITY;  // running max (log2 domain), same in both half-waves
  float l_run = 0.f;        // this lane's partial row sum
  const int q_idx = q_row0 + l32;

  if (T > 0) load_tile(0);
  for (int t = 0; t < T; ++t) {
    __syncthreads();
    store_tile();
    __syncthreads();
    const int lv = tile_level(t);
    const int lt = t - toff[lv];
    const int sbs_log2 = p.bn_log2 - lv;
    const int c_lv = lv == 0 ? cnt[0] : (lv == 1 ? cnt[1] : (lv == 2 ? cnt[2] : cnt[3]));
    const int io_lv = lv == 0 ? ioff[0] : (lv == 1 ? ioff[1] : (lv == 2 ? ioff[2] : ioff[3]));
    if (t + 1 < T) load_tile(t + 1);

    // valid slots form a prefix of the tile
    int nvalid = TK;
    int last_blk;
    if (sbs_log2 >= 6) {
      last_blk = ids[io_lv + (lt >> (sbs_log2 - 6))];
      if (lv == 0) {
        const int rem = p.L - ((last_blk << sbs_log2) + ((lt & ((1 << (sbs_log2 - 6)) - 1)) << 6));
        nvalid = rem < TK ? rem : TK;
      }
    } else {
      const int bpt = 1 << (6 - sbs_log2);
      int nb = c_lv - lt * bpt;
      nb = nb < bpt ? nb : bpt;
      last_blk = ids[io_lv + lt * bpt + nb - 1];
      nvalid = nb << sbs_log2;
      if (lv == 0) {
        const int rem = p.L - (last_blk << sbs_log2);
        if (rem < (1 << sbs_log2)) nvalid -= (1 << sbs_log2) - rem;
      }
    }
    const bool diag = p.causal && ((((int64_t)last_blk + 1) << p.bn_log2) - 1 > (int64_t)I * p.bm);
    const bool masked = diag || nvalid < TK;
    const int nchunk = nvalid > 32 ? 2 : 1;

    // S^T chunks: 32 keys x 32 queries each
    f32x16 s[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[c][i] = 0.f;
      if (c < nchunk) {
        const unsigned char* kr = Ks + (c * 32 + l32) * SM::KST + hh * 16;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const bf16x8 a = *(const bf16x8*)(kr + kk * 32);
          s[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[kk], s[c], 0, 0, 0);
        }
      }
    }

    if (masked) {
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int r0 = c * 32 + g * 8 + hh * 4;
          int src0 = -1;
          if (r0 < nvalid) src0 = slot_src(lv, lt, r0, sbs_log2, c_lv, ids + io_lv, p.L);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            bool ok = src0 >= 0 && (r0 + e) < nvalid;
            if (ok && p.causal) ok = (((int64_t)(src0 + e) + 1) << lv) - 1 <= (int64_t)q_idx;
            if (!ok) s[c][g * 4 + e] = -INFINITY;
          }
        }
    }

    // online softmax over this tile (per query column = per lane, both half-waves)
    float mx = s[0][0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[0][i]);
    if (nchunk == 2) {
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[1][i]);
    }
    mx = fmaxf(mx, shfl_xor32(mx));
    const float bias = (float)lv;
    float m_new = fmaxf(m_run, mx * p.scale_log2 + bias);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // rows that still see no key
    const float alpha = fast_exp2(m_run - m_use);
    const float nb = bias - m_use;
    float lsum = 0.f;
    uint32_t pk[2][8];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (c < nchunk) {
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const float p0 = fast_exp2(__builtin_fmaf(s[c][i], p.scale_log2, nb));
          const float p1 = fast_exp2(__builtin_fmaf(s[c][i + 1], p.scale_log2, nb));
          lsum += p0 + p1;
          pk[c][i >> 1] = pack_bf16x2(p0, p1);
        }
      }
    }
    l_run = l_run * alpha + lsum;
    m_run = m_new;

    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][i] *= alpha;
    }

    // O^T += V^T P^T : per 16-key group g, A = V^T[32 d][16 keys], B = P^T[16 keys][32 q]
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (c < nchunk) {
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          u32x4 bw = {pk[c][g * 4 + 0], pk[c][g * 4 + 1], pk[c][g * 4 + 2], pk[c][g * 4 + 3]};
          const bf16x8 bfrag = __builtin_bit_cast(bf16x8, bw);
          const int key0 = c * 32 + g * 16 + hh * 4;
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const unsigned char* vr = Vt + (db * 32 + l32) * SM::VST + key0 * 2;
            const u32x2 lo = *(const u32x2*)(vr);
            const u32x2 hi = *(const u32x2*)(vr + 16);
            u32x4 aw = {lo[0], lo[1], hi[0], hi[1]};
            acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, aw), bfrag, acc[db], 0, 0, 0);
          }
        }
      }
    }
  }

  // ---- 4. epilogue --------------------------------------------------------------------
  float l_tot = l_run + shfl_xor32(l_run);
  const float l_safe = fmaxf(l_tot, 1e-8f);
  const float inv = 1.0f / l_safe;
  if (p.lse != nullptr && hh == 0 && q_idx < p.L) {
    // natural-log domain: m*ln2 + ln(max(l, 1e-8))
    p.lse[((int64_t)b * p.Hq + h) * p.L + q_idx] = (m_run + fast_log2(l_safe)) * 0.6931471805599453f;
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
      *(u32x2*)(Os + (wave * 32 + l32) * SM::OST + (db * 32 + g * 8 + hh * 4) * 2) = w;
    }
  __syncthreads();
  bf16_t* ob = p.o + b * p.o_sb + h * p.o_sh;
  for (int u = tid; u < BM * CH; u += NT) {
    const int r = u / CH, ch = u % CH;
    const int row = I * BM + r;
    if (row < p.L) *(u32x4*)(ob + (int64_t)row * p.o_sl + ch * 8) = *(const u32x4*)(Os + r * SM::OST + ch * 16);
  }
}

template <int D, int NW>
int launch_fwd(const FwdParams& p, int Nk, hipStream_t stream) {
  using SM = Smem<D>;
  size_t shmem = (size_t)SM::tile_region(NW * 32) + (size_t)Nk * 2;
  if (shmem > 48 * 1024) {
    if (hipFuncSetAttribute((const void*)psa_fwd_kernel<D, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess)
      return PSA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((psa_fwd_kernel<D, NW>), dim3((unsigned)(p.wg_chunk * 8)), dim3(NW * 64), shmem, stream, p);
  return PSA_OK;
}

}  // namespace

extern "C" int psa_fwd(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool,
                       const void* map, int map_elem_bytes, psa_tensor4 out, float* lse, int B, int Hq, int Hkv, int L,
                       int D, int block_m, int block_n, float sm_scale, int causal, psa_stream_t stream) {
  PSA_REQUIRE(q.ptr && k.ptr && v.ptr && out.ptr, PSA_ERR_ARG, "psa_fwd: null pointer");
  PSA_REQUIRE(map == nullptr || (k_pool && v_pool), PSA_ERR_ARG, "psa_fwd: pooled K/V required with a level map");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_fwd: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && L > 0, PSA_ERR_ARG, "psa_fwd: B, H, L must be positive");
  PSA_REQUIRE(Hq % Hkv == 0, PSA_ERR_ARG, "psa_fwd: Hq=%d must be a multiple of Hkv=%d", Hq, Hkv);
  PSA_REQUIRE(D == 64 || D == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: head dim %d not in {64, 128}", D);
  PSA_REQUIRE(block_m == 64 || block_m == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: block_m=%d not in {64, 128}", block_m);
  PSA_REQUIRE(block_n == 32 || block_n == 64 || block_n == 128, PSA_ERR_UNSUPPORTED, "psa_fwd: block_n=%d not in {32, 64, 128}", block_n);
  const psa_tensor4* ts[4] = {&q, &k, &v, &out};
  for (int i = 0; i < 4; ++i)
    PSA_REQUIRE(((uintptr_t)ts[i]->ptr % 16 == 0) && ts[i]->stride_b % 8 == 0 && ts[i]->stride_h % 8 == 0 && ts[i]->stride_l % 8 == 0,
                PSA_ERR_UNSUPPORTED, "psa_fwd: tensors must be 16-byte aligned with strides that are multiples of 8 elements");
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
  p.wg_chunk = (int)((total + 7) / 8);
  int rc;
  if (D == 128 && block_m == 128) rc = launch_fwd<128, 4>(p, Nk, (hipStream_t)stream);
  else if (D == 128) rc = launch_fwd<128, 2>(p, Nk, (hipStream_t)stream);
  else if (block_m == 128) rc = launch_fwd<64, 4>(p, Nk, (hipStream_t)stream);
  else rc = launch_fwd<64, 2>(p, Nk, (hipStream_t)stream);
  PSA_REQUIRE(rc == PSA_OK, rc, "psa_fwd: launch configuration failed (LDS)");
  return psa_check_launch("psa_fwd");
}
