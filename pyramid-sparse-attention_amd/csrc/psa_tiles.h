// Tile bookkeeping shared by the row-walking attention kernels.
//
// A (batch, head, q-block) row of the level map is compacted into four per-level lists of kv-block
// ids; the retained blocks of one level form a stream of cnt * (block_n >> level) pooled keys that is
// cut into tiles of 64 keys.  A 32-bit pair describes a tile:
//   word 0: level (2 bits) | masked (1) | nvalid 0..64 (7) | tile index inside the level (22)
//   word 1: offset of the level's block list (16) | number of blocks of the level (16)
#pragma once

#include "psa_common.h"

namespace psa_tiles {

constexpr int TK = 64;  // pooled keys per tile

__device__ __forceinline__ u32x2 make_desc(int lv, bool masked, int nvalid, int lt, int ioff, int cnt) {
  u32x2 d;
  d[0] = (uint32_t)lv | ((uint32_t)masked << 2) | ((uint32_t)nvalid << 3) | ((uint32_t)lt << 10);
  d[1] = (uint32_t)ioff | ((uint32_t)cnt << 16);
  return d;
}

// Source row (in the level's own row numbering) of tile slot r, or -1 when the slot is empty.
__device__ __forceinline__ int slot_src(int lv, int lt, int r, int sbs_log2, int cnt, const uint16_t* ids, int L) {
  const int g = (lt << 6) + r;
  const int bi = g >> sbs_log2;
  if (bi >= cnt) return -1;
  const int src = ((int)ids[bi] << sbs_log2) + (g & ((1 << sbs_log2) - 1));
  return (lv == 0 && src >= L) ? -1 : src;
}

struct RowSchedule {
  int T;  // number of tiles
};

// Builds ids[] (kv-block ids grouped by level, ascending inside a level) and tdesc[] for the map row
// of (bh, q-block I).  Must be called by every thread of the workgroup; contains barriers.
// s_cnt / s_ioff / s_toff are 4 / 4 / 5 ints of LDS scratch; s_wcnt holds 4 ints per wave.
// Every wave compacts one contiguous share of the row: counts first (one pass over the map row), then,
// once the per-wave counts are known to all, the ids (second pass; the row is in cache by then).
template <int NT>
__device__ __forceinline__ int build_row_schedule(const void* map, int map_elem, int64_t mrow, int Nk, int jmax, int bn_log2,
                                                  int L, bool causal, int64_t q_first_row, uint16_t* ids, u32x2* tdesc,
                                                  int* s_cnt, int* s_ioff, int* s_toff, int* s_wcnt) {
  constexpr int NW = NT / 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // wave w owns columns [w * share, min(jmax, (w + 1) * share)), share a multiple of 64
  const int share = ((jmax + 64 * NW - 1) / (64 * NW)) * 64;
  const int j_lo = wave * share, j_hi = (wave + 1) * share < jmax ? (wave + 1) * share : jmax;
  int cnt[4] = {0, 0, 0, 0};
  if (map == nullptr) {
    cnt[0] = j_hi > j_lo ? j_hi - j_lo : 0;
  } else {
    for (int j0 = j_lo; j0 < j_hi; j0 += 64) {
      const int j = j0 + lane;
      const int lvl = j < j_hi ? load_map(map, mrow + j, map_elem) : 0;
#pragma unroll
      for (int lv = 0; lv < 4; ++lv) cnt[lv] += __popcll(__ballot(lvl == (1 << lv)));
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) s_wcnt[wave * 4 + lv] = cnt[lv];
  }
  __syncthreads();
  {
    // offsets of this wave's share inside each level list; totals for the tile bookkeeping
    int run[4], tot[4];
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) {
      int before = 0, all = 0;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const int c = s_wcnt[w * 4 + lv];
        before += w < wave ? c : 0;
        all += c;
      }
      run[lv] = before;
      tot[lv] = all;
    }
    run[1] += tot[0];
    run[2] += tot[0] + tot[1];
    run[3] += tot[0] + tot[1] + tot[2];
    if (map == nullptr) {
      for (int j = j_lo + lane; j < j_hi; j += 64) ids[j] = (uint16_t)j;
    } else {
      const uint64_t lt_mask = (1ull << lane) - 1ull;
      for (int j0 = j_lo; j0 < j_hi; j0 += 64) {
        const int j = j0 + lane;
        const int lvl = j < j_hi ? load_map(map, mrow + j, map_elem) : 0;
#pragma unroll
        for (int lv = 0; lv < 4; ++lv) {
          const uint64_t bal = __ballot(lvl == (1 << lv));
          if (lvl == (1 << lv)) ids[run[lv] + __popcll(bal & lt_mask)] = (uint16_t)j;
          run[lv] += __popcll(bal);
        }
      }
    }
    if (tid == 0) {
      int io = 0, to = 0;
#pragma unroll
      for (int lv = 0; lv < 4; ++lv) {
        const int c = tot[lv];
        const int sbs_log2 = bn_log2 - lv;
        s_cnt[lv] = c;
        s_ioff[lv] = io;
        s_toff[lv] = to;
        io += c;
        to += ((c << sbs_log2) + 63) >> 6;
      }
      s_toff[4] = to;
    }
  }
  __syncthreads();
  const int T = __builtin_amdgcn_readfirstlane(s_toff[4]);
  for (int t = tid; t < T; t += NT) {
    const int lv = (t >= s_toff[1]) + (t >= s_toff[2]) + (t >= s_toff[3]);
    const int lt = t - s_toff[lv];
    const int c_lv = s_cnt[lv];
    const int io_lv = s_ioff[lv];
    const int sbs_log2 = bn_log2 - lv;
    // valid slots form a prefix of the tile: the level's stream ends, or (level 0) the sequence does
    int nvalid = (c_lv << sbs_log2) - (lt << 6);
    nvalid = nvalid < TK ? nvalid : TK;
    const int last_blk = ids[io_lv + (((lt << 6) + nvalid - 1) >> sbs_log2)];
    if (lv == 0) {
      const int over = (((lt << 6) + nvalid - 1) & ((1 << sbs_log2) - 1)) + 1 - (L - (last_blk << sbs_log2));
      if (over > 0) nvalid = nvalid - over > 0 ? nvalid - over : 0;
    }
    const bool diag = causal && ((((int64_t)last_blk + 1) << bn_log2) - 1 > q_first_row);
    tdesc[t] = make_desc(lv, diag || nvalid < TK, nvalid, lt, io_lv, c_lv);
  }
  __syncthreads();
  return T;
}

struct TileRef {
  int lv, lt, cnt, sbs_log2, nvalid;
  bool masked;
  const uint16_t* ids;
};

__device__ __forceinline__ TileRef tile_ref(const u32x2* tdesc, const uint16_t* ids, int t, int bn_log2) {
  const u32x2 d = tdesc[t];
  const uint32_t d0 = __builtin_amdgcn_readfirstlane(d[0]);
  const uint32_t d1 = __builtin_amdgcn_readfirstlane(d[1]);
  TileRef r;
  r.lv = d0 & 3;
  r.masked = (d0 & 4) != 0;
  r.nvalid = (d0 >> 3) & 127;
  r.lt = d0 >> 10;
  r.cnt = d1 >> 16;
  r.ids = ids + (d1 & 0xffff);
  r.sbs_log2 = bn_log2 - r.lv;
  return r;
}

// worst-case number of tiles of one map row
static inline int max_tiles(int Nk, int block_n) { return (Nk * block_n + 63) / 64 + 4; }

// offset (in elements of D-wide rows) of pooled level lv >= 1 inside a pooled buffer, for (b, h_kv)
__device__ __forceinline__ int64_t pool_row_offset(int lv, int64_t BHkv, int64_t bhk, int64_t npad) {
  const int lm1 = lv > 0 ? lv - 1 : 0;
  return BHkv * (npad - (npad >> lm1)) + bhk * (npad >> lv);
}

}  // namespace psa_tiles
