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
                                                  int* s_cnt, int* s_ioff, int* s_toff, int* s_wcnt, int tid) {
  constexpr int NW = NT / 64;
  const int lane = tid & 63, wave = tid >> 6;
  // wave w owns columns [w * share, min(jmax, (w + 1) * share)), share a multiple of 64
  const int share = ((jmax + 64 * NW - 1) / (64 * NW)) * 64;
  const int j_lo = wave * share, j_hi = (wave + 1) * share < jmax ? (wave + 1) * share : jmax;
  int cnt[4] = {0, 0, 0, 0};
  int lvl_first = 0;  // the first 64 entries of the share stay in a register for the second pass
  if (map == nullptr) {
    cnt[0] = j_hi > j_lo ? j_hi - j_lo : 0;
  } else {
    for (int j0 = j_lo; j0 < j_hi; j0 += 64) {
      const int j = j0 + lane;
      const int lvl = j < j_hi ? load_map(map, mrow + j, map_elem) : 0;
      if (j0 == j_lo) lvl_first = lvl;
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
        int lvl = lvl_first;
        if (j0 != j_lo) lvl = j < j_hi ? load_map(map, mrow + j, map_elem) : 0;
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

template <int NT>
__device__ __forceinline__ int build_row_schedule(const void* map, int map_elem, int64_t mrow, int Nk, int jmax, int bn_log2,
                                                  int L, bool causal, int64_t q_first_row, uint16_t* ids, u32x2* tdesc,
                                                  int* s_cnt, int* s_ioff, int* s_toff, int* s_wcnt) {
  return build_row_schedule<NT>(map, map_elem, mrow, Nk, jmax, bn_log2, L, causal, q_first_row, ids, tdesc, s_cnt, s_ioff,
                                s_toff, s_wcnt, (int)threadIdx.x);
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

// ------------------------------------------------------------------------------------------------------
// LDS tile layout of the kernels that copy tiles with global_load_lds_dwordx4: 64 rows of D bf16 values.
//   * One copy instruction moves 1024 bytes (64 lanes x 16 bytes land at consecutive LDS addresses), i.e. a
//     BLOCK of RPB = 512 / D rows (4 rows of 256 bytes for D = 128, 8 rows of 128 bytes for D = 64); the blocks
//     of a tile are LT_ISTR = 1024 + 64 bytes apart.
//   * Row r of a block stores its 16-byte chunks XOR-swizzled: chunk c sits at position c ^ (r * RPB / 16)...
//     in short c ^ r for D = 128 and c ^ (r >> 1) for D = 64 (applied on the global side: a lane fetches the
//     chunk that belongs at its LDS position).
//   * Inside each group of 16 tile rows the rows are stored transposed (block n, row r holds tile row
//     RPL * r + n, RPL = 16 / RPB blocks per group), so the RPL rows a lane fetches are CONSECUTIVE tile rows.
// Padding and swizzle make the 128-bit row reads and the transposing reads bank-conflict free, and both only
// touch the low two bits of the chunk index, so every operand address is lane base + immediate.
// ------------------------------------------------------------------------------------------------------
constexpr int LT_ISTR = 1024 + 64;
template <int D>
struct LtGeom {
  static constexpr int CH = D / 8;          // 16-byte chunks per row
  static constexpr int RPB = 64 / CH;       // rows per block (per copy instruction)
  static constexpr int RPL = 16 / RPB;      // blocks per 16-row group = consecutive tile rows per lane
  static constexpr int BLOCKS = 64 / RPB;   // blocks per tile
  static constexpr int TILE = BLOCKS * LT_ISTR;
  static constexpr int SW_SHIFT = RPB == 4 ? 0 : 1;  // swizzle key of block row r: r >> SW_SHIFT (0..3)
  static constexpr int HALF = (32 / RPB) * LT_ISTR;  // byte distance of tile rows r and r + 32
  static constexpr int GROUP = RPL * LT_ISTR;        // byte distance of consecutive 16-row groups
};
constexpr int LT_TILE = LtGeom<128>::TILE;

#define PSA_LDS(T) __attribute__((address_space(3))) T*

// copy side: byte offset of the chunk a lane fetches, and the first of its RPL tile rows inside a 16-row group
template <int D>
__device__ __forceinline__ uint32_t lt_fetch_chunk(int lane) {
  using G = LtGeom<D>;
  const int r = lane / G::CH, pos = lane % G::CH;
  return (uint32_t)((pos ^ (r >> G::SW_SHIFT)) * 16);
}
template <int D>
__device__ __forceinline__ int lt_fetch_row(int lane) {
  using G = LtGeom<D>;
  return (lane / G::CH) * G::RPL;
}

// physical position of tile row `row`: block index and row inside the block
template <int D>
__device__ __forceinline__ void lt_place(int row, int& block, int& r) {
  using G = LtGeom<D>;
  const int in_group = row & 15;
  block = (row >> 4) * G::RPL + in_group % G::RPL;
  r = in_group / G::RPL;
}

// MFMA row operand (A: 32 tile rows x 16 channels) of k-step kk for tile row `row`, hh = lane / 32:
// off[kk & 1] + 64 * (kk >> 1)
template <int D>
__device__ __forceinline__ void lt_row_operand(int row, int hh, uint32_t (&off)[2]) {
  using G = LtGeom<D>;
  int block, r;
  lt_place<D>(row, block, r);
  const int base = block * LT_ISTR + r * (D * 2), f = r >> G::SW_SHIFT;
  off[0] = (uint32_t)(base + ((hh ^ f) * 16));
  off[1] = (uint32_t)(base + (((2 + hh) ^ f) * 16));
}

// MFMA transposed operand (A: 32 channels x 16 tile rows) through ds_read_b64_tr_b16.  Inside a block of 16
// lanes, lane i supplies the address of 4 channels (4*(i%4)..) of row i/4 and receives channel i of the
// block's 4 rows.  Lane block bl covers channels 32*db + 16*(bl&1).. and tile rows 16*grp + 8*s + 4*(bl>>1)..
// (s = first / second half of the operand): off[s] + 64 * db + GROUP * grp.  The row order inside the
// operand equals the order in which the 32x32 MFMA accumulator layout hands 8 consecutive registers to a lane.
template <int D>
__device__ __forceinline__ void lt_tr_operand(int lane, uint32_t (&off)[2]) {
  using G = LtGeom<D>;
  const int i16 = lane & 15, bl = lane >> 4;
  const int cl = 2 * (bl & 1) + ((i16 & 3) >> 1), hb = i16 & 1;
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    int block, r;
    lt_place<D>(8 * s + 4 * (bl >> 1) + (i16 >> 2), block, r);
    off[s] = (uint32_t)(block * LT_ISTR + r * (D * 2) + ((cl ^ (r >> G::SW_SHIFT)) * 16) + hb * 8);
  }
}

// Where the K / V rows of a tile come from (uniform per workgroup).
struct KvSource {
  const char *k0, *v0;      // level 0: this (batch, kv head) slice of K and V
  const char *kp, *vp;      // pooled buffers (all batches, heads and levels)
  uint32_t k_strb, v_strb;  // level-0 row strides in bytes
  int64_t BHkv, bhk, npad;
  int bn_log2, L;
};

// Source of tile t for the wave that copies the 16-row groups wave*G16 .. wave*G16 + G16 - 1
template <int G16>
struct TileSrc {
  const char *kbase, *vbase;
  uint32_t kstr, vstr;
  int lim;        // last valid row when the tile may run past the sequence end, else INT_MAX
  int src0[G16];  // first of the lane's consecutive source rows, per group
};

template <int D, int G16>
__device__ __forceinline__ void lt_tile_src(const KvSource& kv, const u32x2* tdesc, const uint16_t* ids, int t, int wave, int lane,
                                            TileSrc<G16>& a) {
  const u32x2 dd = tdesc[t];
  const uint32_t d0 = __builtin_amdgcn_readfirstlane(dd[0]);
  const uint32_t d1 = __builtin_amdgcn_readfirstlane(dd[1]);
  const int lv = d0 & 3, nvalid = (d0 >> 3) & 127, lt = d0 >> 10;
  const int cnt = d1 >> 16;
  const uint16_t* lids = ids + (d1 & 0xffff);
  const int sbs_log2 = kv.bn_log2 - lv;
  // max(lv - 1, 0) from a table in a constant: a saturating subtraction would be a vector instruction and drag the
  // 64-bit offset arithmetic below (and the copy base pointers) from the scalar to the vector unit
  const int lm1 = (0x2100 >> (4 * lv)) & 3;
  const int64_t pool_off = (kv.BHkv * (kv.npad - (kv.npad >> lm1)) + kv.bhk * (kv.npad >> lv)) * (D * 2);
  a.kbase = lv == 0 ? kv.k0 : kv.kp + pool_off;
  a.vbase = lv == 0 ? kv.v0 : kv.vp + pool_off;
  a.kstr = lv == 0 ? kv.k_strb : (uint32_t)(D * 2);
  a.vstr = lv == 0 ? kv.v_strb : (uint32_t)(D * 2);
  const bool ragged = nvalid < TK;  // some slots are empty: clamp them onto real rows (their logits are masked)
  a.lim = (ragged && lv == 0) ? kv.L - 1 : 0x7fffffff;
#pragma unroll
  for (int gi = 0; gi < G16; ++gi) {
    const int g = (lt << 6) + (wave * G16 + gi) * 16 + lt_fetch_row<D>(lane);
    int bi = g >> sbs_log2;
    if (ragged) bi = bi < cnt - 1 ? bi : cnt - 1;
    a.src0[gi] = ((int)lids[bi] << sbs_log2) + (g & ((1 << sbs_log2) - 1));
  }
}

// One global -> LDS copy instruction: lane l's 16 bytes at sbase + voff(l) land at LDS address lds_addr + 16 * l.
// sbase and lds_addr are wave-uniform.  Written as inline assembly on purpose: the compiler then does not know
// that a copy into LDS is in flight and so does not put a vmcnt(0) wait in front of every LDS read it cannot
// tell apart from the copy's target (it cannot for the transposing reads).  The kernels wait (vmcnt) and
// synchronise explicitly before a tile is read.
__device__ __forceinline__ const char* uniform_ptr(const char* p) {  // tells the compiler the value is wave-uniform
  const uint64_t a = (uint64_t)(uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return (const char*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ void lds_copy16(const char* sbase, uint32_t voff, uint32_t lds_addr) {
  sbase = uniform_ptr(sbase);
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory", "m0");
}
// the same with the target given as a uniform LDS address plus a compile-time byte offset (M0 = lds_base + OFF in one
// scalar instruction) and the lane offset row * str + chunk computed between the write of M0 and the copy (the
// instruction that the hardware needs between the two anyway): three instructions per copy
template <int OFF>
__device__ __forceinline__ void lds_copy16_row(const char* sbase, uint32_t row, uint32_t str, uint32_t chunk, uint32_t lds_base) {
  sbase = uniform_ptr(sbase);
  lds_base = __builtin_amdgcn_readfirstlane(lds_base);
  str = __builtin_amdgcn_readfirstlane(str);
  uint32_t voff;
  asm volatile("s_add_u32 m0, %1, %6\n\tv_mad_u32_u24 %0, %2, %3, %4\n\tglobal_load_lds_dwordx4 %0, %5"
               : "=&v"(voff)
               : "s"(lds_base), "v"(row), "s"(str), "v"(chunk), "s"(sbase), "n"(OFF)
               : "memory", "scc", "m0");
}
// the same with every address part but the lane offset in scalar registers: sbase is the (uniform) source of lane
// offset 0 and immediate 0, voff the lane's byte offset; no vector instruction per copy.  The instruction's immediate
// offset IMM is added to the global AND to the LDS address, so M0 gets the target minus IMM.
template <int OFF, int IMM>
__device__ __forceinline__ void lds_copy16_imm(const char* sbase, uint32_t voff, uint32_t lds_base) {
  static_assert(IMM >= 0 && IMM < 4096 && OFF >= IMM, "immediate offset range");
  sbase = uniform_ptr(sbase);
  lds_base = __builtin_amdgcn_readfirstlane(lds_base);
  asm volatile("s_add_u32 m0, %1, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2 offset:%4"
               :
               : "v"(voff), "s"(lds_base), "s"(sbase), "n"(OFF - IMM), "n"(IMM)
               : "memory", "scc", "m0");
}
// the same with a multiply-add a * b + c (a uniform) in the wait state between the write of M0 and the copy, where the
// hardware needs an instruction anyway: the caller passes one that it has to execute in any case
template <int OFF, int IMM>
__device__ __forceinline__ float lds_copy16_imm_fma(const char* sbase, uint32_t voff, uint32_t lds_base, float a, float b, float c) {
  static_assert(IMM >= 0 && IMM < 4096 && OFF >= IMM, "immediate offset range");
  sbase = uniform_ptr(sbase);
  lds_base = __builtin_amdgcn_readfirstlane(lds_base);
  a = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, a)));
  float r;
  asm volatile("s_add_u32 m0, %2, %4\n\tv_fma_f32 %0, %6, %7, %8\n\tglobal_load_lds_dwordx4 %1, %3 offset:%5"
               : "=&v"(r)
               : "v"(voff), "s"(lds_base), "s"(sbase), "n"(OFF - IMM), "n"(IMM), "s"(a), "v"(b), "v"(c)
               : "memory", "scc", "m0");
  return r;
}
// the same with a full per-lane address
__device__ __forceinline__ void lds_copy16_addr(const char* vaddr, uint32_t lds_addr) {
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr), "v"(vaddr) : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_addr_of(const void* p) { return (uint32_t)(uintptr_t)(PSA_LDS(const void))(p); }

// Copies this wave's groups of one tile: one block per instruction goes to block RPL*g16 + n of the tile at `dst`.
template <int D, int G16>
__device__ __forceinline__ void lt_issue_rows(unsigned char* dst, const char* base, uint32_t str, int lim, const int (&src0)[G16],
                                              int wave, uint32_t f_chunk) {
  using G = LtGeom<D>;
#pragma unroll
  for (int gi = 0; gi < G16; ++gi) {
    const int blk = (wave * G16 + gi) * G::RPL;
    if (lim == 0x7fffffff) {
      // the usual case: the uniform base pointer steps from row to row, the lane offset stays
      const uint32_t off = (uint32_t)src0[gi] * str + f_chunk;
#pragma unroll
      for (int n = 0; n < G::RPL; ++n) lds_copy16(base + (uint64_t)(n * str), off, lds_addr_of(dst + (blk + n) * LT_ISTR));
    } else {
#pragma unroll
      for (int n = 0; n < G::RPL; ++n) {
        const int src = src0[gi] + n < lim ? src0[gi] + n : lim;
        lds_copy16(base, (uint32_t)src * str + f_chunk, lds_addr_of(dst + (blk + n) * LT_ISTR));
      }
    }
  }
}

}  // namespace psa_tiles
