// Tile schedule of the row-walking attention kernels, built once per level map and kept in device memory.
//
// A (batch, head, q-block) row of the level map is walked as a sequence of TILES of 64 pooled keys of one level
// (psa_tiles.h).  The schedule stores that sequence per row so that the attention kernels neither compact the map
// row nor look block ids up per lane: with 128-key blocks every 16-key quarter of a tile lies inside ONE kv-block
// (the smallest pooled block holds 16 keys), so a tile is fully described by the source row of each quarter.
//
// Layout of the schedule buffer (all offsets from its start, `rows` = B * Hq * Mq):
//   reserved                                           64 bytes
//   order   int32 [order_entries]                      issue order of the rows (dealt to the XCDs, longest first), -1 = none
//   cost    int32 [rows]                               tiles per row, clamped to the sorter's range
//   tiles   int32 [rows]                               T: number of tiles of the row
//   records u32x4 [rows][rec_stride]                   one record per tile (+ 3), rec_stride = 2 * Nk + 4
//
// Record of a tile: four words, word g for the wave that copies tile rows 16g .. 16g+15 - each word is complete in
// itself, so a wave fetches one word per tile:
//   bits  0..19  first source row of that quarter, in the row numbering of the tile's level
//                (level 0: token index; level l: pooled row index of the level's [Npad >> l] rows)
//   bits 20..22  level code: 0..3 = pooling by 1, 2, 4, 8; 4 = a level-0 tile whose source rows run past the last
//                token (ragged: lanes clamp their rows to L - 1)
//   bit  23      masked: some slots are empty and / or the tile touches the causal diagonal
//   bits 24..30  nvalid: the first nvalid slots of the tile hold keys (0..64)
// Quarters past the end of a level's list point at the level's last retained block (any readable rows: masked).
// The last record of a row is repeated three times behind it (the kernels fetch records up to three tiles ahead).
#pragma once

#include "psa_common.h"

namespace psa_sched {

constexpr int REC_SRC_BITS = 20, REC_CODE_SHIFT = 20, REC_MASKED_BIT = 23, REC_NVALID_SHIFT = 24, REC_PAD = 3;
constexpr uint32_t REC_SRC_MASK = (1u << REC_SRC_BITS) - 1u;
constexpr uint32_t REC_CODE_RAGGED = 4;

struct Layout {
  int64_t order_off, cost_off, tiles_off, rec_off, bytes;
  int64_t order_entries;
  int rec_stride;
};

static inline int rec_stride_of(int Nk) { return 2 * Nk + 4; }

// byte offsets of the parts for `rows` rows; order_entries bounds any dealing of the rows (psa_order::deal)
static inline Layout layout(int64_t rows, int Nk, int64_t order_entries) {
  Layout l;
  l.rec_stride = rec_stride_of(Nk);
  l.order_entries = order_entries;
  l.order_off = 64;
  l.cost_off = l.order_off + ((order_entries * 4 + 63) & ~(int64_t)63);
  l.tiles_off = l.cost_off + ((rows * 4 + 63) & ~(int64_t)63);
  l.rec_off = l.tiles_off + ((rows * 4 + 63) & ~(int64_t)63);
  l.bytes = l.rec_off + rows * (int64_t)l.rec_stride * 16;
  return l;
}

// everything the host derives from a call's shape arguments (the buffer carries no header: nothing is read back)
struct Geometry {
  int64_t rows;
  int Mq, Nk;
  int wg_chunk, wg_groups;  // dealing of the rows: wg_groups shares of wg_chunk entries of order[]
  Layout lay;
};

__device__ __forceinline__ uint32_t rec_code(uint32_t w) { return (w >> REC_CODE_SHIFT) & 7u; }
__device__ __forceinline__ int rec_level(uint32_t w) { return (int)((w >> REC_CODE_SHIFT) & 3u); }
__device__ __forceinline__ bool rec_masked(uint32_t w) { return ((w >> REC_MASKED_BIT) & 1u) != 0; }
__device__ __forceinline__ int rec_nvalid(uint32_t w) { return (int)((w >> REC_NVALID_SHIFT) & 127u); }
__device__ __forceinline__ int rec_src(uint32_t w) { return (int)(w & REC_SRC_MASK); }

}  // namespace psa_sched

// host side (psa_schedule.hip)
// dealing of the rows of the forward walk to the XCDs
void psa_fwd_deal(int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, bool has_map, bool pairs, int& chunk, int& groups);
// shapes for which schedules exist
bool psa_schedule_shape_ok(int D, int block_m, int block_n, int L);
// geometry of the schedule of a shape; false when the shape has none
bool psa_schedule_geometry(int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, psa_sched::Geometry& g);
