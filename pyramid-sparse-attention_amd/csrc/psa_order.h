// Issue order of workgroups: dealing to the XCDs and longest-first sorting (shared by the forward and backward walks).
//
// Workgroup ids are dealt round-robin to the 8 XCDs and each XCD runs its ids in order.  The work items (rows of the
// level map, or kv-block slots of the dK/dV walk) are cut into `groups` contiguous shares of `chunk` items, share g
// runs on XCD g % 8, the shares of an XCD one after the other: items that are neighbours (same head, so the same
// K/V or Q/dO) meet in one XCD's L2, and only a few heads are in flight at a time.  Inside a share the items are
// issued by decreasing cost, which shortens the tail of the launch.  The order only changes WHEN an item is
// computed, never its result.
#pragma once
#include "psa_common.h"

namespace psa_order {
namespace {  // one private copy per translation unit that launches them

constexpr int COST_BINS = 2048, COST_BITS = 11;
static_assert(COST_BINS == 1 << COST_BITS, "cost bins");
constexpr int RADIX_IPT = 16, RADIX_CHUNK = 256 * RADIX_IPT;  // shares up to this many items are radix-sorted in LDS
constexpr int SMALL_CHUNK = 512;  // shares up to this many items are ordered by rank counting in one pass
constexpr int MAX_PHASES = 64;
constexpr int64_t PHASE_BYTES = 128ll << 20;  // operand bytes (K/V + pooled levels, or Q/dO) in use at one time

// position in the dealt order of workgroup `bid` (chunk items per share): share ((bid >> 3) / chunk) * 8 + (bid & 7)
__device__ __forceinline__ int dealt_entry(int bid, int chunk) {
  return (((bid >> 3) / chunk) * 8 + (bid & 7)) * chunk + (bid >> 3) % chunk;
}

// shares for `total` items whose streamed operands take operand_bytes over n_heads (batch x head) slices
static inline void deal(int64_t total, double operand_bytes, int n_heads, int& chunk, int& groups) {
  int phases = (int)(operand_bytes / (double)PHASE_BYTES) + 1;
  const int max_phases = n_heads < MAX_PHASES ? n_heads : MAX_PHASES;
  phases = phases > max_phases ? max_phases : phases;
  groups = 8 * phases;
  chunk = (int)((total + groups - 1) / groups);
}

// tiles of 64 (pooled) keys that each row of the level map retains: the cost of a row walk
__global__ __launch_bounds__(256) void psa_row_cost_kernel(const void* map, int map_elem, int total, int Mq, int Nk, int bn_log2,
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

// one workgroup per share: stable counting sort of its items by decreasing cost (order[] holds item ids, -1 past the last item)
__global__ __launch_bounds__(256) void psa_chunk_sort_kernel(const int32_t* cost, int total, int chunk, int32_t* order) {
  __shared__ int hist[COST_BINS];
  const int x = blockIdx.x, tid = threadIdx.x;
  const int r0 = x * chunk;
  if (chunk <= SMALL_CHUNK) {
    // short shares (the usual case): the slot of an item is its rank among the keys (decreasing cost, then index) -
    // the same stable order as the counting sort below, without histogram, scan and their barriers
    __shared__ __attribute__((aligned(16))) uint32_t keys[SMALL_CHUNK];
    for (int i = tid; i < SMALL_CHUNK; i += 256)
      keys[i] = i < chunk && r0 + i < total ? ((uint32_t)(COST_BINS - 1 - cost[r0 + i]) << 16) | (uint32_t)i : 0xffffffffu;
    __syncthreads();
    const int n4 = (chunk + 3) >> 2;
    for (int i = tid; i < chunk; i += 256) {
      const uint32_t mine = keys[i];
      int rank = 0;
      for (int j = 0; j < n4; ++j) {
        const u32x4 k4 = ((const u32x4*)keys)[j];
        rank += (k4[0] < mine) + (k4[1] < mine) + (k4[2] < mine) + (k4[3] < mine);
      }
      if (mine != 0xffffffffu) order[r0 + rank] = r0 + i;
    }
    const int valid = total - r0 < chunk ? (total - r0 > 0 ? total - r0 : 0) : chunk;
    for (int i = valid + tid; i < chunk; i += 256) order[r0 + i] = -1;
    return;
  }
  if (chunk <= RADIX_CHUNK) {
    // medium shares: stable binary radix sort (least significant bit first) on the inverted cost, one bit per pass; a
    // thread owns a run of consecutive items, so "earlier" is (earlier thread, then earlier in the run)
    __shared__ uint32_t kbuf[2][RADIX_CHUNK];
    __shared__ int wave_tot[4];
    const int ipt = (chunk + 255) >> 8;  // items per thread (<= RADIX_IPT)
    const int i0 = tid * ipt;
    const int lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < chunk; i += 256)
      kbuf[0][i] = r0 + i < total ? ((uint32_t)(COST_BINS - 1 - cost[r0 + i]) << 16) | (uint32_t)i : 0xffffffffu;
    __syncthreads();
    int src = 0;
    for (int bit = 16; bit < 16 + COST_BITS; ++bit) {
      uint32_t k[RADIX_IPT];
      int zeros = 0;
#pragma unroll
      for (int e = 0; e < RADIX_IPT; ++e) {
        k[e] = (e < ipt && i0 + e < chunk) ? kbuf[src][i0 + e] : 0xffffffffu;
        zeros += (e < ipt && i0 + e < chunk && !((k[e] >> bit) & 1u)) ? 1 : 0;
      }
      // exclusive scan of the zero counts over the 256 threads
      int incl = zeros;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        incl += lane >= d ? up : 0;
      }
      if (lane == 63) wave_tot[wave] = incl;
      __syncthreads();
      int before = incl - zeros, all_zeros = 0;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        before += w < wave ? wave_tot[w] : 0;
        all_zeros += wave_tot[w];
      }
      int z = before, o = all_zeros + (i0 < chunk ? i0 : chunk) - before;  // next slot of a zero / of a one
#pragma unroll
      for (int e = 0; e < RADIX_IPT; ++e)
        if (e < ipt && i0 + e < chunk) {
          const bool one = (k[e] >> bit) & 1u;
          kbuf[src ^ 1][one ? o : z] = k[e];
          o += one ? 1 : 0;
          z += one ? 0 : 1;
        }
      __syncthreads();
      src ^= 1;
    }
    for (int i = tid; i < chunk; i += 256) {
      const uint32_t key = kbuf[src][i];
      order[r0 + i] = key != 0xffffffffu ? r0 + (int)(key & 0xffffu) : -1;
    }
    return;
  }
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
  // stable fill (items of equal cost keep their index order, so the issue order is the same in every run): 256 items at
  // a time, an item's slot = start of its bin + the number of earlier items of the same cost
  __shared__ int blk_cost[256];
  for (int i0 = 0; i0 < chunk; i0 += 256) {
    const int i = i0 + tid;
    const bool ok = i < chunk && r0 + i < total;
    const int c = ok ? cost[r0 + i] : -1;
    blk_cost[tid] = c;
    __syncthreads();
    int before = 0, after = 0;
    if (ok) {
      for (int j = 0; j < 256; ++j) {
        const bool same = blk_cost[j] == c;
        before += (same && j < tid) ? 1 : 0;
        after += (same && j > tid) ? 1 : 0;
      }
    }
    const int pos = ok ? hist[c] + before : 0;
    __syncthreads();
    if (ok) {
      order[r0 + pos] = r0 + i;
      if (after == 0) hist[c] = pos + 1;
    }
    __syncthreads();
  }
  // ids past the last row of the last share
  const int valid = total - r0 < chunk ? (total - r0 > 0 ? total - r0 : 0) : chunk;
  for (int i = valid + tid; i < chunk; i += 256) order[r0 + i] = -1;
}

}  // namespace
}  // namespace psa_order
