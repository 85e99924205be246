// Builds the tile schedule of a level map (psa_schedule.h): one pass over the map, one wave per (batch, head,
// q-block) row, followed by the longest-first issue order of the rows (psa_order.h).  HBM-bound on the map
// (rows * Nk bytes in, about 16 bytes per retained tile out); latency-bound at the usual sizes.
#include "psa_common.h"
#include "psa_order.h"
#include "psa_schedule.h"

namespace {

constexpr int ROWS_PER_WG = 4;

__global__ __launch_bounds__(64 * ROWS_PER_WG) void psa_sched_build_kernel(const void* map, int map_elem, int rows, int Mq, int Nk,
                                                                          int bn_log2, int bm, int L, int causal, int32_t* cost,
                                                                          int32_t* tiles, u32x4* recs, int rec_stride) {
  extern __shared__ uint16_t s_ids[];  // [ROWS_PER_WG][Nk]: kv-block ids of a row, grouped by level, ascending inside a level
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = blockIdx.x * ROWS_PER_WG + wave;
  const bool live = row < rows;
  uint16_t* ids = s_ids + wave * Nk;
  const int I = live ? row % Mq : 0;
  int jmax = live ? Nk : 0;
  if (causal) {
    const int ce = (int)((((int64_t)(I + 1) * bm) + (1 << bn_log2) - 1) >> bn_log2);
    jmax = ce < jmax ? ce : jmax;
  }
  const int64_t mrow = (int64_t)row * Nk;
  int cnt[4] = {0, 0, 0, 0};
  for (int j0 = 0; j0 < jmax; j0 += 64) {
    const int j = j0 + lane;
    const int lvl = j < jmax ? load_map(map, mrow + j, map_elem) : 0;
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) cnt[lv] += __popcll(__ballot(lvl == (1 << lv)));
  }
  int io[4], to[5];
  {
    int i = 0, t = 0;
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) {
      io[lv] = i;
      to[lv] = t;
      i += cnt[lv];
      t += ((cnt[lv] << (bn_log2 - lv)) + 63) >> 6;
    }
    to[4] = t;
  }
  {
    int run[4] = {io[0], io[1], io[2], io[3]};
    const uint64_t lt_mask = (1ull << lane) - 1ull;
    for (int j0 = 0; j0 < jmax; j0 += 64) {
      const int j = j0 + lane;
      const int lvl = j < jmax ? load_map(map, mrow + j, map_elem) : 0;
#pragma unroll
      for (int lv = 0; lv < 4; ++lv) {
        const uint64_t bal = __ballot(lvl == (1 << lv));
        if (lvl == (1 << lv)) ids[run[lv] + __popcll(bal & lt_mask)] = (uint16_t)j;
        run[lv] += __popcll(bal);
      }
    }
  }
  __syncthreads();  // (a wave only reads its own ids; the barrier orders the writes before the reads)
  const int T = to[4];
  u32x4* out = recs + (int64_t)row * rec_stride;
  if (live && lane == 0) {
    tiles[row] = T;
    cost[row] = T < psa_order::COST_BINS - 1 ? T : psa_order::COST_BINS - 1;
  }
  const int64_t q_first_row = (int64_t)I * bm;
  for (int t = lane; t < T; t += 64) {
    const int lv = (t >= to[1]) + (t >= to[2]) + (t >= to[3]);
    int lt = t, c_lv = cnt[0], io_lv = io[0];
#pragma unroll
    for (int l = 1; l < 4; ++l)
      if (lv == l) {
        lt = t - to[l];
        c_lv = cnt[l];
        io_lv = io[l];
      }
    const int sbs_log2 = bn_log2 - lv;
    int nvalid = (c_lv << sbs_log2) - (lt << 6);
    nvalid = nvalid < 64 ? nvalid : 64;
    const int last_blk = ids[io_lv + (((lt << 6) + nvalid - 1) >> sbs_log2)];
    if (lv == 0) {
      const int over = (((lt << 6) + nvalid - 1) & ((1 << sbs_log2) - 1)) + 1 - (L - (last_blk << sbs_log2));
      if (over > 0) nvalid = nvalid - over > 0 ? nvalid - over : 0;
    }
    const bool diag = causal && ((((int64_t)last_blk + 1) << bn_log2) - 1 > q_first_row);
    u32x4 r;
    bool ragged = false;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int gpos = (lt << 6) + 16 * g;
      int bi = gpos >> sbs_log2;
      bi = bi < c_lv - 1 ? bi : c_lv - 1;
      const int src = ((int)ids[io_lv + bi] << sbs_log2) + (gpos & ((1 << sbs_log2) - 1));
      ragged |= lv == 0 && src + 15 >= L;
      r[g] = (uint32_t)src;
    }
    const uint32_t hi = ((ragged ? psa_sched::REC_CODE_RAGGED : (uint32_t)lv) << psa_sched::REC_CODE_SHIFT) |
                        ((uint32_t)(diag || nvalid < 64) << psa_sched::REC_MASKED_BIT) | ((uint32_t)nvalid << psa_sched::REC_NVALID_SHIFT);
#pragma unroll
    for (int g = 0; g < 4; ++g) r[g] |= hi;
    out[t] = r;
    if (t == T - 1) {
#pragma unroll
      for (int e = 1; e <= psa_sched::REC_PAD; ++e) out[t + e] = r;
    }
  }
}

}  // namespace

// dealing of the rows of the forward walk: shared by psa_build_schedule and the forward launch
void psa_fwd_deal(int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, bool has_map, bool pairs, int& chunk, int& groups) {
  const int Mq = (L + block_m - 1) / block_m, Nk = (L + block_n - 1) / block_n;
  const int64_t total = (int64_t)B * Hq * Mq;
  const double kv_bytes = 2.0 * B * Hkv * ((double)Nk * block_n) * D * 2.0 * (has_map ? 1.875 : 1.0);
  psa_order::deal(total, kv_bytes, B * Hkv, chunk, groups);
  if (pairs) chunk = (chunk + 1) & ~1;  // pairs of rows never straddle two shares
}

bool psa_schedule_shape_ok(int D, int block_m, int block_n, int L) {
  return (D == 128 || D == 64) && block_m == 128 && block_n == 128 && (int64_t)((L + 127) / 128) * 128 <= (1 << psa_sched::REC_SRC_BITS);
}

bool psa_schedule_geometry(int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, psa_sched::Geometry& g) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || L <= 0 || Hq % Hkv != 0 || !psa_schedule_shape_ok(D, block_m, block_n, L)) return false;
  if (B >= 65536 || Hq >= 65536) return false;
  g.Mq = (L + block_m - 1) / block_m;
  g.Nk = (L + block_n - 1) / block_n;
  g.rows = (int64_t)B * Hq * g.Mq;
  if (g.rows >= (1ll << 28)) return false;
  psa_fwd_deal(B, Hq, Hkv, L, D, block_m, block_n, true, true, g.wg_chunk, g.wg_groups);
  g.lay = psa_sched::layout(g.rows, g.Nk, (int64_t)g.wg_chunk * g.wg_groups);
  return true;
}

extern "C" int64_t psa_schedule_bytes(int B, int Hq, int Hkv, int L, int D, int block_m, int block_n) {
  psa_sched::Geometry g;
  return psa_schedule_geometry(B, Hq, Hkv, L, D, block_m, block_n, g) ? g.lay.bytes : 0;
}

extern "C" int psa_build_schedule(const void* map, int map_elem_bytes, void* schedule, int B, int Hq, int Hkv, int L, int D,
                                  int block_m, int block_n, int causal, psa_stream_t stream) {
  PSA_REQUIRE(map != nullptr && schedule != nullptr, PSA_ERR_ARG, "psa_build_schedule: null pointer");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_build_schedule: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && L > 0 && Hq % Hkv == 0, PSA_ERR_ARG, "psa_build_schedule: bad B / H / L");
  PSA_REQUIRE(psa_schedule_shape_ok(D, block_m, block_n, L), PSA_ERR_UNSUPPORTED,
              "psa_build_schedule: schedules exist for D = 64 or 128, block_m = block_n = 128 (got D=%d, block_m=%d, block_n=%d)", D, block_m, block_n);
  PSA_REQUIRE((uintptr_t)schedule % 16 == 0, PSA_ERR_ARG, "psa_build_schedule: schedule must be 16-byte aligned");
  psa_sched::Geometry g;
  PSA_REQUIRE(psa_schedule_geometry(B, Hq, Hkv, L, D, block_m, block_n, g), PSA_ERR_UNSUPPORTED, "psa_build_schedule: shape out of range");
  PSA_REQUIRE((size_t)ROWS_PER_WG * g.Nk * 2 <= 64 * 1024, PSA_ERR_UNSUPPORTED, "psa_build_schedule: more than 8192 kv-blocks");
  char* base = (char*)schedule;
  hipStream_t s = (hipStream_t)stream;
  int32_t* order = (int32_t*)(base + g.lay.order_off);
  int32_t* cost = (int32_t*)(base + g.lay.cost_off);
  int32_t* tiles = (int32_t*)(base + g.lay.tiles_off);
  u32x4* recs = (u32x4*)(base + g.lay.rec_off);
  hipLaunchKernelGGL(psa_sched_build_kernel, dim3((unsigned)((g.rows + ROWS_PER_WG - 1) / ROWS_PER_WG)), dim3(64 * ROWS_PER_WG),
                     (size_t)ROWS_PER_WG * g.Nk * 2, s, map, map_elem_bytes, (int)g.rows, g.Mq, g.Nk, psa_ilog2(block_n), block_m, L,
                     causal ? 1 : 0, cost, tiles, recs, g.lay.rec_stride);
  if (int e = psa_check_launch("psa_build_schedule (tiles)")) return e;
  hipLaunchKernelGGL(psa_order::psa_chunk_sort_kernel, dim3(g.wg_groups), dim3(256), 0, s, cost, (int)g.rows, g.wg_chunk, order);
  return psa_check_launch("psa_build_schedule (order)");
}
