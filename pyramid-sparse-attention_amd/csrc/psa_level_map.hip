// Scores -> pyramid level map (and the index-list format), plus small map utilities.
//
// One workgroup per (b, h, q-block) row.  The row (<= a few thousand fp32 scores) lives in LDS:
//   1. stable descending order by rank counting on a 64-bit key (inverted order-preserving score
//      bits, then column index) - keys are unique so ties resolve to the lower column;
//   2. thresholdbound only: sequential fp64 prefix sums rounded to fp32 (one lane walks the row,
//      which keeps the additions in exactly the order a serial CPU scan uses), r = c / c[last] with
//      an IEEE fp32 division, per-threshold counts of r <= thr;
//   3. integer interval logic per item (alignment of each level's count to ceil(level/align_div));
//   4. scatter of levels to their columns.
// Latency-bound: about 1 KB read and 0.25-1 KB written per row.
#include "psa_level_map_row.h"

__global__ __launch_bounds__(256) void psa_level_map_kernel(LevelMapParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int s_cnt[PSA_MAX_LEVEL_ITEMS];
  __shared__ int s_iv[PSA_MAX_LEVEL_ITEMS][2];
  const int64_t row = blockIdx.x;
  level_map_row(p, p.scores + row * p.Nk, row, smem, s_cnt, s_iv, (int)threadIdx.x, (int)blockDim.x);
}

extern "C" int psa_level_map(const float* scores, void* map_out, int map_elem_bytes, int32_t* list_out, int64_t rows,
                             int Nk, int mode, int n_items, const int32_t* item_level, const double* item_hi,
                             int align_div, int text_blocks, double min_full_attn_ratio, psa_stream_t stream) {
  PSA_REQUIRE(scores && (map_out || list_out), PSA_ERR_ARG, "psa_level_map: null pointer");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_level_map: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(rows > 0 && rows < (1ll << 31), PSA_ERR_UNSUPPORTED, "psa_level_map: rows=%lld out of range", (long long)rows);
  LevelMapParams p;
  const int rc = level_map_fill_params(p, Nk, mode, n_items, item_level, item_hi, align_div, text_blocks, min_full_attn_ratio);
  if (rc != PSA_OK) return rc;
  p.scores = scores; p.map_out = map_out; p.list_out = list_out; p.map_elem = map_elem_bytes;
  size_t shmem = level_map_lds_bytes(Nk);
  if (shmem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)psa_level_map_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    PSA_REQUIRE(e == hipSuccess, PSA_ERR_LAUNCH, "psa_level_map: cannot reserve %zu bytes of LDS", shmem);
  }
  const int nt = Nk >= 256 ? 256 : ((Nk + 63) / 64) * 64;  // one thread per score up to 256: idle waves only take up slots
  hipLaunchKernelGGL(psa_level_map_kernel, dim3((unsigned)rows), dim3(nt), shmem, (hipStream_t)stream, p);
  return psa_check_launch("psa_level_map");
}

// ---------------------------------------------------------------------------------------
// level map of the causal Qwen2.5-VL example: square map, per-row ratio windows, fix-ups
// ---------------------------------------------------------------------------------------
struct QwenMapParams {
  const float* scores;
  void* map_out;
  int map_elem;
  int S;       // blocks per side
  int mode;    // PSA_MODE_TOPK: rank windows on the causal row length; PSA_MODE_THRESHOLDBOUND: cumulative-mass windows
  int n_items;
  int level[PSA_MAX_LEVEL_ITEMS];
  float lo[PSA_MAX_LEVEL_ITEMS];  // energy mode: max(lo, previous hi); rank mode: lo
  float hi[PSA_MAX_LEVEL_ITEMS];
  int special;  // trailing blocks (rows and columns) forced to level 1
  int causal;
};

__global__ __launch_bounds__(256) void psa_level_map_qwen_kernel(QwenMapParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int N = p.S;
  uint64_t* key = (uint64_t*)smem;
  float* sw = (float*)(key + sort_pad(N));
  int* sidx = (int*)(sw + N);
  float* c32 = (float*)(sidx + N);
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t row = blockIdx.x;
  const int i_row = (int)(row % N);
  const float* src = p.scores + row * N;
  sort_row_desc(key, sw, sidx, src, N, tid, nt);
  if (p.mode == PSA_MODE_THRESHOLDBOUND) {
    row_prefix_sums((double*)key, sw, c32, N, tid, nt);
  }
  const float total = p.mode == PSA_MODE_THRESHOLDBOUND ? fmaxf(c32[N - 1], 1e-10f) : 1.f;
  const float valid_len = p.causal ? (float)(i_row + 1) : (float)N;
  for (int pos = tid; pos < N; pos += nt) {
    int lv = 0;
    if (p.mode == PSA_MODE_THRESHOLDBOUND) {
      const float r = c32[pos] / total;
      for (int t = 0; t < p.n_items; ++t)
        if (r > p.lo[t] && r <= p.hi[t]) lv = p.level[t];
    } else {
      for (int t = 0; t < p.n_items; ++t) {
        int s0 = (int)(valid_len * p.lo[t]), e0 = (int)(valid_len * p.hi[t]);
        s0 = s0 < N ? s0 : N;
        e0 = e0 < N ? e0 : N;
        if (pos >= s0 && pos < e0) lv = p.level[t];
      }
    }
    const int col = sidx[pos];
    if (col >= N - p.special || i_row >= N - p.special) lv = 1;
    if (p.causal && col > i_row) lv = 0;
    if (col == i_row || col == 0) lv = 1;
    store_map(p.map_out, row * N + col, p.map_elem, lv);
  }
}

extern "C" int psa_level_map_qwen(const float* scores, void* map_out, int map_elem_bytes, int64_t bh, int S, int mode,
                                  int n_items, const int32_t* item_level, const double* item_lo, const double* item_hi,
                                  int special_blocks, int causal, psa_stream_t stream) {
  PSA_REQUIRE(scores && map_out && item_level && item_lo && item_hi, PSA_ERR_ARG, "psa_level_map_qwen: null pointer");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_level_map_qwen: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(mode == PSA_MODE_TOPK || mode == PSA_MODE_THRESHOLDBOUND, PSA_ERR_ARG, "mode must be 'topk' or 'energybound'");
  PSA_REQUIRE(n_items >= 1 && n_items <= PSA_MAX_LEVEL_ITEMS, PSA_ERR_ARG, "mask_ratios must not be empty (1..%d items)", PSA_MAX_LEVEL_ITEMS);
  PSA_REQUIRE(bh > 0 && S > 0 && S <= 6144 && bh * S < (1ll << 31), PSA_ERR_UNSUPPORTED, "psa_level_map_qwen: sizes out of range");
  QwenMapParams p;
  p.scores = scores; p.map_out = map_out; p.map_elem = map_elem_bytes; p.S = S; p.mode = mode; p.n_items = n_items;
  p.special = special_blocks < 0 ? 0 : (special_blocks > S ? S : special_blocks);
  p.causal = causal ? 1 : 0;
  double prev_hi = 0.0;
  for (int t = 0; t < PSA_MAX_LEVEL_ITEMS; ++t) {
    p.level[t] = 0; p.lo[t] = 0.f; p.hi[t] = 0.f;
  }
  for (int t = 0; t < n_items; ++t) {
    const int lv = item_level[t];
    PSA_REQUIRE(lv == 0 || lv == 1 || lv == 2 || lv == 4 || lv == 8, PSA_ERR_ARG, "psa_level_map_qwen: level %d not in {0,1,2,4,8}", lv);
    p.level[t] = lv;
    if (mode == PSA_MODE_THRESHOLDBOUND) {
      const double lower = item_lo[t] > prev_hi ? item_lo[t] : prev_hi;
      prev_hi = item_hi[t];
      p.lo[t] = (float)lower;
    } else {
      p.lo[t] = (float)item_lo[t];
    }
    p.hi[t] = (float)item_hi[t];
  }
  size_t shmem = (size_t)sort_pad(S) * 8 + (size_t)S * 12;
  if (shmem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)psa_level_map_qwen_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    PSA_REQUIRE(e == hipSuccess, PSA_ERR_LAUNCH, "psa_level_map_qwen: cannot reserve %zu bytes of LDS", shmem);
  }
  const int nt = S >= 256 ? 256 : ((S + 63) / 64) * 64;
  hipLaunchKernelGGL(psa_level_map_qwen_kernel, dim3((unsigned)(bh * S)), dim3(nt), shmem, (hipStream_t)stream, p);
  return psa_check_launch("psa_level_map_qwen");
}

// ---------------------------------------------------------------------------------------
// index list -> dense map
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void psa_map_from_list_kernel(const int32_t* list, void* map, int map_elem, int width, int Nk) {
  __shared__ int s_wave_sep[4];
  const int64_t row = blockIdx.x;
  const int32_t* src = list + row * width;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int j = tid; j < Nk; j += 256) store_map(map, row * Nk + j, map_elem, 0);
  __syncthreads();
  int seps_before = 0;  // separators in columns before the current chunk
  for (int c0 = 0; c0 < width; c0 += 256) {
    const int c = c0 + tid;
    const int v = c < width ? src[c] : 0;
    const bool is_sep = c < width && v == -1;
    const uint64_t bal = __ballot(is_sep);
    if (lane == 0) s_wave_sep[wave] = __popcll(bal);
    __syncthreads();
    int before = seps_before;
    for (int w = 0; w < wave; ++w) before += s_wave_sep[w];
    before += __popcll(bal & ((1ull << lane) - 1ull));
    if (c < width && !is_sep && before <= 3 && v >= 0 && v < Nk) store_map(map, row * Nk + v, map_elem, 1 << before);
    seps_before += s_wave_sep[0] + s_wave_sep[1] + s_wave_sep[2] + s_wave_sep[3];
    __syncthreads();
  }
}

extern "C" int psa_map_from_list(const int32_t* list, void* map_out, int map_elem_bytes, int64_t rows, int width, int Nk,
                                 psa_stream_t stream) {
  PSA_REQUIRE(list && map_out, PSA_ERR_ARG, "psa_map_from_list: null pointer");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_map_from_list: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(rows > 0 && rows < (1ll << 31) && Nk > 0 && width >= Nk, PSA_ERR_ARG, "psa_map_from_list: bad sizes");
  hipLaunchKernelGGL(psa_map_from_list_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, list, map_out,
                     map_elem_bytes, width, Nk);
  return psa_check_launch("psa_map_from_list");
}

// ---------------------------------------------------------------------------------------
// dense map -> index list (five segments: levels 1, 2, 4, 8, then the skipped blocks; -1 after each)
// ---------------------------------------------------------------------------------------
// One wave per row.  Blocks are listed by level, ascending inside a level; a segment's length is rounded down to a
// multiple of ceil(level / align_div) and the blocks that do not fit lead the next segment.
__global__ __launch_bounds__(256) void psa_list_from_map_kernel(const void* map, int map_elem, int32_t* list, int64_t rows, int Nk,
                                                              int align_div) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t mrow = row * Nk;
  int32_t* out = list + row * (Nk + 5);
  // segment of a level value: 1, 2, 4, 8 -> 0..3, anything else (0 = skipped) -> 4
  auto seg_of = [](int lvl) { return lvl == 1 ? 0 : lvl == 2 ? 1 : lvl == 4 ? 2 : lvl == 8 ? 3 : 4; };
  int cnt[5] = {0, 0, 0, 0, 0};
  for (int j0 = 0; j0 < Nk; j0 += 64) {
    const int j = j0 + lane;
    const int sg = j < Nk ? seg_of(load_map(map, mrow + j, map_elem)) : -1;
#pragma unroll
    for (int t = 0; t < 5; ++t) cnt[t] += __popcll(__ballot(sg == t));
  }
  int start[5], bound[5];  // first sorted position of a level; end of a segment after the rounding
  {
    int a = 0;
#pragma unroll
    for (int t = 0; t < 5; ++t) {
      start[t] = a;
      a += cnt[t];
    }
    int carry = 0, b = 0;
#pragma unroll
    for (int t = 0; t < 5; ++t) {
      int len = cnt[t] + carry;
      carry = 0;
      if (t < 4) {
        const int mult = ((1 << t) + align_div - 1) / align_div;
        carry = mult > 1 ? len % mult : 0;
        len -= carry;
      }
      b += len;
      bound[t] = b;
    }
  }
  if (lane < 5) out[bound[lane] + lane] = -1;  // the separator behind segment `lane`
  int run[5] = {start[0], start[1], start[2], start[3], start[4]};
  const uint64_t lt_mask = (1ull << lane) - 1ull;
  for (int j0 = 0; j0 < Nk; j0 += 64) {
    const int j = j0 + lane;
    const int sg = j < Nk ? seg_of(load_map(map, mrow + j, map_elem)) : -1;
#pragma unroll
    for (int t = 0; t < 5; ++t) {
      const uint64_t bal = __ballot(sg == t);
      if (sg == t) {
        const int pos = run[t] + __popcll(bal & lt_mask);  // position in the list sorted by level
        const int seps = (pos >= bound[0]) + (pos >= bound[1]) + (pos >= bound[2]) + (pos >= bound[3]) + (pos >= bound[4]);
        out[pos + seps] = j;
      }
      run[t] += __popcll(bal);
    }
  }
}

extern "C" int psa_list_from_map(const void* map, int map_elem_bytes, int32_t* list_out, int64_t rows, int Nk, int align_div,
                                 psa_stream_t stream) {
  PSA_REQUIRE(map && list_out, PSA_ERR_ARG, "psa_list_from_map: null pointer");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_list_from_map: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(rows > 0 && rows < (1ll << 31) && Nk > 0 && align_div >= 1, PSA_ERR_ARG, "psa_list_from_map: bad sizes");
  hipLaunchKernelGGL(psa_list_from_map_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream, map,
                     map_elem_bytes, list_out, rows, Nk, align_div);
  return psa_check_launch("psa_list_from_map");
}

// ---------------------------------------------------------------------------------------
// map = min(map, cap[bh, col])
// ---------------------------------------------------------------------------------------
__global__ void psa_map_min_cap_kernel(void* map, int map_elem, const int32_t* cap, int Mq, int Nk) {
  const int64_t bh = blockIdx.y;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)Mq * Nk) return;
  const int col = (int)(i % Nk);
  const int64_t idx = bh * Mq * Nk + i;
  const int m = load_map(map, idx, map_elem);
  const int c = cap[bh * Nk + col];
  if (c < m) store_map(map, idx, map_elem, c);
}

extern "C" int psa_map_min_cap(void* map, int map_elem_bytes, const int32_t* cap, int64_t bh, int Mq, int Nk,
                               psa_stream_t stream) {
  PSA_REQUIRE(map && cap, PSA_ERR_ARG, "psa_map_min_cap: null pointer");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_map_min_cap: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(bh > 0 && bh <= 65535 && Mq > 0 && Nk > 0, PSA_ERR_ARG, "psa_map_min_cap: bad sizes");
  int64_t n = (int64_t)Mq * Nk;
  hipLaunchKernelGGL(psa_map_min_cap_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)bh), dim3(256), 0,
                     (hipStream_t)stream, map, map_elem_bytes, cap, Mq, Nk);
  return psa_check_launch("psa_map_min_cap");
}

// ---------------------------------------------------------------------------------------
// density = mean(1/level)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void psa_density_kernel(const void* map, int map_elem, int Mq, int Nk, int causal, int BH,
                                                           float* out) {
  __shared__ float s_part[16];
  const int64_t bh = blockIdx.x;
  const int64_t n = (int64_t)Mq * Nk;
  const int tid = threadIdx.x;
  // counts per level are exact integers; 1/level sums are exact in fp32 up to 2^24/8 blocks
  int c1 = 0, c2 = 0, c4 = 0, c8 = 0;
  auto count = [&](int lv, int64_t idx) {
    if (causal) {
      const int64_t r = idx / Nk, c = idx - r * Nk;
      if (c > r) return;
    }
    c1 += lv == 1; c2 += lv == 2; c4 += lv == 4; c8 += lv == 8;
  };
  const unsigned char* base = (const unsigned char*)map + bh * n * map_elem;
  const int epu = 16 / map_elem;  // map entries per 16-byte load
  const int64_t units = (((uintptr_t)base & 15) == 0) ? n / epu : 0;
  for (int64_t u = tid; u < units; u += 1024) {
    const u32x4 w = *(const u32x4*)(base + u * 16);
    if (map_elem == 1) {
#pragma unroll
      for (int e = 0; e < 16; ++e) count((int)(signed char)((w[e >> 2] >> ((e & 3) * 8)) & 0xff), u * 16 + e);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) count((int)w[e], u * 4 + e);
    }
  }
  for (int64_t idx = units * epu + tid; idx < n; idx += 1024) count(load_map(map, bh * n + idx, map_elem), idx);
  float v = (float)c1 + 0.5f * (float)c2 + 0.25f * (float)c4 + 0.125f * (float)c8;
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  if ((tid & 63) == 0) s_part[tid >> 6] = v;
  __syncthreads();
  if (tid == 0) {
    float tot = 0.f;
    for (int w = 0; w < 16; ++w) tot += s_part[w];  // exact: multiples of 1/8 below 2^21
    const double cnt = causal ? ((double)(Mq < Nk ? Mq : Nk) * ((Mq < Nk ? Mq : Nk) + 1) / 2.0 +
                                 (Mq > Nk ? (double)(Mq - Nk) * Nk : 0.0))
                              : (double)n;
    const float d = (float)((double)tot / cnt);
    out[bh] = d;
  }
}

// overall mean in a fixed order (deterministic)
__global__ void psa_density_mean_kernel(float* out, int BH) {
  double acc = 0.0;
  for (int i = 0; i < BH; ++i) acc += (double)out[i];
  out[BH] = (float)(acc / (double)BH);
}

extern "C" int psa_density(const void* map, int map_elem_bytes, int64_t bh, int Mq, int Nk, int causal, float* density_out,
                           psa_stream_t stream) {
  PSA_REQUIRE(map && density_out, PSA_ERR_ARG, "psa_density: null pointer");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_density: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(bh > 0 && bh < (1 << 30) && Mq > 0 && Nk > 0, PSA_ERR_ARG, "psa_density: bad sizes");
  hipLaunchKernelGGL(psa_density_kernel, dim3((unsigned)bh), dim3(1024), 0, (hipStream_t)stream, map, map_elem_bytes, Mq,
                     Nk, causal, (int)bh, density_out);
  hipLaunchKernelGGL(psa_density_mean_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, density_out, (int)bh);
  return psa_check_launch("psa_density");
}
