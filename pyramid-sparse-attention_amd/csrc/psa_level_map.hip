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
#include "psa_common.h"

struct LevelMapParams {
  const float* scores;
  void* map_out;
  int32_t* list_out;
  int map_elem;
  int Nk;
  int mode;
  int n_items;
  int level[PSA_MAX_LEVEL_ITEMS];
  int align[PSA_MAX_LEVEL_ITEMS];
  float thr[PSA_MAX_LEVEL_ITEMS];     // thresholdbound: fp32(hi + 1e-6)
  int fixed_s[PSA_MAX_LEVEL_ITEMS];   // topk: row-independent intervals
  int fixed_e[PSA_MAX_LEVEL_ITEMS];
  int min_index;                      // thresholdbound: floor for the level-1 interval
  int text_blocks;
};

__device__ __forceinline__ uint32_t desc_key(float s) {
  s += 0.0f;  // -0.0 -> +0.0 so that both zeros tie
  uint32_t u = __builtin_bit_cast(uint32_t, s);
  u ^= (u >> 31) ? 0xffffffffu : 0x80000000u;  // ascending order-preserving
  return ~u;                                   // descending
}

// Stable descending order of one row of scores: sw[i] / sidx[i] = score and column of sorted position i.
// The 64-bit keys (inverted score bits, column) are unique, so every correct sort gives the same order.
// Rows of up to 256 scores are ranked by counting (one pass of N comparisons per score, no barriers inside);
// longer rows (32-key blocks: 1024 scores) are sorted in place by a bitonic network over key[0 .. Npad), Npad the
// next power of two, padded with keys that sort last: N/2 compare-exchanges per stage instead of N comparisons
// per score (1024 scores: 55 stages of 2 exchanges per thread against 4096 comparisons per thread).
constexpr int RANK_SORT_MAX = 256;
__host__ __device__ inline int sort_pad(int N) {
  if (N <= RANK_SORT_MAX) return N;
  int n = 1;
  while (n < N) n <<= 1;
  return n;
}
__device__ __forceinline__ void sort_row_desc(uint64_t* key, float* sw, int* sidx, const float* src, int N, int tid, int nt) {
  const int Npad = sort_pad(N);
  for (int j = tid; j < Npad; j += nt) key[j] = j < N ? (((uint64_t)desc_key(src[j]) << 32) | (uint32_t)j) : ~0ull;
  __syncthreads();
  if (N <= RANK_SORT_MAX) {
    for (int j = tid; j < N; j += nt) {
      const uint64_t kj = key[j];
      int rank = 0;
      for (int i = 0; i < N; ++i) rank += key[i] < kj ? 1 : 0;
      sw[rank] = src[j];
      sidx[rank] = j;
    }
  } else {
    for (int k = 2; k <= Npad; k <<= 1) {
      for (int j = k >> 1; j > 0; j >>= 1) {
        for (int e = tid; e < (Npad >> 1); e += nt) {
          // pair e of this stage: i has bit j clear, its partner is i + j; ascending where bit k of i is clear
          const int i = ((e & ~(j - 1)) << 1) | (e & (j - 1));
          const uint64_t a = key[i], b = key[i + j];
          const bool up = (i & k) == 0;
          if ((a > b) == up) {
            key[i] = b;
            key[i + j] = a;
          }
        }
        __syncthreads();
      }
    }
    for (int i = tid; i < N; i += nt) {
      const int col = (int)(uint32_t)key[i];
      sidx[i] = col;
      sw[i] = src[col];
    }
  }
  __syncthreads();
}

// Prefix sums of the sorted scores, accumulated strictly sequentially in fp64 and rounded to fp32 (the order
// matters for bit-exactness).  All threads widen the scores into `wide` (the sort's key buffer, free by now) and
// round the sums afterwards, so that the dependent chain one lane has to run is a load, an addition and a store
// per two scores; that lane runs it at raised wave priority, because up to seven other waves compete with it for
// every instruction slot of the SIMD and the rest of its workgroup waits for it.
__device__ __forceinline__ void row_prefix_sums(double* wide, const float* sw, float* c32, int N, int tid, int nt) {
  typedef double f64x2 __attribute__((ext_vector_type(2)));
  for (int i = tid; i < N; i += nt) wide[i] = (double)sw[i];
  __syncthreads();
  if (tid == 0) {
    __builtin_amdgcn_s_setprio(3);
    double acc = 0.0;
    int i = 0;
    for (; i + 4 <= N; i += 4) {
      const f64x2 w0 = *(const f64x2*)(wide + i), w1 = *(const f64x2*)(wide + i + 2);
      const double a0 = acc + w0[0];
      const double a1 = a0 + w0[1];
      const double a2 = a1 + w1[0];
      acc = a2 + w1[1];
      *(f64x2*)(wide + i) = f64x2{a0, a1};
      *(f64x2*)(wide + i + 2) = f64x2{a2, acc};
    }
    for (; i < N; ++i) {
      acc += wide[i];
      wide[i] = acc;
    }
    __builtin_amdgcn_s_setprio(0);
  }
  __syncthreads();
  for (int i = tid; i < N; i += nt) c32[i] = (float)wide[i];
  __syncthreads();
}

__global__ __launch_bounds__(256) void psa_level_map_kernel(LevelMapParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int N = p.Nk;
  uint64_t* key = (uint64_t*)smem;            // [sort_pad(N)]
  float* sw = (float*)(key + sort_pad(N));    // [N] scores in sorted order
  int* sidx = (int*)(sw + N);                 // [N] column of sorted position
  float* c32 = (float*)(sidx + N);            // [N] prefix sums
  __shared__ int s_cnt[PSA_MAX_LEVEL_ITEMS];
  __shared__ int s_iv[PSA_MAX_LEVEL_ITEMS][2];

  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t row = blockIdx.x;
  const float* src = p.scores + row * N;

  if (tid < PSA_MAX_LEVEL_ITEMS) s_cnt[tid] = 0;
  sort_row_desc(key, sw, sidx, src, N, tid, nt);

  if (p.mode == PSA_MODE_THRESHOLDBOUND) {
    row_prefix_sums((double*)key, sw, c32, N, tid, nt);
    const float total = c32[N - 1];
    // positions whose cumulative ratio is within each item's bound: one ballot per item and pass, one LDS
    // atomic per wave and item (integer counts: the order of the additions does not matter)
    int local[PSA_MAX_LEVEL_ITEMS];
#pragma unroll
    for (int t = 0; t < PSA_MAX_LEVEL_ITEMS; ++t) local[t] = 0;
    for (int i0 = 0; i0 < N; i0 += nt) {
      const int i = i0 + tid;
      const float r = i < N ? c32[i] / total : 0.f;
#pragma unroll
      for (int t = 0; t < PSA_MAX_LEVEL_ITEMS; ++t)
        if (t < p.n_items) local[t] += __popcll(__ballot(i < N && r <= p.thr[t]));
    }
    if ((tid & 63) == 0) {
#pragma unroll
      for (int t = 0; t < PSA_MAX_LEVEL_ITEMS; ++t)
        if (t < p.n_items && local[t]) atomicAdd(&s_cnt[t], local[t]);
    }
    __syncthreads();
    if (tid == 0) {
      // a short dependent chain in one lane while the workgroup waits: raised priority, and no integer
      // division for the usual power-of-two alignments
      __builtin_amdgcn_s_setprio(3);
      int last = 0;
      for (int t = 0; t < p.n_items; ++t) {
        const int cnt = s_cnt[t];
        const int end0 = cnt > 0 ? cnt + 1 : last;
        const int start = last;
        const int al = p.align[t];
        int end;
        if (al > 1) {
          int len = end0 - start;
          len = len > 0 ? len : 0;
          const bool pow2 = (al & (al - 1)) == 0;
          const int rem = pow2 ? (len & (al - 1)) : len % al;
          if (rem) len += al - rem;
          end = start + len;
          end = end < N ? end : N;
          if (end == N) end = start + (pow2 ? ((end - start) & ~(al - 1)) : ((end - start) / al) * al);
        } else {
          end = end0 < 0 ? 0 : (end0 > N ? N : end0);
          end = end > start ? end : start;
          if (p.level[t] == 1) end = end > p.min_index ? end : p.min_index;
        }
        s_iv[t][0] = start;
        s_iv[t][1] = end;
        last = end;
      }
      __builtin_amdgcn_s_setprio(0);
    }
  } else {
    if (tid < p.n_items) {
      s_iv[tid][0] = p.fixed_s[tid];
      s_iv[tid][1] = p.fixed_e[tid];
    }
  }
  __syncthreads();

  if (p.map_out) {
    for (int i = tid; i < N; i += nt) {
      int lv = 0;
      for (int t = 0; t < p.n_items; ++t)
        if (i >= s_iv[t][0] && i < s_iv[t][1]) lv = p.level[t];
      const int col = sidx[i];
      if (col >= N - p.text_blocks) lv = 1;
      store_map(p.map_out, row * N + col, p.map_elem, lv);
    }
  }
  if (p.list_out) {
    const int W = N + p.n_items;
    int32_t* dst = p.list_out + row * W;
    for (int cidx = tid; cidx < W; cidx += nt) {
      int v = 0;
      for (int t = 0; t < p.n_items; ++t) {
        const int pos = cidx - t;  // sorted position if this column belongs to segment t
        if (pos >= s_iv[t][0] && pos < s_iv[t][1]) v = sidx[pos];
        int sep = s_iv[t][1] + t;
        sep = sep > W - 1 ? W - 1 : sep;
        if (cidx == sep) v = -1;   // a separator written for item t survives later items' segments
      }
      dst[cidx] = v;
    }
  }
}

extern "C" int psa_level_map(const float* scores, void* map_out, int map_elem_bytes, int32_t* list_out, int64_t rows,
                             int Nk, int mode, int n_items, const int32_t* item_level, const double* item_hi,
                             int align_div, int text_blocks, double min_full_attn_ratio, psa_stream_t stream) {
  PSA_REQUIRE(scores && (map_out || list_out), PSA_ERR_ARG, "psa_level_map: null pointer");
  PSA_REQUIRE(item_level && item_hi, PSA_ERR_ARG, "psa_level_map: mask_ratios must be provided");
  PSA_REQUIRE(map_elem_bytes == 1 || map_elem_bytes == 4, PSA_ERR_ARG, "psa_level_map: map_elem_bytes must be 1 or 4");
  PSA_REQUIRE(mode == PSA_MODE_TOPK || mode == PSA_MODE_THRESHOLDBOUND, PSA_ERR_ARG,
              "Unknown mode: %d. Must be 'topk' or 'thresholdbound'", mode);
  PSA_REQUIRE(n_items >= 1 && n_items <= PSA_MAX_LEVEL_ITEMS, PSA_ERR_ARG, "psa_level_map: 1..%d items", PSA_MAX_LEVEL_ITEMS);
  PSA_REQUIRE(rows > 0 && rows < (1ll << 31) && Nk > 0 && Nk <= 6144, PSA_ERR_UNSUPPORTED,
              "psa_level_map: rows=%lld Nk=%d out of range (Nk <= 6144)", (long long)rows, Nk);
  PSA_REQUIRE(align_div >= 1 && text_blocks >= 0, PSA_ERR_ARG, "psa_level_map: bad align_div/text_blocks");
  LevelMapParams p;
  p.scores = scores; p.map_out = map_out; p.list_out = list_out; p.map_elem = map_elem_bytes;
  p.Nk = Nk; p.mode = mode; p.n_items = n_items;
  p.text_blocks = text_blocks > Nk ? Nk : text_blocks;
  int m = (int)((double)Nk * min_full_attn_ratio) + 1;
  p.min_index = m < Nk ? m : Nk;
  int last_end = 0;
  for (int t = 0; t < PSA_MAX_LEVEL_ITEMS; ++t) {
    p.level[t] = 0; p.align[t] = 1; p.thr[t] = 0.f; p.fixed_s[t] = 0; p.fixed_e[t] = 0;
  }
  for (int t = 0; t < n_items; ++t) {
    const int lv = item_level[t];
    PSA_REQUIRE(lv == 0 || lv == 1 || lv == 2 || lv == 4 || lv == 8, PSA_ERR_ARG, "psa_level_map: level %d not in {0,1,2,4,8}", lv);
    p.level[t] = lv;
    const int al = (lv + align_div - 1) / align_div;  // ceil(level / (block_n / tile_n)); 0 for the skip level
    if (mode == PSA_MODE_THRESHOLDBOUND) {
      p.align[t] = al;
      p.thr[t] = (float)(item_hi[t] + 1e-6);
    } else {
      const int a = lv == 0 ? 1 : al;
      const int start = last_end;
      int end0 = (int)((double)Nk * item_hi[t]);
      end0 = end0 < Nk ? end0 : Nk;
      int end;
      const int len = end0 - start;
      if (a > 1 && len > 0) {
        const int rem = len % a;
        const int alen = rem ? len + (a - rem) : len;
        end = start + alen < Nk ? start + alen : Nk;
        if (end == Nk) end = start + ((end - start) / a) * a;
      } else {
        end = end0;
      }
      if (start < end) {
        p.fixed_s[t] = start; p.fixed_e[t] = end; last_end = end;
      } else {
        p.fixed_s[t] = start; p.fixed_e[t] = start;
      }
    }
  }
  size_t shmem = (size_t)sort_pad(Nk) * 8 + (size_t)Nk * (4 + 4 + 4);
  if (shmem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)psa_level_map_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    PSA_REQUIRE(e == hipSuccess, PSA_ERR_LAUNCH, "psa_level_map: cannot reserve %zu bytes of LDS", shmem);
  }
  int nt = Nk <= 64 ? 64 : (Nk <= 128 ? 128 : 256);
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
  const int nt = S <= 64 ? 64 : (S <= 128 ? 128 : 256);
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
