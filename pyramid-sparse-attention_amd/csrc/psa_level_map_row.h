// One row of scores -> pyramid levels: the device code shared by the level-map kernel and the fused estimator
// epilogue, and the host-side parameter set-up.  See psa_level_map.hip for the algorithm.
#pragma once
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

// One row of the level map.  `src` = the row's N scores (global memory or LDS), `smem` = level_map_lds_bytes(N) bytes
// of 16-byte aligned LDS, s_cnt / s_iv = PSA_MAX_LEVEL_ITEMS (x2) ints of LDS; called by all nt threads of the workgroup.
__device__ __forceinline__ void level_map_row(const LevelMapParams& p, const float* src, int64_t row, unsigned char* smem,
                                              int* s_cnt, int (*s_iv)[2], int tid, int nt) {
  const int N = p.Nk;
  uint64_t* key = (uint64_t*)smem;            // [sort_pad(N)]
  float* sw = (float*)(key + sort_pad(N));    // [N] scores in sorted order
  int* sidx = (int*)(sw + N);                 // [N] column of sorted position
  float* c32 = (float*)(sidx + N);            // [N] prefix sums

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


// Host side: the kernel parameters of a level map with `Nk` columns (everything but the pointers).
static inline int level_map_fill_params(LevelMapParams& p, int Nk, int mode, int n_items, const int32_t* item_level,
                                        const double* item_hi, int align_div, int text_blocks, double min_full_attn_ratio) {
  PSA_REQUIRE(item_level && item_hi, PSA_ERR_ARG, "psa_level_map: mask_ratios must be provided");
  PSA_REQUIRE(mode == PSA_MODE_TOPK || mode == PSA_MODE_THRESHOLDBOUND, PSA_ERR_ARG,
              "Unknown mode: %d. Must be 'topk' or 'thresholdbound'", mode);
  PSA_REQUIRE(n_items >= 1 && n_items <= PSA_MAX_LEVEL_ITEMS, PSA_ERR_ARG, "psa_level_map: 1..%d items", PSA_MAX_LEVEL_ITEMS);
  PSA_REQUIRE(Nk > 0 && Nk <= 6144, PSA_ERR_UNSUPPORTED, "psa_level_map: Nk=%d out of range (Nk <= 6144)", Nk);
  PSA_REQUIRE(align_div >= 1 && text_blocks >= 0, PSA_ERR_ARG, "psa_level_map: bad align_div/text_blocks");
  p.scores = nullptr; p.map_out = nullptr; p.list_out = nullptr; p.map_elem = 4;
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
  return PSA_OK;
}

static inline size_t level_map_lds_bytes(int Nk) { return (size_t)sort_pad(Nk) * 8 + (size_t)Nk * (4 + 4 + 4); }
