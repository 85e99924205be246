/*
 * psa_hip.h - C ABI of libpsa_hip.so: Pyramid Sparse Attention kernels for AMD MI355X (gfx950).
 *
 * The reference (ziplab/Pyramid-Sparse-Attention) has no FFI: its boundary is a set of Python
 * callables that launch Triton kernels.  Each entry point below replaces one of those
 * callables (cited as reference file:line); the Python package psa_hip binds them with ctypes
 * and re-exposes the reference's names and signatures.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller (the small item_* configuration arrays of
 *     psa_level_map are the one exception: they are read on the host); nothing is allocated or freed here;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*), no host synchronisation;
 *   - return value 0 = ok, negative = error (see PSA_ERR_*); psa_last_error() gives a
 *     thread-local human-readable message for the last failing call on this thread;
 *   - activations are bf16, fp16 or fp32 (psa_tensor4.dtype; see PSA_DTYPE_* for which entry points take which),
 *     [B, H, L, D] with the D axis contiguous; batch/head/row strides are given in elements (psa_tensor4), so
 *     transposed [B, L, H, D] views need no copy;
 *   - D in {64, 128}; block_m in {64, 128}; block_n in {32, 64, 128};
 *   - level maps hold one of {0, 1, 2, 4, 8} per (q-block, kv-block): 0 = skip, l = attend to the
 *     kv-block's keys mean-pooled by l.  `map_elem_bytes` is 1 (int8) or 4 (int32, the reference's
 *     dtype), layout [B, Hq, Mq, Nk] contiguous, Mq = ceil(L/block_m), Nk = ceil(L/block_n).
 */
#ifndef PSA_HIP_H
#define PSA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PSA_OK 0
#define PSA_ERR_ARG (-1)         /* null pointer, bad enum, bad size */
#define PSA_ERR_UNSUPPORTED (-2) /* shape outside what the kernels are built for */
#define PSA_ERR_LAUNCH (-3)      /* hip reported a launch error */

#define PSA_MODE_TOPK 0
#define PSA_MODE_THRESHOLDBOUND 1
#define PSA_MAX_LEVEL_ITEMS 8

typedef void* psa_stream_t; /* hipStream_t */

/* Element types.  The kernels compute in the type of their tensors, as the reference's do (tl.dot on q / k as loaded,
 * p.to(v.dtype): reference src/psa_triton/kernels/psa_kernel.py:49-77): bf16 and fp16 operands on the matrix cores with
 * fp32 accumulation, fp32 tensors in fp32 throughout.  All tensors of one call (and its pooled buffers) share one
 * type.  bf16 and fp16: every entry point that takes tensors, except psa_estimate_xattn (bf16 only).  fp32: psa_pool_kv*,
 * psa_estimate_sampled* and the psa_fwd* family (vector-unit kernels; psa_build_schedule / psa_fwd_scheduled are for the
 * 16-bit types); psa_bwd, psa_ksim and psa_estimate_xattn return PSA_ERR_UNSUPPORTED for fp32 tensors. */
#define PSA_DTYPE_BF16 0
#define PSA_DTYPE_F16 1
#define PSA_DTYPE_F32 2

/* [B, H, L, D] view; strides in elements; the D stride is 1.  dtype: PSA_DTYPE_* (0 = bf16). */
typedef struct psa_tensor4 {
  void* ptr;
  int64_t stride_b;
  int64_t stride_h;
  int64_t stride_l;
  int32_t dtype;
  int32_t reserved;
} psa_tensor4;

int psa_version(void);
const char* psa_last_error(void);

/* Number of elements (of the tensors' type) of one pooled buffer (levels 2, 4, 8 back to back):
 * B*Hkv*Npad*D*7/8 with Npad = ceil(L/block_n)*block_n.  Level l starts at element
 * psa_pool_level_offset(...) and is a contiguous [B, Hkv, Npad/l, D]. */
int64_t psa_pool_elems(int B, int Hkv, int L, int D, int block_n);
int64_t psa_pool_level_offset(int B, int Hkv, int L, int D, int block_n, int level);

/* Pyramid pooling of K and V: one pass that reads K, V once and writes the 2x, 4x, 8x mean-pooled
 * levels (each level rounded to the tensors' type before the next, tail replicate-padded to block_n).
 * Replaces pad_to_multiple + pooling x3 per tensor:
 *   reference src/psa_triton/kernels/psa_kernel.py:318-349,381-388
 *   (same code at src/psa_triton/kernels/psa_kernel_legacy.py:806-834,868-875). */
int psa_pool_kv(psa_tensor4 k, psa_tensor4 v, void* k_pool, void* v_pool,
                int B, int Hkv, int L, int D, int block_n, psa_stream_t stream);

/* Bytes of scratch psa_estimate_sampled needs (the per-row key-group maxima in fp32). */
int64_t psa_estimate_workspace_bytes(int B, int Hq, int Lq, int Lk, int block_m, int block_n,
                                     int keep_m, int keep_n);

/* Sampled block-importance estimate.  Row r of the sampled Q is source row
 * min((r/keep_m)*block_m + off_q[b,h,r%keep_m], Lq-1) (off_q == NULL: offsets 0..keep_m-1, i.e. the
 * input is already sampled when block_m == keep_m); rows past the last sampled row replicate it up to
 * a multiple of 64, as the reference pads.  Same for K with off_k [B, Hkv, keep_n].
 * scores [B, Hq, out_rows, out_cols] fp32 = rows normalised by the sum over ALL key groups
 * (including the padding groups), cropped to out_rows x out_cols.  `workspace` is caller-allocated
 * device memory of psa_estimate_workspace_bytes(...) bytes; its contents are overwritten.
 * Replaces _random_sample_tokens' gather + attn_with_pooling_optimized:
 *   reference src/psa_triton/attention.py:116-137,178-223,
 *   src/psa_triton/kernels/attn_pooling_kernel.py:12-116,119-282,285-451. */
int psa_estimate_sampled(psa_tensor4 q, psa_tensor4 k, const int32_t* off_q, const int32_t* off_k,
                         float* scores, void* workspace, int B, int Hq, int Hkv, int Lq, int Lk, int D,
                         int block_m, int block_n, int keep_m, int keep_n, float sm_scale,
                         int out_rows, int out_cols, psa_stream_t stream);

/* Draws the estimator's sampling offsets on the device, in one launch: off_q [B*Hq, keep_m] and off_k [B*Hkv, keep_n]
 * int32, per (batch, head) the positions of the keep largest of `block` uniform random numbers in decreasing order of
 * the numbers (distinct offsets in 0 .. block-1; every block of a head uses the same offsets).  The numbers come from a
 * counter-based generator keyed on `seed`: the same seed gives the same offsets, nothing is read from or written to
 * the host.  bh_q = B * Hq, bh_kv = B * Hkv; blocks of at most 128 tokens.
 * Replaces the rand -> topk of _random_sample_tokens: reference src/psa_triton/attention.py:128-133. */
int psa_draw_sample_offsets(int32_t* off_q, int32_t* off_k, int bh_q, int bh_kv, int block_m, int keep_m, int block_n,
                            int keep_n, uint64_t seed, psa_stream_t stream);

/* Scores -> level map.  One row = one (b, h, q-block).  Items are (level, upper bound) in the order
 * the reference walks them: dict order for PSA_MODE_TOPK, ascending upper bound (stable) for
 * PSA_MODE_THRESHOLDBOUND - the caller passes them already in that order.  align_div = block_n/tile_n.
 * Writes map_out [rows, Nk] (map_elem_bytes 1 or 4; may be NULL) and/or list_out [rows, Nk+n_items]
 * int32 (the reference's "new mask type" index list with -1 separators; may be NULL).
 * Sort contract: descending, ties -> lower kv-block index; thresholdbound uses sequential fp64
 * prefix sums rounded to fp32 and compares r <= fp32(hi + 1e-6).
 * Replaces transfer_attn_to_mask: reference src/psa_triton/utils/transfer_attn_to_mask.py:6-507. */
int psa_level_map(const float* scores, void* map_out, int map_elem_bytes, int32_t* list_out,
                  int64_t rows, int Nk, int mode, int n_items, const int32_t* item_level,
                  const double* item_hi, int align_div, int text_blocks, double min_full_attn_ratio,
                  psa_stream_t stream);

/* psa_estimate_sampled followed by psa_level_map (dense map only) in two launches instead of three: the kernel that
 * reduces the estimator's workspace to a row of scores goes on to rank that row while it is still in LDS.  The map
 * [B, Hq, out_rows, out_cols] is the one psa_level_map computes from the scores psa_estimate_sampled returns, bit for
 * bit; `scores` may be NULL when only the map is wanted, except for maps wider than about 5000 columns (the row and
 * the ranking scratch then exceed LDS together and the function runs the two kernels one after the other, which needs
 * the scores buffer: PSA_ERR_ARG without it).  Arguments as in the two functions (Nk = out_cols).
 * Replaces the same reference code as they do (attn_with_pooling_optimized + transfer_attn_to_mask as called from
 * reference src/psa_triton/attention.py:178-235). */
int psa_estimate_sampled_map(psa_tensor4 q, psa_tensor4 k, const int32_t* off_q, const int32_t* off_k,
                             float* scores, void* workspace, int B, int Hq, int Hkv, int Lq, int Lk, int D,
                             int block_m, int block_n, int keep_m, int keep_n, float sm_scale,
                             int out_rows, int out_cols, void* map_out, int map_elem_bytes, int mode, int n_items,
                             const int32_t* item_level, const double* item_hi, int align_div, int text_blocks,
                             double min_full_attn_ratio, psa_stream_t stream);

/* Level map of the causal Qwen2.5-VL example: scores [bh, S, S] fp32 -> map [bh, S, S].  Items (level, lo, hi) in
 * dict order (host arrays).  PSA_MODE_TOPK: sorted positions [floor(len*lo), floor(len*hi)) get the level, len = row+1
 * if causal else S; PSA_MODE_THRESHOLDBOUND ("energybound"): positions whose cumulative ratio r satisfies
 * max(lo, previous hi) < r <= hi.  Then: the last special_blocks rows and columns := 1, the strict upper triangle := 0
 * (causal), the diagonal := 1, column 0 := 1.  r = prefix sum / max(last prefix sum, 1e-10) with the prefix sums
 * accumulated sequentially in fp64 over the sorted row (the reference divides by torch's sum of the unsorted row).
 * Replaces the Qwen transfer_attn_to_mask:
 *   reference qwen2.5-vl-example/src/attention/PSA_casual/PyramidAdaptiveBlockSparseAttn.py:84-168. */
int psa_level_map_qwen(const float* scores, void* map_out, int map_elem_bytes, int64_t bh, int S, int mode,
                       int n_items, const int32_t* item_level, const double* item_lo, const double* item_hi,
                       int special_blocks, int causal, psa_stream_t stream);

/* Bytes of scratch psa_estimate_xattn needs. */
int64_t psa_estimate_xattn_workspace_bytes(int B, int Hq, int Lq, int Lk, int block_size, int stride,
                                           int chunk_size);

/* Antidiagonal ("xattn") block-importance estimate of the causal Qwen2.5-VL path:
 * A[m,n] = sum_{i<stride} q[m*stride + stride-1-i] . k[n*stride + i], logits A / (sqrt(D) * stride), causal n <= m
 * (key-aligned), row softmax over all strided keys, probabilities summed inside (block_size/stride)^2 cells.
 * q, k are zero-padded to a multiple of chunk_size tokens; est [B, Hq, ceil(Lq/block), ceil(Lk/block)] fp32.
 * K has Hkv heads (query head h uses kv head h / (Hq/Hkv)); the logits never reach HBM.
 * Replaces estimate_block_importance's Triton path:
 *   reference qwen2.5-vl-example/src/attention/PSA_casual/utils/block_importance.py:282-562,
 *   qwen2.5-vl-example/src/attention/PSA_casual/kernels/block_importance_kernels.py:6-192,255-323. */
int psa_estimate_xattn(psa_tensor4 q, psa_tensor4 k, float* est, void* workspace, int B, int Hq, int Hkv,
                       int Lq, int Lk, int D, int block_size, int stride, int chunk_size, int causal,
                       psa_stream_t stream);

/* Index list ("new mask type", [rows, width] int32) -> dense level map [rows, Nk], read the way the
 * reference's list-walking kernel reads it: segment level starts at 1, doubles at every -1, stops
 * after 8.  reference src/psa_triton/kernels/psa_kernel.py:207-217. */
int psa_map_from_list(const int32_t* list, void* map_out, int map_elem_bytes, int64_t rows,
                      int width, int Nk, psa_stream_t stream);

/* Dense level map [rows, Nk] -> index list [rows, Nk + 5] int32: the kv-blocks at levels 1, 2, 4, 8 and then the skipped
 * ones, each segment followed by -1 (blocks of a level in ascending order).  A segment's length is rounded down to a
 * multiple of ceil(level / align_div), align_div = blocksize / compute_tile, and the blocks that do not fit lead the next
 * segment (they are pooled one level coarser), as in the reference.
 * Replaces transfer_mask_to_new_type: reference src/psa_triton/utils/transfer_attn_to_mask.py:624-750. */
int psa_list_from_map(const void* map, int map_elem_bytes, int32_t* list_out, int64_t rows, int Nk, int align_div,
                      psa_stream_t stream);

/* Key-similarity cap: cap_out [B, H, Nk] int32 in {1, 2, 4, 8}.  For a kv-block, sim_l = mean cosine
 * similarity of the token pairs (g*l, g*l + l-1); the cap is the largest l in {2, 4, 8} with
 * sim_l > thr_l (strictly), else 1.  cos = a.b / (sqrt(|a|^2 + 1e-12) sqrt(|b|^2 + 1e-12) + 1e-6), fp32;
 * tokens past L replicate token L-1.
 * Replaces calc_k_similarity_triton: reference src/psa_triton/kernels/calc_ksim_kernel.py:6-157,160-225. */
int psa_ksim(psa_tensor4 k, int32_t* cap_out, int B, int H, int L, int D, int block_n,
             float thr2, float thr4, float thr8, psa_stream_t stream);

/* out[i] = min(map[i], cap[col]) with cap [B*Hkv... given per (b, h, kv-block)] broadcast over q-blocks:
 * the "sim mask" clamp.  reference src/psa_triton/attention.py:296-299. */
int psa_map_min_cap(void* map, int map_elem_bytes, const int32_t* cap, int64_t bh, int Mq, int Nk,
                    psa_stream_t stream);

/* Token re-ordering: dst[t][b, h, i, :] = src[t][b, h, index[i], :] for i < L_dst, for n_tensors (1..3) tensors
 * that share the index vector (q, k, v in one launch; heads[t] heads each).  index: int32 [L_dst], values in
 * [0, L_src).  Rows are D elements of elem_bytes (2 or 4) bytes; strides are in elements.
 * Replaces the index_select + cat of GilbertRearranger.rearrange / reversed_rearrange:
 * reference src/psa_triton/utils/rearranger.py:14-132. */
int psa_gather_rows(const psa_tensor4* src, const psa_tensor4* dst, const int* heads, int n_tensors,
                    const int32_t* index, int B, int L_dst, int L_src, int D, int elem_bytes,
                    psa_stream_t stream);

/* Token re-ordering folded into the layer's own kernels (no separate gather pass over Q, K, V and the output).
 * index: int32 [L], a permutation of 0..L-1; position i of the re-ordered sequence is source row index[i].
 *   psa_pool_kv_indexed          pools the re-ordered K, V (the result psa_pool_kv gives on the gathered tensors, bit for
 *                                bit) and also writes the re-ordered rows themselves to k_ord, v_ord [B, Hkv, L, D]: the
 *                                level-1 keys / values the attention kernel reads.
 *   psa_estimate_sampled_indexed, psa_estimate_sampled_map_indexed
 *                                the estimator with q read through the index (k is passed already re-ordered: k_ord).
 *   psa_fwd_indexed              the attention kernel with q read through the index and row i of the result (and of lse)
 *                                written to row index[i] of out: out comes back in the caller's original token order.
 * Together they give exactly what gather -> layer -> inverse gather gives.  Other arguments as in the functions they
 * extend.  Replaces GilbertRearranger.rearrange before and reversed_rearrange after the attention call:
 *   reference src/psa_triton/utils/rearranger.py:14-132 as used at src/psa_triton/pyramid_sparse_attention.py:326-344,386-400. */
int psa_pool_kv_indexed(psa_tensor4 k, psa_tensor4 v, const int32_t* index, psa_tensor4 k_ord, psa_tensor4 v_ord,
                        void* k_pool, void* v_pool, int B, int Hkv, int L, int D, int block_n, psa_stream_t stream);
int psa_estimate_sampled_indexed(psa_tensor4 q, const int32_t* q_index, psa_tensor4 k, const int32_t* off_q,
                                 const int32_t* off_k, float* scores, void* workspace, int B, int Hq, int Hkv, int Lq,
                                 int Lk, int D, int block_m, int block_n, int keep_m, int keep_n, float sm_scale,
                                 int out_rows, int out_cols, psa_stream_t stream);
int psa_estimate_sampled_map_indexed(psa_tensor4 q, const int32_t* q_index, psa_tensor4 k, const int32_t* off_q,
                                     const int32_t* off_k, float* scores, void* workspace, int B, int Hq, int Hkv, int Lq,
                                     int Lk, int D, int block_m, int block_n, int keep_m, int keep_n, float sm_scale,
                                     int out_rows, int out_cols, void* map_out, int map_elem_bytes, int mode, int n_items,
                                     const int32_t* item_level, const double* item_hi, int align_div, int text_blocks,
                                     double min_full_attn_ratio, psa_stream_t stream);
int psa_fwd_indexed(psa_tensor4 q, const int32_t* q_index, psa_tensor4 k, psa_tensor4 v, const void* k_pool,
                    const void* v_pool, const void* map, int map_elem_bytes, psa_tensor4 out, float* lse, int B, int Hq,
                    int Hkv, int L, int D, int block_m, int block_n, float sm_scale, int causal, void* workspace,
                    psa_stream_t stream);

/* mean(1/level) over the map, skipped blocks counting 0; causal != 0 counts lower-triangle pairs only.
 * density_out: one float per (b, h) row of the [BH] vector, plus the overall mean at index BH.
 * reference src/psa_triton/utils/transfer_attn_to_mask.py:510-544. */
int psa_density(const void* map, int map_elem_bytes, int64_t bh, int Mq, int Nk, int causal,
                float* density_out, psa_stream_t stream);

/* Sparse attention forward from a level map.  out [B, Hq, L, D] in the type of q / k / v (bf16, fp16 or fp32); lse (may be NULL)
 * [B, Hq, L] fp32 = natural-log softmax denominator incl. the +ln(level) bias; map == NULL means
 * dense attention (every pair at level 1; k_pool/v_pool may then be NULL).  K/V have Hkv heads,
 * query head h uses kv head h / (Hq/Hkv).  causal != 0: kv-blocks above the diagonal are never
 * visited and a pooled key t of level l is visible to query i iff (t+1)*l-1 <= i.
 * Replaces the kernels behind sparse_attention_factory(...)(q, k, v, mask, sm_scale):
 *   reference src/psa_triton/kernels/psa_kernel.py:24-316,351-457 (list walk, non-causal),
 *   src/psa_triton/kernels/psa_kernel_legacy.py:34-799,837-938 (dense map, causal, L/M rows). */
int psa_fwd(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool,
            const void* map, int map_elem_bytes, psa_tensor4 out, float* lse,
            int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, float sm_scale,
            int causal, void* workspace, psa_stream_t stream);

/* Bytes of the optional psa_fwd workspace.  With it, rows of the level map are issued longest first
 * (per share of the chip), which shortens the tail of the launch when rows retain different numbers of
 * blocks; results are identical with and without it.  workspace == NULL issues rows in natural order.
 * The reference balances load through the Triton launch grid alone
 * (src/psa_triton/kernels/psa_kernel.py:398-431). */
int64_t psa_fwd_workspace_bytes(int B, int Hq, int L, int block_m);

/* Tile schedule of a level map: what the attention kernel walks, built once per map instead of inside every launch
 * that walks it.  Per (batch, head, q-block) row it holds the row's tiles of 64 pooled keys (level, source rows, fill,
 * diagonal / ragged flags: 16 bytes per tile) and the rows' issue order (dealt to the chip's XCDs, longest first, equal
 * rows in index order - the same order in every run).  It is the counterpart of the reference's index list, which is
 * also computed once per map and then walked by the kernel:
 *   reference src/psa_triton/utils/transfer_attn_to_mask.py:271-500 (list built), src/psa_triton/kernels/psa_kernel.py:207-302 (walked).
 * Schedules exist for D = 64 or 128, block_m = block_n = 128 (psa_schedule_bytes returns 0 otherwise and psa_build_schedule
 * PSA_ERR_UNSUPPORTED; psa_fwd covers every shape).  `schedule`: caller-allocated device memory of psa_schedule_bytes(...)
 * bytes, 16-byte aligned (the bound is the worst case, every pair at level 1: 32 bytes per (q-block, kv-block) pair; only
 * the retained tiles are written and read).  It stays valid for as long as the map is unchanged and may be used by any
 * number of psa_fwd_scheduled calls with the same shape arguments. */
int64_t psa_schedule_bytes(int B, int Hq, int Hkv, int L, int D, int block_m, int block_n);
int psa_build_schedule(const void* map, int map_elem_bytes, void* schedule, int B, int Hq, int Hkv, int L, int D,
                       int block_m, int block_n, int causal, psa_stream_t stream);

/* psa_fwd on a prebuilt schedule (same results as psa_fwd on the map the schedule was built from; rows are walked in
 * the same tile order).  q_index may be NULL; otherwise as in psa_fwd_indexed.  `map` is the map the schedule was built
 * from (kept in the signature for the shapes' sake; the kernel reads the schedule).
 * Replaces the same reference code as psa_fwd. */
int psa_fwd_scheduled(psa_tensor4 q, const int32_t* q_index, psa_tensor4 k, psa_tensor4 v, const void* k_pool,
                      const void* v_pool, const void* map, int map_elem_bytes, const void* schedule, psa_tensor4 out,
                      float* lse, int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, float sm_scale,
                      int causal, psa_stream_t stream);

/* psa_fwd without a workspace argument and without any allocation: the row-ordering scratch is a fixed array inside
 * the library (one copy per GPU, about 0.5 MiB, held until the process ends).  This entry point has no counterpart in
 * the reference; it exists for callers that cannot allocate device memory around the call - code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It calls no hipMalloc / hipFree or other allocating
 * routine.  Same arguments, kernels and results (bit for bit) as psa_fwd with a workspace.  Limit: at most
 * psa_fwd_noalloc_max_rows() = 65536 rows of the level map, rows = B * Hq * ceil(L / block_m); larger shapes return
 * PSA_ERR_UNSUPPORTED.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams
 * or threads) race on it and must be serialised by the caller; consecutive calls need no clearing in between. */
int psa_fwd_noalloc(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool,
                    const void* map, int map_elem_bytes, psa_tensor4 out, float* lse,
                    int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, float sm_scale,
                    int causal, psa_stream_t stream);
int64_t psa_fwd_noalloc_max_rows(void);

/* Bytes of workspace psa_bwd needs (fp32 dK/dV per pyramid level, delta, lse in log2 units, cost and issue order of
 * the dQ rows and of the dK/dV workgroups). */
int64_t psa_bwd_workspace_bytes(int B, int Hq, int Hkv, int L, int D, int block_n);

/* Backward of psa_fwd w.r.t. q, k, v (the map carries no gradient).  bf16 or fp16 tensors; dq/dk/dv are views like
 * q/k/v in the same type; workspace is caller-allocated (psa_bwd_workspace_bytes) and is overwritten.
 * Gradients of pooled keys are spread over their constituent tokens (/level) and the part that
 * lands on replicate-pad positions is added to the last real token.
 * Replaces _sparse_attention.backward and its kernels:
 *   reference src/psa_triton/kernels/psa_kernel_legacy.py:948-1069,1072-1234,1237-1320. */
int psa_bwd(psa_tensor4 q, psa_tensor4 k, psa_tensor4 v, const void* k_pool, const void* v_pool,
            const void* map, int map_elem_bytes, psa_tensor4 out, psa_tensor4 dout, const float* lse,
            psa_tensor4 dq, psa_tensor4 dk, psa_tensor4 dv, void* workspace,
            int B, int Hq, int Hkv, int L, int D, int block_m, int block_n, float sm_scale,
            int causal, psa_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PSA_HIP_H */
