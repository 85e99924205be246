// Draw of the in-block sampling offsets of the block-importance estimator, on the device, in one launch: per
// (batch, head), `keep` distinct offsets out of `block` - the positions of the `keep` largest of `block` uniform
// random numbers, in decreasing order of the numbers, which is what the reference's rand -> topk gives.  The numbers
// come from a counter-based generator (a 64-bit mix of seed, tensor, head and position), so a draw is reproducible
// from its seed and needs no generator state on the device.  Latency-bound (a few microseconds).
#include "psa_common.h"

namespace {

__device__ __forceinline__ uint64_t mix64(uint64_t x) {  // splitmix64 finaliser
  x += 0x9e3779b97f4a7c15ull;
  x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
  x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
  return x ^ (x >> 31);
}

// one workgroup of `block` threads (<= 128) per (tensor, batch * head)
__global__ __launch_bounds__(128) void psa_draw_offsets_kernel(int32_t* off_q, int32_t* off_k, int bh_q, int block_m, int keep_m,
                                                             int block_n, int keep_n, uint64_t seed) {
  __shared__ uint64_t s_key[128];
  const bool is_k = (int)blockIdx.x >= bh_q;
  const int bh = is_k ? (int)blockIdx.x - bh_q : (int)blockIdx.x;
  const int block = is_k ? block_n : block_m, keep = is_k ? keep_n : keep_m;
  int32_t* out = (is_k ? off_k : off_q) + (int64_t)bh * keep;
  const int i = threadIdx.x;
  // 64-bit key: random number above, position below (keys are distinct, so the ranking is a strict order)
  const uint64_t r = mix64(mix64(seed ^ (is_k ? 0x6b6b6b6bull : 0x71717171ull)) + ((uint64_t)bh << 20) + (uint64_t)i);
  const uint64_t key = (r & ~(uint64_t)0xff) | (uint64_t)i;
  if (i < block) s_key[i] = key;
  __syncthreads();
  if (i < block) {
    int rank = 0;
    for (int j = 0; j < block; ++j) rank += s_key[j] > key ? 1 : 0;
    if (rank < keep) out[rank] = i;
  }
}

}  // namespace

extern "C" int psa_draw_sample_offsets(int32_t* off_q, int32_t* off_k, int bh_q, int bh_kv, int block_m, int keep_m, int block_n,
                                       int keep_n, uint64_t seed, psa_stream_t stream) {
  PSA_REQUIRE(off_q != nullptr && off_k != nullptr, PSA_ERR_ARG, "psa_draw_sample_offsets: null pointer");
  PSA_REQUIRE(bh_q > 0 && bh_kv > 0, PSA_ERR_ARG, "psa_draw_sample_offsets: B * H must be positive");
  PSA_REQUIRE(block_m > 0 && block_m <= 128 && block_n > 0 && block_n <= 128, PSA_ERR_UNSUPPORTED,
              "psa_draw_sample_offsets: blocks of at most 128 tokens");
  PSA_REQUIRE(keep_m > 0 && keep_m <= block_m && keep_n > 0 && keep_n <= block_n, PSA_ERR_ARG,
              "psa_draw_sample_offsets: keep must be in 1 .. block");
  hipLaunchKernelGGL(psa_draw_offsets_kernel, dim3((unsigned)(bh_q + bh_kv)), dim3(128), 0, (hipStream_t)stream, off_q, off_k, bh_q,
                     block_m, keep_m, block_n, keep_n, (uint64_t)seed);
  return psa_check_launch("psa_draw_sample_offsets");
}
