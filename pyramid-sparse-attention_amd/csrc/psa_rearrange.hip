// Token re-ordering (Hilbert-curve "Gilbert" order and back): dst[b, h, i, :] = src[b, h, index[i], :].
//
// HBM-bound row gather.  A row is D elements of 2 or 4 bytes (128 - 512 bytes); LPR = row bytes / 16 lanes move
// one row with 16-byte loads and stores, a wave 64 / LPR rows at a time, so every row is read and written as one
// contiguous run.  Up to three tensors (q, k, v) share the index vector and go in one launch (grid z).
// Algorithmic bytes: 2 * B * H * L * row bytes per tensor.
#include "psa_common.h"

namespace {

struct GatherParams {
  const char* src[3];
  char* dst[3];
  int64_t s_sb[3], s_sh[3], s_sl[3], d_sb[3], d_sh[3], d_sl[3];  // strides in bytes
  int H[3], BH[3];
  const int32_t* index;
  int L, L_src, row_bytes;
};

__global__ __launch_bounds__(256) void psa_gather_rows_kernel(GatherParams p) {
  const int z = blockIdx.z;
  const int bh = blockIdx.y;
  const int H = p.H[z];
  if (bh >= p.BH[z]) return;  // a tensor with fewer heads than the largest one of the launch
  const int b = bh / H, h = bh % H;
  const int lpr = p.row_bytes >> 4;             // lanes per row
  const int rows_per_wg = 256 / lpr;
  const int r = threadIdx.x / lpr, c = threadIdx.x % lpr;
  const char* src = p.src[z] + b * p.s_sb[z] + h * p.s_sh[z] + c * 16;
  char* dst = p.dst[z] + b * p.d_sb[z] + h * p.d_sh[z] + c * 16;
  // 4 rows per thread and step: the loads of a step are in flight together
  for (int i0 = blockIdx.x * rows_per_wg * 4; i0 < p.L; i0 += gridDim.x * rows_per_wg * 4) {
    u32x4 w[4];
    int idx[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * rows_per_wg + r;
      int s = i < p.L ? p.index[i] : 0;
      s = s < 0 ? 0 : (s < p.L_src ? s : p.L_src - 1);  // indices are validated on the host; never read out of bounds
      idx[u] = s;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) w[u] = *(const u32x4*)(src + (int64_t)idx[u] * p.s_sl[z]);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * rows_per_wg + r;
      if (i < p.L) __builtin_nontemporal_store(w[u], (u32x4*)(dst + (int64_t)i * p.d_sl[z]));  // streaming: written once, read by later kernels
    }
  }
}

}  // namespace

extern "C" int psa_gather_rows(const psa_tensor4* src, const psa_tensor4* dst, const int* heads, int n_tensors,
                               const int32_t* index, int B, int L_dst, int L_src, int D, int elem_bytes,
                               psa_stream_t stream) {
  PSA_REQUIRE(src && dst && heads && index, PSA_ERR_ARG, "psa_gather_rows: null pointer");
  PSA_REQUIRE(n_tensors >= 1 && n_tensors <= 3, PSA_ERR_ARG, "psa_gather_rows: 1 to 3 tensors per call");
  PSA_REQUIRE(B > 0 && L_dst > 0 && L_src > 0 && D > 0, PSA_ERR_ARG, "psa_gather_rows: sizes must be positive");
  PSA_REQUIRE(elem_bytes == 2 || elem_bytes == 4, PSA_ERR_UNSUPPORTED, "psa_gather_rows: element size %d not in {2, 4}", elem_bytes);
  const int row_bytes = D * elem_bytes;
  PSA_REQUIRE(row_bytes % 16 == 0 && row_bytes <= 4096 && 256 % (row_bytes / 16) == 0, PSA_ERR_UNSUPPORTED,
              "psa_gather_rows: rows of %d bytes (a power-of-two multiple of 16 up to 4096 is needed)", row_bytes);
  GatherParams p;
  int maxH = 0;
  for (int z = 0; z < 3; ++z) {
    const int zz = z < n_tensors ? z : 0;
    PSA_REQUIRE(src[zz].ptr && dst[zz].ptr && heads[zz] > 0, PSA_ERR_ARG, "psa_gather_rows: null tensor or no heads");
    PSA_REQUIRE((uintptr_t)src[zz].ptr % 16 == 0 && (uintptr_t)dst[zz].ptr % 16 == 0, PSA_ERR_UNSUPPORTED,
                "psa_gather_rows: tensors must be 16-byte aligned");
    const int64_t sm = 16 / elem_bytes;
    PSA_REQUIRE(src[zz].stride_b % sm == 0 && src[zz].stride_h % sm == 0 && src[zz].stride_l % sm == 0 && dst[zz].stride_b % sm == 0 &&
                    dst[zz].stride_h % sm == 0 && dst[zz].stride_l % sm == 0,
                PSA_ERR_UNSUPPORTED, "psa_gather_rows: strides must be multiples of 16 bytes");
    p.src[z] = (const char*)src[zz].ptr; p.dst[z] = (char*)dst[zz].ptr;
    p.s_sb[z] = src[zz].stride_b * elem_bytes; p.s_sh[z] = src[zz].stride_h * elem_bytes; p.s_sl[z] = src[zz].stride_l * elem_bytes;
    p.d_sb[z] = dst[zz].stride_b * elem_bytes; p.d_sh[z] = dst[zz].stride_h * elem_bytes; p.d_sl[z] = dst[zz].stride_l * elem_bytes;
    p.H[z] = heads[zz];
    p.BH[z] = B * heads[zz];
    if (z < n_tensors && heads[zz] > maxH) maxH = heads[zz];
  }
  PSA_REQUIRE((int64_t)B * maxH <= 65535, PSA_ERR_UNSUPPORTED, "psa_gather_rows: B*H too large");
  p.index = index; p.L = L_dst; p.L_src = L_src; p.row_bytes = row_bytes;
  const int rows_per_wg = 256 / (row_bytes / 16) * 4;
  int gx = (L_dst + rows_per_wg - 1) / rows_per_wg;
  gx = gx > 1024 ? 1024 : gx;
  // tensors with fewer heads than the largest (GQA) leave their surplus workgroups idle
  hipLaunchKernelGGL(psa_gather_rows_kernel, dim3((unsigned)gx, (unsigned)(B * maxH), (unsigned)n_tensors), dim3(256), 0, (hipStream_t)stream, p);
  return psa_check_launch("psa_gather_rows");
}
