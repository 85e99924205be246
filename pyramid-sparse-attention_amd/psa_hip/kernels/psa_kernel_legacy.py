"""Sparse attention from the dense level mask ("old mask type"): forward (optionally causal) and
backward.

reference: src/psa_triton/kernels/psa_kernel_legacy.py:837-938 (_forward), :941-1069
(_sparse_attention autograd function), :1323-1370 (sparse_attention_factory).
"""
import torch

from .. import ops


class _sparse_attention(torch.autograd.Function):
    """Differentiable in q, k, v; the mask carries no gradient."""

    @staticmethod
    def forward(ctx, q, k, v, block_sparse_dense, sm_scale, block_m=128, block_n=128, causal=False):
        sm_scale = sm_scale if sm_scale is not None else q.shape[-1] ** -0.5
        need_backward = q.requires_grad or k.requires_grad or v.requires_grad
        if not need_backward:
            return ops.sparse_attention_fwd(q, k, v, block_sparse_dense, block_m, block_n, sm_scale, causal=causal)
        o, lse, pools = ops.sparse_attention_fwd(q, k, v, block_sparse_dense, block_m, block_n, sm_scale, causal=causal,
                                               return_lse=True)
        ctx.save_for_backward(q, k, v, block_sparse_dense, o, lse, pools[0], pools[1])
        ctx.sm_scale, ctx.causal, ctx.block_m, ctx.block_n = sm_scale, causal, block_m, block_n
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, mask, o, lse, kp, vp = ctx.saved_tensors
        dq, dk, dv = ops.sparse_attention_bwd(q, k, v, mask, o, do, lse, ctx.block_m, ctx.block_n, ctx.sm_scale,
                                              causal=ctx.causal, pools=(kp, vp))
        return dq, dk, dv, None, None, None, None, None


def sparse_attention_factory(BLOCK_M=128, BLOCK_N=32, POOLING_BLOCK_N=128, causal=False, **kwargs):
    """(block_m, tile_n, block_n[, causal]) -> fn(q, k, v, mask, sm_scale=None); same restrictions as
    the reference: block_m = 128, tile_n = 32, block_n = 128."""
    if BLOCK_M != 128:
        raise ValueError(
            f"BLOCK_M must be 128, got {BLOCK_M}. "
            "Current version only supports BLOCK_M=128, BLOCK_N=32, POOLING_BLOCK_N=128. "
            "For more flexible configurations, please use psa_hip/kernels/psa_kernel.py"
        )
    if BLOCK_N != 32:
        raise ValueError(
            f"BLOCK_N must be 32, got {BLOCK_N}. "
            "Current version only supports BLOCK_M=128, BLOCK_N=32, POOLING_BLOCK_N=128. "
            "For more flexible configurations, please use psa_hip/kernels/psa_kernel.py"
        )
    if POOLING_BLOCK_N != 128:
        raise ValueError(
            f"POOLING_BLOCK_N must be 128, got {POOLING_BLOCK_N}. "
            "Current version only supports BLOCK_M=128, BLOCK_N=32, POOLING_BLOCK_N=128. "
            "For more flexible configurations, please use psa_hip/kernels/psa_kernel.py"
        )

    def _fn(q, k, v, block_sparse_dense, sm_scale=None):
        return _sparse_attention.apply(q, k, v, block_sparse_dense, sm_scale, BLOCK_M, POOLING_BLOCK_N, causal)

    return _fn


def block_sparse_triton_fn(q, k, v, block_sparse_dense, sm_scale=None):
    return _sparse_attention.apply(q, k, v, block_sparse_dense, sm_scale, 128, 128, False)
