"""Sparse attention from the index-list mask ("new mask type"), forward only.

reference: src/psa_triton/kernels/psa_kernel.py:351-457 (sparse_attention_factory and _forward).
"""
import torch

from .. import ops


def _forward(q, k, v, block_sparse_mask, sm_scale, BLOCK_M, BLOCK_N, POOLING_BLOCK_N):
    assert q.shape[-1] == k.shape[-1] == v.shape[-1]
    assert k.shape[2] == v.shape[2]
    assert q.shape[-1] in [64, 128]
    Nk = -(-k.shape[2] // POOLING_BLOCK_N)
    if block_sparse_mask.shape[-1] == Nk:
        dense = block_sparse_mask  # already a dense level map
    else:
        # index list with -1 separators -> dense int8 level map (segment order 1, 2, 4, 8)
        dense = ops.map_from_list(block_sparse_mask, Nk, torch.int8)
    return ops.sparse_attention_fwd(q, k, v, dense, BLOCK_M, POOLING_BLOCK_N, sm_scale, causal=False)


def sparse_attention_factory(BLOCK_M=128, BLOCK_N=128, POOLING_BLOCK_N=128, **kwargs):
    """(block_m, tile_n, block_n) -> fn(q, k, v, mask, sm_scale=None).  tile_n (BLOCK_N) only shaped
    the reference's inner tiles; the HIP kernel picks its own and ignores it."""
    if BLOCK_M not in (64, 128):
        raise ValueError(f"BLOCK_M must be 64 or 128, got {BLOCK_M}")
    if POOLING_BLOCK_N not in (128, 64, 32):
        raise ValueError(f"POOLING_BLOCK_N must be 128, 64 or 32, got {POOLING_BLOCK_N}")

    def _sparse_attention_fn(q, k, v, block_sparse_dense, sm_scale=None):
        sm_scale = sm_scale if sm_scale is not None else q.shape[-1] ** -0.5
        return _forward(q, k, v, block_sparse_dense, sm_scale, BLOCK_M, BLOCK_N, POOLING_BLOCK_N)

    return _sparse_attention_fn


def sparse_attention(q, k, v, block_sparse_dense, sm_scale=None):
    sm_scale = sm_scale if sm_scale is not None else q.shape[-1] ** -0.5
    return _forward(q, k, v, block_sparse_dense, sm_scale, 64, 64, 128)


block_sparse_triton_fn = sparse_attention
