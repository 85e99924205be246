"""Block-importance estimator entry point with the reference's call signature.

reference: src/psa_triton/kernels/attn_pooling_kernel.py:434-451 (attn_with_pooling_optimized)
and its assertions at :342-355.
"""
import torch

from .. import ops

_SIZES = {4, 8, 16, 32, 64, 128}


def attn_with_pooling_optimized(q, k, v, causal, sm_scale, block_size_m, block_size_n, tile_m=64, tile_n=64):
    """q [B,Hq,Ms,D] and k [B,Hkv,Ns,D] are ALREADY-sampled rows, padded to multiples of 64 by the
    caller; consecutive groups of block_size_m rows / block_size_n keys form one block.

    Returns (None, Po) with Po [B,Hq,ceil(Ms/block_size_m),ceil(Ns/block_size_n)]: rows normalised to
    sum 1.  Differences from the reference, both deliberate: Po is fp32 (the reference rounds the
    intermediate maxima and Po to q.dtype), and the unused attention output is None instead of an
    uninitialised tensor.  `v` is accepted for signature compatibility and not read.
    """
    assert block_size_m in _SIZES and block_size_n in _SIZES
    assert tile_n % block_size_n == 0 and tile_m % block_size_m == 0
    assert 0 < tile_m <= 256 and 0 < tile_n <= 256
    assert q.shape[-1] == k.shape[-1] and q.shape[-1] in {16, 32, 64, 128, 256}
    if causal:
        raise ValueError("the causal variant of the sampled estimator is not used by PSA and is not built")
    if block_size_m < 8 or block_size_n < 8 or block_size_m > 32 or block_size_n > 32:
        raise ValueError("block_size_m / block_size_n (rows kept per block) must be 8, 16 or 32")
    Ms, Ns = q.shape[2], k.shape[2]
    m_d = -(-(-(-Ms // 64) * 64) // block_size_m)
    n_d = -(-(-(-Ns // 64) * 64) // block_size_n)
    # rows are already sampled: block == keep and the offsets are 0..keep-1
    po = ops.estimate_sampled(q, k, None, None, block_size_m, block_size_n, block_size_m, block_size_n, sm_scale,
                              out_rows=m_d, out_cols=n_d)
    return None, po
