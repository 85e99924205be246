"""Per kv-block cap on the pooling level from the similarity of neighbouring keys ("sim mask").

reference: src/psa_triton/kernels/calc_ksim_kernel.py:6-157 (kernel), :160-225 (host wrapper).
"""
import torch

from .. import ops


def calc_k_similarity(k: torch.Tensor, blocksize: int, config) -> torch.Tensor:
    """k [B,H,L,D] -> int32 [B,H,ceil(L/blocksize)] in {1,2,4,8}: the largest l in {2,4,8} whose mean
    cosine similarity of token pairs (0,1), (0,3), (0,7) (per aligned group of l tokens) exceeds
    config.sim_{l}x_threshold; 1 if none does.  Tokens past L replicate the last one."""
    t2 = float(getattr(config, "sim_2x_threshold", 0.0))
    t4 = float(getattr(config, "sim_4x_threshold", 0.0))
    t8 = float(getattr(config, "sim_8x_threshold", -1.0))
    return ops.k_similarity(k, blocksize, t2, t4, t8)


calc_k_similarity_triton = calc_k_similarity
