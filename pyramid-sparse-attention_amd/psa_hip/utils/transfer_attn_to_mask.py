"""Scores -> pyramid level mask, and density of a mask.

reference: src/psa_triton/utils/transfer_attn_to_mask.py:6-507 (transfer_attn_to_mask),
:510-544 (calc_density), :547-622 (calc_density_newtype), :624-750 (transfer_mask_to_new_type).
"""
from typing import Dict, Optional, Tuple

import torch

from .. import ops


def transfer_attn_to_mask(
    attn: torch.Tensor,
    mask_ratios: Optional[Dict[int, Tuple[float, float]]] = None,
    text_length: int = 226,
    mode: str = "topk",
    min_full_attn_ratio: float = 0.06,
    blocksize=32,
    compute_tile=32,
) -> torch.Tensor:
    """attn [B,H,Mq,Nk] block importance -> int32 mask.

    mode 'topk' / 'thresholdbound': dense mask of levels {0,1,2,4,8}, with the last
    ceil(text_length/blocksize) kv-blocks forced to 1.  mode '*_newtype': index list of width
    Nk+len(mask_ratios) with -1 separators (text_length ignored).  Ties in `attn` are broken towards
    the lower kv-block index (the reference leaves tie order to torch.sort)."""
    if mask_ratios is None:
        raise ValueError("mask_ratios must be provided")
    return ops.level_map(attn, mask_ratios, text_length, mode, min_full_attn_ratio, blocksize, compute_tile, torch.int32)


def calc_density(mask: torch.Tensor):
    """(mean density, per-head densities) of a dense level mask; density of a block = 1/level."""
    B, H = mask.shape[0], mask.shape[1]
    d = ops.density(mask if mask.dtype in (torch.int8, torch.int32) else mask.to(torch.int32)).cpu()
    per_bh = d[:-1].view(B, H)
    return float(d[-1]), [float(x) for x in per_bh.mean(0)]


def calc_density_newtype(mask: torch.Tensor):
    """Same for the index-list format."""
    n_sep = 5
    Nk = mask.shape[-1] - n_sep
    return calc_density(ops.map_from_list(mask, Nk, torch.int8))


def transfer_mask_to_new_type(mask: torch.Tensor, blocksize=32, compute_tile=32) -> torch.Tensor:
    """Dense level mask [B,H,Mq,Nk] (values 0, 1, 2, 4, 8) -> index list [B,H,Mq,Nk+5] int32: the kv-blocks at levels
    1, 2, 4, 8 and the skipped ones, -1 behind each segment.  Blocks of a level are listed in ascending order (the
    reference leaves their order to torch.sort); segment lengths are rounded down to the level's alignment
    ceil(level / (blocksize // compute_tile)), the excess leading the next segment."""
    return ops.list_from_map(mask, blocksize, compute_tile)
