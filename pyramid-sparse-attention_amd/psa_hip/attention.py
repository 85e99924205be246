"""Plug-and-play Pyramid Sparse Attention: `PSAAttention()(q, k, v)`.

Same names, fields, defaults and errors as the reference module
(reference: src/psa_triton/attention.py:36-103 PSAConfig, :178-223 estimate, :226-310 module,
:314-367 functional form).  The pipeline behind it is four HIP kernels on the current stream:

    estimate (sampled rows gathered in-kernel)  ->  level map  ->  pyramid pooling  ->  sparse forward
"""
from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from . import ops
from .kernels.psa_kernel import sparse_attention_factory as psa_sparse_attention
from .kernels.psa_kernel_legacy import sparse_attention_factory as psa_sparse_attention_legacy
from .kernels.calc_ksim_kernel import calc_k_similarity


def _default_mask_ratios():
    return {
        1: (0.0, 0.1),     # most important 10 %: full resolution
        2: (0.1, 0.15),    # next 5 %: K/V pooled by 2
        4: (0.15, 0.15),   # (empty) pooled by 4
        8: (0.15, 0.35),   # next 20 %: pooled by 8
        0: (0.35, 1.0),    # remaining 65 %: skipped
    }


@dataclass
class PSAConfig:
    """Configuration of PSAAttention (defaults: about 85 % sparsity)."""

    block_m: int = 128   # query block
    block_n: int = 64    # key/value block (new_mask_type: 128/64/32, old_mask_type: 128)
    tile_n: int = 32     # only enters the level-count alignment of the mask
    mask_ratios: Dict[int, Tuple[float, float]] = field(default_factory=_default_mask_ratios)
    mask_mode: str = "topk"          # 'topk' (fixed quotas) or 'thresholdbound' (cumulative mass)
    use_sim_mask: bool = False       # cap the pooling level by key similarity (old_mask_type only)
    sim_2x_threshold: float = 0.0
    sim_4x_threshold: float = 0.0
    sim_8x_threshold: float = -1.0
    rearrange_method: str = None     # 'Gilbert', 'STA', 'SemanticAware', 'Hybrid' (unused here)
    attn_impl: str = "new_mask_type"  # mask format: "new_mask_type" (index list) / "old_mask_type" (dense)

    def __post_init__(self):
        if self.attn_impl == "new_mask_type" and self.use_sim_mask:
            raise ValueError(
                "Incompatible configuration: 'new_mask_type' does not support 'use_sim_mask=True'.\n"
                "Please choose one of the following options:\n"
                "  1. Set 'use_sim_mask=False' to disable similarity mask\n"
                "  2. Use 'attn_impl=\"old_mask_type\"' with block_size config (m=128, n=128, tile_n=32)"
            )
        if self.attn_impl == "old_mask_type":
            if self.block_m != 128 or self.block_n != 128:
                raise ValueError(
                    f"attn_impl='old_mask_type' only supports block_m=128 and block_n=128.\n"
                    f"Got block_m={self.block_m}, block_n={self.block_n}.\n"
                    f"Use attn_impl='new_mask_type' for flexible block sizes (128/64/32)."
                )
        if self.attn_impl == "new_mask_type":
            if self.block_n not in [128, 64, 32]:
                raise ValueError(
                    f"attn_impl='new_mask_type' only supports block_n in [128, 64, 32].\n"
                    f"Got block_n={self.block_n}."
                )


def draw_sample_offsets(B: int, H: int, block: int, keep: int, device, generator=None) -> torch.Tensor:
    """`keep` distinct in-block offsets per (b, h), int32 [B,H,keep]; every block of a head uses the
    same offsets.  reference: src/psa_triton/attention.py:132-133 (rand -> topk).  With a torch generator the draw is
    torch's own rand -> topk on that generator's device; without one it is a single kernel on the GPU
    (ops.draw_sample_offsets: both tensors of a layer in one launch, nothing crosses the host)."""
    if generator is not None:
        r = torch.rand(B, H, block, device=generator.device, generator=generator)
        return torch.topk(r, keep, dim=2).indices.to(torch.int32).contiguous().to(device)
    return ops.draw_sample_offsets(B, H, H, block, keep, block, keep, device)[0]


def draw_layer_offsets(B: int, Hq: int, Hkv: int, block_m: int, block_n: int, device):
    """(off_q, off_k) of one layer: a quarter of each block, drawn on the device in one launch."""
    return ops.draw_sample_offsets(B, Hq, Hkv, block_m, block_m // 4, block_n, block_n // 4, device)


def _compute_attention_pooling(q, k, v, config, sample_offsets=None):
    """Block importance [B,H,Mq,Nk] (fp32) and the optional similarity cap [B,H,Nk].
    reference: src/psa_triton/attention.py:178-223."""
    keep_m, keep_n = config.block_m // 4, config.block_n // 4
    B, H = q.shape[0], q.shape[1]
    Hkv = k.shape[1]
    sim_cap = None
    if config.use_sim_mask:
        sim_cap = calc_k_similarity(k, config.block_n, config)
    if sample_offsets is None:
        off_q, off_k = draw_layer_offsets(B, H, Hkv, config.block_m, config.block_n, q.device)
    else:
        off_q, off_k = sample_offsets
    pooling = ops.estimate_sampled(q, k, off_q, off_k, config.block_m, config.block_n, keep_m, keep_n, q.size(-1) ** -0.5)
    return pooling, sim_cap


class PSAAttention(nn.Module):
    """Drop-in sparse attention: out = PSAAttention(config)(q, k, v) with q, k, v [B,H,L,D]."""

    def __init__(self, config: PSAConfig = None):
        super().__init__()
        self.config = config if config is not None else PSAConfig()
        if self.config.attn_impl == "old_mask_type":
            self.sparse_attention_fn = psa_sparse_attention_legacy(self.config.block_m, self.config.tile_n, self.config.block_n)
        else:
            self.sparse_attention_fn = psa_sparse_attention(self.config.block_m, self.config.tile_n, self.config.block_n)
        self.sample_offsets = None  # set to (off_q, off_k) to make the estimate reproducible

    def build_mask(self, q, k, v):
        """estimate -> level mask in the format `attn_impl` selects (no gradient)."""
        config = self.config
        with torch.no_grad():
            pooling, sim_cap = _compute_attention_pooling(q, k, v, config, self.sample_offsets)
            mode = config.mask_mode if config.attn_impl == "old_mask_type" else f"{config.mask_mode}_newtype"
            mask = ops.level_map(pooling, config.mask_ratios, 0, mode, blocksize=config.block_n, compute_tile=config.tile_n)
            if config.use_sim_mask and sim_cap is not None:
                mask = ops.map_min_cap(mask, sim_cap)
        return mask

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        config = self.config
        needs_grad = torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)
        if not needs_grad:
            # inference: the stages back to back with a dense int8 level map (same levels as the mask formats)
            if self.sample_offsets is None:
                B, H, Hkv = q.shape[0], q.shape[1], k.shape[1]
                off_q, off_k = draw_layer_offsets(B, H, Hkv, config.block_m, config.block_n, q.device)
            else:
                off_q, off_k = self.sample_offsets
            cap = calc_k_similarity(k, config.block_n, config) if config.use_sim_mask else None
            return ops.psa_layer_fwd(q, k, v, off_q, off_k, config.mask_ratios, config.mask_mode, config.block_m,
                                     config.block_n, config.tile_n, level_cap=cap)
        mask = self.build_mask(q, k, v)
        return self.sparse_attention_fn(q, k, v, mask, None)


def psa_attention(q, k, v, *, config: PSAConfig = None, mask_ratios=None, mask_mode: str = None, block_m: int = None,
                  block_n: int = None) -> torch.Tensor:
    """Functional form; keyword overrides as in the reference (block_n also sets tile_n = min(32, block_n))."""
    if config is None:
        config = PSAConfig()
    if mask_ratios is not None:
        config.mask_ratios = mask_ratios
    if mask_mode is not None:
        config.mask_mode = mask_mode
    if block_m is not None:
        config.block_m = block_m
    if block_n is not None:
        config.block_n = block_n
        config.tile_n = min(32, block_n)
    return PSAAttention(config)(q, k, v)
