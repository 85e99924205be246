"""Full-featured PSA module used by the diffusers attention processors:
`attn.inner_attention(q, k, v, layer_idx)`.

reference: src/psa_triton/pyramid_sparse_attention.py:28-83 (AttentionConfig), :139-249
(estimate + mask + kernel), :252-413 (PyramidSparseAttention: warm-up steps, step counter,
density logging, rearrangement hooks).
"""
import json
import os
import time
from dataclasses import asdict, dataclass
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from . import ops
from .attention import draw_layer_offsets, draw_sample_offsets
from .kernels.calc_ksim_kernel import calc_k_similarity
from .kernels.psa_kernel import sparse_attention_factory as psa_sparse_attention
from .kernels.psa_kernel_legacy import sparse_attention_factory as psa_sparse_attention_legacy


@dataclass
class AttentionConfig:
    """All tunables of the module (field names and defaults as in the reference)."""

    # latent video grid and text tokens
    width: int = 45
    height: int = 30
    depth: int = 13
    text_length: int = 226
    # attention
    use_rearrange: bool = True
    block_m: int = 32
    block_n: int = 32
    tile_n: int = 32
    use_sim_mask: bool = True
    mask_ratios: Dict[int, Tuple[float, float]] = None
    mask_mode: str = "topk"
    warmup_steps: int = 12
    tile_size: Optional[Tuple[int, int, int]] = None
    rearrange_method: str = None
    attn_impl: str = "new_mask_type"
    # logging
    verbose: bool = False
    enable_logging: bool = True
    log_dir: str = "./psa_logs/"
    # similarity thresholds of the sim mask
    sim_2x_threshold: float = 0
    sim_4x_threshold: float = 0
    sim_8x_threshold: float = -1

    def __post_init__(self):
        if self.mask_ratios is None:
            self.mask_ratios = {1: (0.0, 0.05), 2: (0.05, 0.15), 4: (0.15, 0.25), 8: (0.25, 0.5), 0: (0.5, 1.0)}
        if self.attn_impl == "new_mask_type" and self.use_sim_mask:
            raise ValueError(
                "Incompatible configuration: 'new_mask_type' does not support 'use_sim_mask=True'.\n"
                "Please choose one of the following options:\n"
                "  1. Set 'use_sim_mask: false' to disable similarity mask\n"
                "  2. Use 'attn_impl: old_mask_type' with block_size config (m=128, n=128, tile_n=32)"
            )


def efficient_attn_with_pooling(q, k, v, config, num_keep_m=32, num_keep_n=32, sample_offsets=None, q_index=None):
    """Block importance [B,H,Mq,Nk] fp32 and the similarity cap [B,H,Nk] (or None).  q_index: see
    adaptive_block_sparse_attn.
    reference: src/psa_triton/pyramid_sparse_attention.py:139-187."""
    sim_cap = calc_k_similarity(k, config.block_n, config) if getattr(config, "use_sim_mask", True) else None
    B, H, Hkv = q.shape[0], q.shape[1], k.shape[1]
    if sample_offsets is None:
        off_q, off_k = ops.draw_sample_offsets(B, H, Hkv, config.block_m, num_keep_m, config.block_n, num_keep_n, q.device)
    else:
        off_q, off_k = sample_offsets
    pooling = ops.estimate_sampled(q, k, off_q, off_k, config.block_m, config.block_n, num_keep_m, num_keep_n, q.size(-1) ** -0.5,
                                   q_index=q_index)
    return pooling, sim_cap


def adaptive_block_sparse_attn(q, k, v, config, sparse_attention_fn, compute_stats=False, sample_offsets=None, q_index=None,
                               pools=None):
    """estimate -> mask (-> min with the similarity cap) -> sparse attention.
    Returns (out, sparsity, per_head_density, sim_cap); the statistics are device tensors
    (no host synchronisation) unless compute_stats is False, in which case they are 0.0 / [].
    q_index / pools (token re-ordering without gather passes, forward only): k, v are the re-ordered rows and pools their
    pooled levels (ops.pool_kv_indexed), q is in the original order and read through q_index, and out comes back in the
    original order.
    reference: src/psa_triton/pyramid_sparse_attention.py:188-249."""
    with torch.no_grad():
        pooling, sim_cap = efficient_attn_with_pooling(q, k, v, config, config.block_m // 4, config.block_n // 4, sample_offsets,
                                                       q_index)
        if config.attn_impl == "old_mask_type":
            mask = ops.level_map(pooling, config.mask_ratios, config.text_length, config.mask_mode, blocksize=config.block_n,
                                 compute_tile=config.tile_n)
        elif config.attn_impl == "new_mask_type":
            mode = {"topk": "topk_newtype", "thresholdbound": "thresholdbound_newtype"}.get(config.mask_mode, "topk_newtype")
            mask = ops.level_map(pooling, config.mask_ratios, config.text_length, mode, blocksize=config.block_n,
                                 compute_tile=config.tile_n)
        else:
            raise ValueError(f"Unknown attn_impl: {config.attn_impl}")
        if getattr(config, "use_sim_mask", True) and sim_cap is not None:
            mask = ops.map_min_cap(mask, sim_cap)
    dense = None
    if q_index is None:
        out = sparse_attention_fn(q, k, v, mask, None)
    else:
        dense = mask if config.attn_impl == "old_mask_type" else ops.map_from_list(mask, -(-k.shape[2] // config.block_n), torch.int8)
        out = ops.sparse_attention_fwd(q, k, v, dense, config.block_m, config.block_n, pools=pools, q_index=q_index)
    if compute_stats:
        if dense is None:
            dense = mask if config.attn_impl == "old_mask_type" else ops.map_from_list(mask, -(-k.shape[2] // config.block_n))
        d = ops.density(dense)  # [B*H + 1] on the device
        sparsity = 1 - d[-1]
        per_head = d[:-1].view(q.shape[0], q.shape[1]).mean(0)
    else:
        sparsity, per_head = 0.0, []
    return out, sparsity, per_head, sim_cap


class PyramidSparseAttention(nn.Module):
    """One instance is shared by every transformer block: forward(q, k, v, layer_idx)."""

    def __init__(self, config: AttentionConfig = None, inference_num=50, layer_num=42, model_type="wan"):
        super().__init__()
        if config is None:
            config = AttentionConfig()
        self.config = config
        self.model_type = model_type.lower()
        self.rearranger = None
        if config.use_rearrange:
            if config.rearrange_method == "Gilbert":
                from .utils.rearranger import GilbertRearranger

                self.rearranger = GilbertRearranger(config.width, config.height, config.depth, config.text_length)
            else:
                raise NotImplementedError(
                    f"rearrange_method={config.rearrange_method!r}: only 'Gilbert' (the method every shipped preset selects) is built"
                )
        self.sparsity_acc = 0.0
        self.sparsity_counter = 0
        self.use_rearrange = config.use_rearrange
        # True: the re-ordering is read / written by the layer's own kernels through the token index (no gather passes);
        # False: rearrange() before and reversed_rearrange() after, the reference's sequence of operations.  The two give
        # the same bits outside the warm-up steps (during warm-up the first runs dense attention in the original order,
        # which differs from the re-ordered dense attention only in the order of the fp32 sums over the keys).
        self.fuse_rearrange = True
        self.inference_num = inference_num
        self.layer_num = layer_num
        self.sample_offsets = None
        if config.attn_impl == "old_mask_type":
            self.sparse_attention_fn = psa_sparse_attention_legacy(config.block_m, config.tile_n, config.block_n)
        elif config.attn_impl == "new_mask_type":
            self.sparse_attention_fn = psa_sparse_attention(config.block_m, config.tile_n, config.block_n)
        else:
            raise ValueError(f"Unknown attn_impl: {config.attn_impl}")
        self.logger = None
        if config.enable_logging:
            from .utils.psa_logger import PSALogger

            self.logger = PSALogger(config.log_dir, config, model_type, layer_num, inference_num)

    def get_current_time(self):
        """Denoising step index derived from the call counter (Wan runs cond + uncond per step)."""
        if self.model_type == "cogvideo" or self.model_type == "wan2.1_1.3b_4steps":
            return (self.sparsity_counter // self.layer_num) % self.inference_num
        return (self.sparsity_counter // (2 * self.layer_num)) % self.inference_num

    def forward(self, q, k, v, layer_idx):
        is_warmup = self.get_current_time() < self.config.warmup_steps
        compute_stats = self.config.verbose or self.logger is not None
        fused = (self.rearranger is not None and self.fuse_rearrange
                 and not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)))
        restore = self.rearranger is not None and not fused
        if restore:
            q_r, k_r, v_r = self.rearranger.rearrange(q, k, v)
        else:
            q_r, k_r, v_r = q, k, v
        sim_cap = None
        if is_warmup:
            out_r = ops.sparse_attention_fwd(q_r, k_r, v_r, None, 128, 128)  # dense attention, same kernel
            sparsity = 0.0
            per_head_density = [1.0] * q_r.shape[1] if compute_stats else []
        elif not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)):
            out_r, sparsity, per_head_density, sim_cap = self._sparse_layer(q_r, k_r, v_r, fused, compute_stats)
            if compute_stats:
                self.sparsity_acc = self.sparsity_acc + sparsity
        else:
            out_r, sparsity, per_head_density, sim_cap = adaptive_block_sparse_attn(
                q_r, k_r, v_r, self.config, self.sparse_attention_fn, compute_stats=compute_stats, sample_offsets=self.sample_offsets
            )
            if compute_stats:
                self.sparsity_acc = self.sparsity_acc + sparsity
        self.sparsity_counter += 1
        if self.logger is not None:
            self.logger.log_sparsity(layer_idx=layer_idx, sparsity=sparsity, per_head_density=per_head_density,
                                     sequence_length=q.shape[2], batch_size=q.shape[0], num_heads=q.shape[1], sim_mask=sim_cap,
                                     is_warmup=is_warmup)
        return self.rearranger.reversed_rearrange(out_r) if restore else out_r

    def _sparse_layer(self, q, k, v, through_index, compute_stats):
        """The sparse layer without gradients through the layer operator (ops.psa_layer_fwd): estimate and level map in
        two launches, the similarity cap, pooling and the token re-ordering inside the layer's kernels, and a dense
        int8 level map for either mask type (the index-list modes select the same levels and ignore the text
        columns).  Same outputs, bit for bit, as adaptive_block_sparse_attn on re-ordered tensors."""
        cfg = self.config
        B, H, Hkv = q.shape[0], q.shape[1], k.shape[1]
        if self.sample_offsets is None:
            off_q, off_k = draw_layer_offsets(B, H, Hkv, cfg.block_m, cfg.block_n, q.device)
        else:
            off_q, off_k = self.sample_offsets
        if cfg.mask_mode not in ("topk", "thresholdbound"):
            raise ValueError(f"Unknown mask_mode: {cfg.mask_mode}")
        thr = None
        if getattr(cfg, "use_sim_mask", True):
            thr = (float(cfg.sim_2x_threshold), float(cfg.sim_4x_threshold), float(cfg.sim_8x_threshold))
        out, mp, cap = ops.psa_layer_fwd(
            q, k, v, off_q, off_k, cfg.mask_ratios, cfg.mask_mode, cfg.block_m, cfg.block_n, cfg.tile_n,
            text_length=cfg.text_length if cfg.attn_impl == "old_mask_type" else 0,
            token_index=self.rearranger.token_index(q.device) if through_index else None,
            sim_thresholds=thr, return_map=True, return_cap=True)
        if compute_stats:
            d = ops.density(mp)  # [B*H + 1] on the device
            return out, 1 - d[-1], d[:-1].view(B, H).mean(0), cap
        return out, 0.0, [], cap

    def close_logger(self):
        if self.logger is not None:
            self.logger.close()

    def __del__(self):
        if getattr(self, "logger", None) is not None:
            try:
                self.logger.close()
            except Exception:  # the interpreter is shutting down: builtins and torch may already be gone
                pass
