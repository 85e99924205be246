"""Causal pyramid sparse attention module: antidiagonal block-importance estimate -> causal level map
(-> min with the key-similarity cap) -> causal sparse attention.

reference: qwen2.5-vl-example/src/attention/PSA_casual/PyramidAdaptiveBlockSparseAttn.py:22-57 (AttentionConfig),
:60-82 (x_block_imp_estimate), :84-168 (transfer_attn_to_mask), :171-195 (calc_density), :198-248
(adaptive_block_sparse_attn), :250-333 (PyramidAdaptiveBlockSparseAttnTrain).

K and V may carry fewer heads than Q (grouped-query attention): the kernels map query head h to kv head
h // (Hq // Hkv), so the caller does not need to repeat K/V first.
"""
import json
import os
from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from .. import ops
from ..kernels.psa_kernel_legacy import _sparse_attention


@dataclass
class AttentionConfig:
    """Runtime configuration (field names and defaults as in the reference)."""

    text_length: int = 512
    query_block: int = 128
    warmup_steps: int = 0
    mask_ratios: Dict[int, Tuple[float, float]] = field(
        default_factory=lambda: {1: (0.0, 0.05), 2: (0.05, 0.15), 4: (0.15, 0.25), 8: (0.25, 0.5), 0: (0.5, 1.0)}
    )
    mask_mode: str = "topk"
    importance_method: str = "xattn"
    xattn_stride: int = 16
    xattn_chunk_size: int = 4096
    causal_main: bool = True
    sim_2x_threshold: float = 0.75
    sim_4x_threshold: float = 0.7
    sim_8x_threshold: float = 0.7

    def __post_init__(self) -> None:
        self.importance_method = self.importance_method.lower()
        if self.importance_method not in {"xattn"}:
            raise ValueError("importance_method must be 'xattn'")
        self.mask_mode = self.mask_mode.lower()
        if self.mask_mode not in {"topk", "energybound"}:
            raise ValueError("mask_mode must be 'topk' or 'energybound'")


def sparse_attention_factory(BLOCK_M=128, BLOCK_N=32, POOLING_BLOCK_N=128, causal=False, **kwargs):
    """The causal copy of the dense-map kernel factory (no block-size validation in the reference:
    qwen2.5-vl-example/src/attention/PSA_casual/kernels/psa_kernel_causal.py:930-955)."""

    def _fn(q, k, v, block_sparse_dense, sm_scale=None):
        return _sparse_attention.apply(q, k, v, block_sparse_dense, sm_scale, BLOCK_M, POOLING_BLOCK_N, causal)

    return _fn


def x_block_imp_estimate(query, key, *, block_size: int, stride: int, chunk_size: int, causal: bool) -> torch.Tensor:
    """fp32 [B,Hq,ceil(L/block),ceil(L/block)] importance of kv-blocks per q-block."""
    return ops.estimate_xattn(query, key, block_size=block_size, stride=stride, causal=causal, chunk_size=chunk_size)


def transfer_attn_to_mask(attn, mask_ratios, text_length: int, mode: str, *, block_size: int, causal: bool) -> torch.Tensor:
    """Block scores [B,H,S,S] -> int32 level map with the causal fix-ups (trailing text blocks, diagonal and first
    column at level 1, nothing above the diagonal)."""
    if not mask_ratios:
        raise ValueError("mask_ratios must not be empty")
    if mode not in {"topk", "energybound"}:
        raise ValueError("mode must be 'topk' or 'energybound'")
    return ops.level_map_qwen(attn, mask_ratios, text_length, mode, block_size=block_size, causal=causal)


def calc_density(mask: torch.Tensor, causal: bool):
    """(mean density, per-head densities) over the lower triangle (causal) or the full map."""
    B, H = mask.shape[0], mask.shape[1]
    d = ops.density(mask if mask.dtype in (torch.int8, torch.int32) else mask.to(torch.int32), causal=causal).cpu()
    return float(d[-1]), [float(x) for x in d[:-1].view(B, H).mean(0)]


def adaptive_block_sparse_attn(q, k, v, config: AttentionConfig, sparse_attention_fn, compute_stats: bool = True):
    block = config.query_block
    with torch.no_grad():
        if config.importance_method != "xattn":
            raise ValueError(f"Unknown importance_method: {config.importance_method}")
        est = x_block_imp_estimate(q, k, block_size=block, stride=config.xattn_stride, chunk_size=config.xattn_chunk_size,
                                   causal=config.causal_main)
        mask = transfer_attn_to_mask(est, config.mask_ratios, config.text_length, config.mask_mode, block_size=block,
                                     causal=config.causal_main)
        cap = ops.k_similarity(k, block, config.sim_2x_threshold, config.sim_4x_threshold, config.sim_8x_threshold)
        n_rep = q.shape[1] // k.shape[1]
        if n_rep > 1:
            cap = cap.repeat_interleave(n_rep, dim=1)
        mask = ops.map_min_cap(mask, cap)
    out = sparse_attention_fn(q, k, v, mask, None)
    if not compute_stats:
        return out, 0.0, []
    d = ops.density(mask, causal=config.causal_main)  # stays on the device
    return out, 1 - d[-1], d[:-1].view(q.shape[0], q.shape[1]).mean(0)


class PyramidAdaptiveBlockSparseAttnTrain(nn.Module):
    """forward(q, k, v, ..., layer_idx=...) -> out; dense attention during the first `warmup_steps` calls."""

    def __init__(self, config: Optional[AttentionConfig] = None, *, layer_idx: int = -1, log_dir: Optional[str] = None,
                 log_prefix: str = "psa_sparsity", session_name: Optional[str] = None, **extra: object) -> None:
        super().__init__()
        self.config = config or AttentionConfig()
        self.layer_idx = layer_idx
        self.sparse_attention_fn = sparse_attention_factory(causal=self.config.causal_main)
        self.sparsity_acc = 0.0
        self.sparsity_counter = 0
        if log_dir is None and "save_dir" in extra:
            log_dir = extra["save_dir"]
        self.log_path = None
        self._pending = []
        if log_dir is not None:
            os.makedirs(log_dir, exist_ok=True)
            self.log_path = os.path.join(log_dir, f"{session_name or log_prefix}_layer{layer_idx}.jsonl")

    def forward(self, q, k, v, frame_num=None, height=None, width=None, *, layer_idx: Optional[int] = None):
        if layer_idx is not None:
            self.layer_idx = layer_idx
        self.sparsity_counter += 1
        if self.sparsity_counter <= self.config.warmup_steps:
            # dense and NOT causal, as the reference does during warm-up (scaled_dot_product_attention(q, k, v) without a
            # mask: qwen2.5-vl-example/src/attention/PSA_casual/PyramidAdaptiveBlockSparseAttn.py:306-308)
            return ops.sparse_attention_fwd(q, k, v, None, 128, 128, causal=False)
        out, sparsity, per_head = adaptive_block_sparse_attn(q, k, v, self.config, self.sparse_attention_fn,
                                                             compute_stats=self.log_path is not None)
        if self.log_path is not None:
            self.sparsity_acc = self.sparsity_acc + sparsity
            self._pending.append((self.layer_idx, sparsity, per_head, q.size(2), q.size(0), q.size(1)))
            if len(self._pending) >= 256:
                self.flush_log()
        return out

    def flush_log(self) -> None:
        """Bring the logged densities to the host and append them to the JSONL file."""
        if self.log_path is None or not self._pending:
            return
        with open(self.log_path, "a") as f:
            for layer, sp, ph, L, B, H in self._pending:
                f.write(json.dumps(dict(layer_idx=layer, sparsity=float(sp), per_head_density=[float(x) for x in ph.cpu()],
                                        sequence_length=L, batch_size=B, num_heads=H)) + "\n")
        self._pending = []

    def __del__(self) -> None:
        try:
            self.flush_log()
        except Exception:
            pass
