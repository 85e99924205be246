"""Causal PSA for decoder prefill (the Qwen2.5-VL example of the reference), on the HIP kernels.
reference: qwen2.5-vl-example/src/attention/PSA_casual/."""
from .PyramidAdaptiveBlockSparseAttn import (
    AttentionConfig,
    PyramidAdaptiveBlockSparseAttnTrain,
    adaptive_block_sparse_attn,
    calc_density,
    transfer_attn_to_mask,
    x_block_imp_estimate,
)

__all__ = ["AttentionConfig", "PyramidAdaptiveBlockSparseAttnTrain", "adaptive_block_sparse_attn", "calc_density",
           "transfer_attn_to_mask", "x_block_imp_estimate"]
