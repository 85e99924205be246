"""HIP-backed counterparts of the reference's kernel modules (same module and function names)."""
from .psa_kernel import sparse_attention_factory as psa_sparse_attention
from .psa_kernel_legacy import sparse_attention_factory as psa_sparse_attention_legacy
from .attn_pooling_kernel import attn_with_pooling_optimized
from .calc_ksim_kernel import calc_k_similarity, calc_k_similarity_triton

__all__ = [
    "psa_sparse_attention",
    "psa_sparse_attention_legacy",
    "attn_with_pooling_optimized",
    "calc_k_similarity",
    "calc_k_similarity_triton",
]
