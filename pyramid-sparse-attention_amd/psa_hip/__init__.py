"""psa_hip - Pyramid Sparse Attention on AMD MI355X (gfx950) through hand-written HIP kernels.

Public names follow the reference package (src/psa_triton/__init__.py:9-31)."""
from .attention import PSAAttention, PSAConfig, psa_attention
from .pyramid_sparse_attention import PyramidSparseAttention, AttentionConfig

__version__ = "0.1.0"

__all__ = ["PSAAttention", "PSAConfig", "psa_attention", "PyramidSparseAttention", "AttentionConfig"]
