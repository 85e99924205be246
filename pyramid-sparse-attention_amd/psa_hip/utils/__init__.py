"""Utilities of the reference's psa_triton.utils that lie on the attention path: the Gilbert curve and its
re-ordering, scores -> level mask, densities, dense mask -> index list.
reference: src/psa_triton/utils/__init__.py:7-21 (the k-means / STA / hybrid re-orderings and the timer are not on the path)."""
from .gilbert3d import gilbert3d
from .rearranger import GilbertRearranger
from .transfer_attn_to_mask import calc_density, calc_density_newtype, transfer_attn_to_mask, transfer_mask_to_new_type

__all__ = ["gilbert3d", "transfer_attn_to_mask", "transfer_mask_to_new_type", "calc_density", "calc_density_newtype",
           "GilbertRearranger"]
