from .transfer_attn_to_mask import transfer_attn_to_mask, calc_density, calc_density_newtype

__all__ = ["transfer_attn_to_mask", "calc_density", "calc_density_newtype"]
