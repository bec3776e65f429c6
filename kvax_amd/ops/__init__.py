from kvax_amd.ops.flash_attention import flash_attention
from kvax_amd.ops.mask_creator import create_attention_mask

__all__ = [
    "flash_attention",
    "create_attention_mask",
]
