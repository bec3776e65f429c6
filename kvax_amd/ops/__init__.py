from kvax_amd.ops.mask_creator import create_attention_mask

__all__ = ["create_attention_mask"]
