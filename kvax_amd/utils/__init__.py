from kvax_amd.utils.common import PADDING_SEGMENT_ID, FlashAttentionParamsConfig
from kvax_amd.utils.permutation import (
    permute_tokens_context_parallelism,
    unpermute_tokens_context_parallelism,
)
from kvax_amd.utils.sharding import Mesh
from kvax_amd.utils.specs import attention_specs

__all__ = [
    "FlashAttentionParamsConfig",
    "PADDING_SEGMENT_ID",
    "attention_specs",
    "permute_tokens_context_parallelism",
    "unpermute_tokens_context_parallelism",
    "Mesh",
]
