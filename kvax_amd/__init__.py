"""MI355X-native implementation of the kvax attention hot path (block-mask builder,
flash-attention forward and backward) behind kvax's public Python surface."""
__version_info__ = (0, 1, 0)
__version__ = ".".join(str(v) for v in __version_info__)

import kvax_amd.ops as ops  # noqa: E402
import kvax_amd.utils as utils  # noqa: E402
from kvax_amd.ops import create_attention_mask, flash_attention  # noqa: E402,F401
from kvax_amd.utils import (  # noqa: E402,F401
    PADDING_SEGMENT_ID,
    FlashAttentionParamsConfig,
    Mesh,
    attention_specs,
    permute_tokens_context_parallelism,
    unpermute_tokens_context_parallelism,
)

__all__ = []
__all__ += ops.__all__
__all__ += utils.__all__
