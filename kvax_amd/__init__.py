"""MI355X-native implementation of the kvax attention hot path (block-mask builder,
flash-attention forward and backward) behind kvax's public Python surface."""
__version_info__ = (0, 1, 0)
__version__ = ".".join(str(v) for v in __version_info__)

from kvax_amd import utils  # noqa: E402,F401
