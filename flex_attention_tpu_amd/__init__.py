"""MI355X-native flex-attention: hand-written gfx950 HIP kernels behind the Python call surface of
james-zhengql/flex_attention_tpu (forward, dq backward, dk/dv backward, score and mask factories).
"""
from . import constants, masks, scores  # noqa: F401
from .block_mask import BlockMap, build_block_map, create_block_mask  # noqa: F401
from .flex_attention_dkv_kernel import flash_attention_bwd_dkv  # noqa: F401
from .flex_attention_dq_bwd import compute_delta, flex_attention_bwd_dq  # noqa: F401
from .flex_attention_kernel import _flex_attention_impl  # noqa: F401
from .flex_attention import flex_attention, flex_attention_bwd  # noqa: F401

__all__ = [
    "flex_attention", "flex_attention_bwd", "_flex_attention_impl", "flex_attention_bwd_dq", "flash_attention_bwd_dkv", "compute_delta",
    "BlockMap", "build_block_map", "create_block_mask", "masks", "scores", "constants",
]
