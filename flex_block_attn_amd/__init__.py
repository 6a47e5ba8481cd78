"""Block-sparse attention for AMD MI355X (gfx950): hand-written HIP kernels behind the flex-block-attn operator API."""
from .interface import (
    BlockLists,
    FlexBlockAttnFunc,
    _flex_block_attn_backward,
    _flex_block_attn_forward,
    backward_with_lists,
    compact_block_mask,
    flex_block_attn_func,
    forward_with_lists,
    lists_for,
    number_pairs,
    tile_block_mask,
)
from . import masks, video
from .video import (
    block_mean,
    create_moba_3d_mask,
    create_ssta_3d_mask,
    create_ssta_mask,
    create_sta_3d_mask,
    ssta_3d_attention,
    tile_tokens,
    untile_tokens,
)

__all__ = [
    "flex_block_attn_func",
    "_flex_block_attn_forward",
    "_flex_block_attn_backward",
    "FlexBlockAttnFunc",
    "BlockLists",
    "compact_block_mask",
    "forward_with_lists",
    "backward_with_lists",
    "lists_for",
    "number_pairs",
    "tile_block_mask",
    "masks",
    "video",
    "block_mean",
    "create_ssta_mask",
    "create_sta_3d_mask",
    "create_ssta_3d_mask",
    "create_moba_3d_mask",
    "ssta_3d_attention",
    "tile_tokens",
    "untile_tokens",
]
