"""Import-name alias: `from flex_block_attn import flex_block_attn_func` resolves to the MI355X implementation."""
from .flex_block_attn_interface import _flex_block_attn_backward, _flex_block_attn_forward, flex_block_attn_func  # noqa: F401
