"""Module-path alias of the reference's flex_block_attn/flex_block_attn_interface.py (its package __init__ imports the
operator from here, flex_block_attn/__init__.py:1-5): the same four names, backed by the MI355X implementation."""
from flex_block_attn_amd.interface import (  # noqa: F401
    FlexBlockAttnFunc,
    _flex_block_attn_backward,
    _flex_block_attn_forward,
    flex_block_attn_func,
)
