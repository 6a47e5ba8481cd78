"""The helpers the reference's benchmark scripts import for this operator (benchmark/utils/utils.py:31-119, :294-297),
under the same module path, backed by flex_block_attn_amd.  Helpers of other libraries that module also holds
(flex_attention, MagiAttention, FlashAttention, SpargeAttn wrappers) have no counterpart here."""
import torch

from flex_block_attn_amd import flex_block_attn_func
from flex_block_attn_amd.benchmark import append_to_csv
from flex_block_attn_amd.masks import (
    create_sparse_mask,
    create_torch_mask,
    generate_selected_blocks,
    generate_swa_selected_blocks,
)

__all__ = [
    "append_to_csv",
    "generate_input",
    "generate_selected_blocks",
    "generate_swa_selected_blocks",
    "create_sparse_mask",
    "create_torch_mask",
    "ptm_sparse_attn",
]


def generate_input(batch_size, seq_len, num_heads, head_dim, device):
    """query, key, value ~ N(0,1), bf16, (batch, seq, heads, head_dim) with requires_grad (utils.py:61-67); the scripts
    transpose them to (batch, heads, seq, head_dim) before the call."""
    shape = (batch_size, seq_len, num_heads, head_dim)
    return tuple(torch.randn(shape, dtype=torch.bfloat16, device=device, requires_grad=True) for _ in range(3))


def ptm_sparse_attn(query, key, value, block_size, block_mask):
    """utils.py:294-297: the operator with equal query and key block sizes."""
    return flex_block_attn_func(query, key, value, block_size, block_size, block_mask)
