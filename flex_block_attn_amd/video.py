"""Caller-side steps of the operator in video models, on the GPU: score-driven ("SSTA" style) block masks and the tile
permutation of a latent grid.

The reference names these (create_sta_3d_mask, create_ssta_3d_mask, create_moba_3d_mask, ssta_3d_attention) but has
not released them (flex_block_attn/__init__.py:7-12, README.md:54-55); the definitions below are this package's own and
are stated in include/fba.h.  The static sliding-tile mask is `masks.sta_3d_block_mask`.
"""
import torch

from . import _lib
from .interface import HEAD_DIM, _ptr, _require_device, _stream


def _check_seq(x, name):
    _require_device(x, name)
    if x.dtype != torch.bfloat16 or x.dim() != 4 or x.shape[-1] != HEAD_DIM:
        raise ValueError(f"{name} must be a (batch, heads, seq, {HEAD_DIM}) bfloat16 tensor, got {tuple(x.shape)} {x.dtype}")
    return x.contiguous()


def block_mean(x, block_size):
    """(B, H, S, 128) bf16 -> (B, H, S / block_size, 128) fp32: the mean of every block of `block_size` rows."""
    x = _check_seq(x, "x")
    B, H, S, _ = x.shape
    if block_size <= 0 or S % block_size:
        raise ValueError(f"seq_len ({S}) must be divisible by block_size ({block_size})")
    out = torch.empty((B, H, S // block_size, HEAD_DIM), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.call("fba_block_mean", _ptr(x), _ptr(out), B * H, S, block_size, HEAD_DIM, _stream())
    return out


def ssta_mask_from_means(q_mean, k_mean, q_block_size, kv_block_size, topk=16, band=1, sink_blocks=1, base_mask=None):
    """Block means (B, Hq, nQ, 128), (B, Hkv, nK, 128) fp32 -> bool mask (B, Hq, nQ, nK)."""
    _require_device(q_mean, "q_mean")
    _require_device(k_mean, "k_mean")
    if q_mean.dtype != torch.float32 or k_mean.dtype != torch.float32 or q_mean.dim() != 4 or k_mean.dim() != 4:
        raise ValueError("q_mean and k_mean must be 4-D float32 tensors")
    if q_mean.shape[-1] != HEAD_DIM or k_mean.shape[-1] != HEAD_DIM or q_mean.shape[0] != k_mean.shape[0]:
        raise ValueError("q_mean and k_mean must be (B, H, blocks, 128) with equal batch")
    q_mean, k_mean = q_mean.contiguous(), k_mean.contiguous()
    B, Hq, nQ, _ = q_mean.shape
    Hkv, nK = k_mean.shape[1], k_mean.shape[2]
    if base_mask is not None:
        _require_device(base_mask, "base_mask")
        if base_mask.dtype != torch.bool or tuple(base_mask.shape) != (nQ, nK):
            raise ValueError(f"base_mask must be a bool tensor of shape ({nQ}, {nK})")
        base_mask = base_mask.contiguous()
    mask = torch.empty((B, Hq, nQ, nK), dtype=torch.bool, device=q_mean.device)
    with torch.cuda.device(q_mean.device):
        _lib.call("fba_ssta_mask", _ptr(q_mean), _ptr(k_mean), _ptr(base_mask) if base_mask is not None else None, _ptr(mask), B, Hq, Hkv, nQ, nK, q_block_size, kv_block_size,
                  topk, band, sink_blocks, _stream())
    return mask


def create_ssta_mask(q, k, q_block_size, kv_block_size, topk=16, band=1, sink_blocks=1, base_mask=None):
    """Block mask (B, Hq, nQ, nK), bool, for `flex_block_attn_func(q, k, v, q_block_size, kv_block_size, mask)`:
    query block i keeps the key block that holds its first row and its `band` neighbours on either side, the first
    `sink_blocks` key blocks, the `topk` key blocks with the largest <mean(q block i), mean(k block j)>, and whatever
    the optional 2-D `base_mask` (nQ, nK) selects (band=-1 switches the band off)."""
    return ssta_mask_from_means(block_mean(q, q_block_size), block_mean(k, kv_block_size), q_block_size, kv_block_size,
                                topk, band, sink_blocks, base_mask)


def create_moba_mask(q, k, q_block_size, kv_block_size, topk):
    """Top-k block selection alone (no band, no sink), plus the query block's own key block."""
    return create_ssta_mask(q, k, q_block_size, kv_block_size, topk=topk, band=0, sink_blocks=0)


def _permute(x, grid, tile, to_tiles):
    x = _check_seq(x, "x")
    B, H, S, _ = x.shape
    T, Hh, W = grid
    if T * Hh * W != S:
        raise ValueError(f"grid {tuple(grid)} does not have seq_len ({S}) tokens")
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _lib.call("fba_tile_permute", _ptr(x), _ptr(out), B * H, T, Hh, W, tile[0], tile[1], tile[2], HEAD_DIM, int(to_tiles), _stream())
    return out


class _TilePermute(torch.autograd.Function):
    """A permutation of token rows: the gradient is the inverse permutation of the incoming gradient."""

    @staticmethod
    def forward(ctx, x, grid, tile, to_tiles):
        ctx.args = (tuple(grid), tuple(tile), to_tiles)
        return _permute(x, grid, tile, to_tiles)

    @staticmethod
    def backward(ctx, g):
        grid, tile, to_tiles = ctx.args
        return _permute(g.to(torch.bfloat16), grid, tile, not to_tiles), None, None, None


def tile_tokens(x, grid, tile=(6, 8, 8)):
    """(B, H, T*Hh*W, 128) in raster order of the latent grid -> tile order: the tokens of each `tile` become one
    contiguous block (384 tokens for 6x8x8), tiles in raster order of the tile grid."""
    return _TilePermute.apply(x, grid, tile, True)


def untile_tokens(x, grid, tile=(6, 8, 8)):
    """Inverse of `tile_tokens`."""
    return _TilePermute.apply(x, grid, tile, False)


def create_sta_3d_mask(tiles, window, device=None, clamp=True):
    """Static sliding-tile mask over a (t, h, w) grid of tiles: `masks.sta_3d_block_mask`, moved to `device`."""
    from . import masks

    m = masks.sta_3d_block_mask(tiles, window, clamp=clamp)
    return m if device is None else m.to(device)


def create_ssta_3d_mask(q, k, grid, tile=(6, 8, 8), window=(3, 3, 3), topk=16, sink_blocks=1):
    """Sliding-tile window united with score-selected tiles, for q, k already in tile order: bool (B, H, n, n) with
    n = number of tiles."""
    tiles = tuple(g // t for g, t in zip(grid, tile))
    block = tile[0] * tile[1] * tile[2]
    base = create_sta_3d_mask(tiles, window, device=q.device)
    return create_ssta_mask(q, k, block, block, topk=topk, band=-1, sink_blocks=sink_blocks, base_mask=base)


def create_moba_3d_mask(q, k, grid, tile=(6, 8, 8), topk=16):
    """Score-selected tiles plus the query tile itself, for q, k in tile order."""
    block = tile[0] * tile[1] * tile[2]
    return create_moba_mask(q, k, block, block, topk)


def ssta_3d_attention(q, k, v, grid, tile=(6, 8, 8), window=(3, 3, 3), topk=16, sink_blocks=1):
    """Attention over a video latent in raster order: tokens go to tile order, every query tile attends to its
    sliding-tile window, to the sink tiles and to its top-k tiles by mean scores, and the output returns to raster
    order.  Differentiable in q, k, v; the mask is a constant of the backward pass."""
    from .interface import flex_block_attn_func

    block = tile[0] * tile[1] * tile[2]
    qt, kt, vt = (tile_tokens(x, grid, tile) for x in (q, k, v))
    with torch.no_grad():
        mask = create_ssta_3d_mask(qt.detach(), kt.detach(), grid, tile, window, topk, sink_blocks)
    return untile_tokens(flex_block_attn_func(qt, kt, vt, block, block, mask), grid, tile)
