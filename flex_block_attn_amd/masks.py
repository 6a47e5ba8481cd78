"""Block-mask helpers.

The first group keeps the names and argument order of the reference's caller-side helpers
(benchmark/utils/utils.py:69-119) so that code written against them runs unchanged.  The second group builds the
masks of the benchmark configurations directly as tensors (no Python loop over blocks).
"""
import itertools
import random

import numpy as np
import torch


# ---------------------------------------------------------------------------------------------------------------
# drop-in helpers
# ---------------------------------------------------------------------------------------------------------------
def generate_selected_blocks(Q, block_size, percentage, seed=None):
    """Per block row, `int(block_num * percentage)` distinct random columns, as (row, col) pairs
    (benchmark/utils/utils.py:69-83; there the draw is unseeded, here `seed` makes it reproducible)."""
    block_num = int(Q.size(2) / block_size)
    keep = int(block_num * percentage)
    rng = random.Random(seed) if seed is not None else random
    cols = list(range(block_num))
    selected = []
    for i in range(block_num):
        for j in rng.sample(cols, keep):
            selected.append((i, j))
    return selected


def generate_swa_selected_blocks(Q, block_size, window_size):
    """Block sliding window |i - j| < window_size (benchmark/utils/utils.py:85-92)."""
    block_num = Q.size(2) // block_size
    return [(i, j) for i in range(block_num) for j in range(max(0, i + 1 - window_size), min(block_num, i + window_size))]


def create_sparse_mask(Q, block_size, selected_blocks):
    """(row, col) pairs -> bool [block_num, block_num] on Q's device (benchmark/utils/utils.py:94-103)."""
    block_num = int(Q.size(2) / block_size)
    m = np.zeros((block_num, block_num), dtype=bool)
    n = len(selected_blocks)
    if n:
        # flattening the pairs through an iterator is several times faster than np.asarray on a list of tuples
        flat = np.fromiter(itertools.chain.from_iterable(selected_blocks), dtype=np.int64, count=2 * n)
        m[flat[0::2], flat[1::2]] = True
    return torch.from_numpy(m).to(Q.device)


def create_torch_mask(Q, block_size, selected_blocks):
    """(row, col) pairs -> dense token-level bool [seq, seq] (benchmark/utils/utils.py:105-119)."""
    return expand_block_mask(create_sparse_mask(Q, block_size, selected_blocks), block_size, block_size)


# ---------------------------------------------------------------------------------------------------------------
# tensor-level builders
# ---------------------------------------------------------------------------------------------------------------
def expand_block_mask(block_mask, q_block_size, kv_block_size):
    """Block mask [..., nQ, nK] -> token mask [..., nQ*q_block, nK*kv_block]."""
    return block_mask.repeat_interleave(q_block_size, dim=-2).repeat_interleave(kv_block_size, dim=-1)


def full_block_mask(nQ, nK, device="cpu"):
    return torch.ones((nQ, nK), dtype=torch.bool, device=device)


def random_block_mask(B, H, nQ, nK, keep, seed, device="cpu", force_diagonal=True):
    """Independent mask per (b, h): every query-block row keeps exactly `keep` key blocks, drawn without replacement
    from a seeded CPU generator; with `force_diagonal` the block nearest the diagonal is one of them."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    scores = torch.rand((B, H, nQ, nK), generator=g)
    if force_diagonal:
        diag = (torch.arange(nQ) * nK) // nQ
        scores[:, :, torch.arange(nQ), diag] = 2.0
    top = scores.topk(keep, dim=-1).indices
    m = torch.zeros((B, H, nQ, nK), dtype=torch.bool)
    m.scatter_(-1, top, True)
    return m.to(device)


def bernoulli_block_mask(nQ, nK, p, seed, device="cpu", force_diagonal=True):
    """2-D mask with i.i.d. Bernoulli(p) entries from a seeded CPU generator, diagonal forced on."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    m = torch.rand((nQ, nK), generator=g) < p
    if force_diagonal:
        diag = (torch.arange(nQ) * nK) // nQ
        m[torch.arange(nQ), diag] = True
    return m.to(device)


def swa_block_mask(nQ, nK, window, device="cpu"):
    """Block sliding window |i - j| < window."""
    i = torch.arange(nQ, device=device)[:, None]
    j = torch.arange(nK, device=device)[None, :]
    return (i - j).abs() < window


def sta_3d_block_mask(tiles_thw, window_thw, device="cpu", clamp=True):
    """Sliding-tile attention over a 3-D grid of tiles (each tile = one attention block).

    tiles_thw: number of tiles along (T, H, W); window_thw: odd neighbourhood extents in tiles.  With `clamp` the
    window of a border tile is shifted inwards so that every query tile sees the same number of key tiles;
    otherwise it is clipped at the border.  Returns bool [n_tiles, n_tiles], tiles enumerated T-major, W-minor.
    """
    nt, nh, nw = tiles_thw
    wt, wh, ww = window_thw
    per_axis = []
    for n, w in ((nt, wt), (nh, wh), (nw, ww)):
        c = torch.arange(n, device=device)
        if clamp:
            c = c.clamp(min(w // 2, n - 1), max(n - 1 - w // 2, 0))
        per_axis.append((c[:, None] - torch.arange(n, device=device)[None, :]).abs() <= w // 2)
    mt, mh, mw = per_axis
    m = mt[:, None, None, :, None, None] & mh[None, :, None, None, :, None] & mw[None, None, :, None, None, :]
    n = nt * nh * nw
    return m.reshape(n, n)
