"""GPU parity of the caller-side steps for video models: block means, score-driven masks, tile permutation.

Block means and scores are floating point: the kernel sums in fp32 in its own order, the oracle in float64, so a
selected block may differ from the oracle's only where two scores of a row are closer than the fp32 rounding of the
sums (bound written in `_check_ssta`); everything else about the mask, and the whole permutation, is bit-exact.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

MEAN_TOL = 2e-6   # |mean_gpu - mean_fp64| for N(0,1) data: fp32 accumulation over at most 384 rows
SCORE_TOL = 1e-5  # scores of unit-variance means over 128 dims: |<q,k>_fp32 - <q,k>_fp64| stays far below this


def _check_ssta(oracle, got, scores, q_block, kv_block, topk, band, sink, base=None):
    """`got` must equal the oracle's mask except where the k-th and (k+1)-th best scores of the row are within
    SCORE_TOL; in such rows the selection may swap those near-equal blocks, nothing else."""
    want = oracle.ssta_mask(scores, q_block, kv_block, topk, band, sink, base)
    got = got.cpu()
    diff = got != want
    if not diff.any():
        return 0
    nK = scores.shape[-1]
    srt = scores.sort(dim=-1, descending=True).values
    kth, nxt = srt[..., min(topk, nK) - 1], srt[..., min(topk, nK - 1)]
    rows = diff.any(-1)
    assert ((kth - nxt)[rows].abs() <= SCORE_TOL).all(), "mask differs in a row without a near-tie"
    # a swapped row still holds as many selected blocks as the oracle's and only differs at near-tied scores
    for b, h, i in rows.nonzero().tolist():
        js = diff[b, h, i].nonzero().flatten()
        assert ((scores[b, h, i, js] - kth[b, h, i]).abs() <= SCORE_TOL).all()
    return int(rows.sum())


@pytest.mark.parametrize("block,S", [(16, 256), (128, 1024), (384, 1536), (80, 640), (48, 96)])
def test_block_mean(oracle, gpu, block, S):
    import flex_block_attn_amd as fba

    x = torch.randn((2, 3, S, 128), generator=torch.Generator().manual_seed(block)).to(torch.bfloat16)
    got = fba.block_mean(x.to(gpu), block)
    want = oracle.block_mean(x, block)
    assert got.dtype == torch.float32 and got.shape == want.shape
    assert (got.cpu().double() - want).abs().max().item() <= MEAN_TOL
    assert torch.equal(got, fba.block_mean(x.to(gpu), block))


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Skv,qbs,kbs,topk,band,sink", [
    (1, 2, 2, 2048, 2304, 128, 384, 3, 1, 1),      # the q128 / k384 asymmetric shape, scaled down
    (2, 4, 2, 1024, 1024, 128, 128, 4, 1, 1),      # grouped kv heads
    (1, 1, 1, 384 * 70, 384 * 70, 384, 384, 16, 1, 1),   # more than one 64-block chunk of key blocks
    (1, 2, 1, 256, 64 * 200, 128, 64, 16, 0, 0),   # 200 key blocks, moba style
    (1, 1, 1, 1152, 64 * 1500, 128, 64, 16, 1, 1), # 1500 key blocks: the kernel that ranks up to 4096
    (1, 1, 1, 256, 64 * 4096, 128, 64, 7, 0, 1),   # the largest number of key blocks it takes
    (1, 1, 1, 512, 512, 128, 128, 9, -1, 0),       # topk beyond the number of key blocks
    (1, 1, 1, 1152, 384, 128, 384, 0, 1, 2),       # nothing ranked: band and sink only
])
def test_ssta_mask(oracle, gpu, B, Hq, Hkv, Sq, Skv, qbs, kbs, topk, band, sink):
    import flex_block_attn_amd as fba

    g = torch.Generator().manual_seed(Sq + Skv + topk)
    q = torch.randn((B, Hq, Sq, 128), generator=g).to(torch.bfloat16)
    k = torch.randn((B, Hkv, Skv, 128), generator=g).to(torch.bfloat16)
    got = fba.create_ssta_mask(q.to(gpu), k.to(gpu), qbs, kbs, topk=topk, band=band, sink_blocks=sink)
    assert got.dtype == torch.bool and tuple(got.shape) == (B, Hq, Sq // qbs, Skv // kbs)
    scores = oracle.ssta_scores(oracle.block_mean(q, qbs), oracle.block_mean(k, kbs))
    swapped = _check_ssta(oracle, got, scores, qbs, kbs, topk, band, sink)
    print(f"    ssta mask {tuple(got.shape)}: {swapped} rows with near-tied scores", flush=True)


def test_ssta_mask_exact_ties_and_base_mask(oracle, gpu):
    """Scores that are exactly equal (identical key blocks) must resolve to the lower index, as the definition says.
    Small integer means keep every dot product exact in fp32 and in the oracle's float64, whatever the summation order."""
    from flex_block_attn_amd import video

    g = torch.Generator().manual_seed(3)
    qm = torch.randint(-4, 5, (1, 2, 6, 128), generator=g).float()
    km = torch.randint(-4, 5, (1, 2, 5, 128), generator=g).float()[:, :, [0, 1, 1, 0, 1]].contiguous()  # blocks 1,2,4 and 0,3 identical
    base = torch.rand((6, 5), generator=g) < 0.3
    got = video.ssta_mask_from_means(qm.to(gpu), km.to(gpu), 128, 128, topk=2, band=-1, sink_blocks=0, base_mask=base.to(gpu))
    sc = oracle.ssta_scores(qm, km)
    want = oracle.ssta_mask(sc, 128, 128, 2, -1, 0, base)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("grid,tile", [((6, 8, 16), (6, 8, 8)), ((12, 16, 8), (6, 8, 8)), ((4, 6, 4), (2, 3, 2)), ((3, 5, 7), (1, 1, 1))])
def test_tile_permutation_bit_exact(oracle, gpu, grid, tile):
    import flex_block_attn_amd as fba

    S = grid[0] * grid[1] * grid[2]
    x = torch.randn((2, 3, S, 128), generator=torch.Generator().manual_seed(S)).to(torch.bfloat16)
    idx = oracle.tile_order(grid, tile)
    tiled = fba.tile_tokens(x.to(gpu), grid, tile)
    assert torch.equal(tiled.cpu(), x[:, :, idx])
    assert torch.equal(fba.untile_tokens(tiled, grid, tile).cpu(), x)


def test_ssta_3d_attention_end_to_end(oracle, gpu):
    """Raster-order latent -> tiles -> mask -> attention -> raster order, against the oracle's dense attention driven by
    the mask the GPU built (the mask itself is checked above), including gradients through the permutations."""
    import flex_block_attn_amd as fba

    grid, tile, window, topk = (12, 8, 16), (6, 8, 8), (1, 1, 1), 2
    S, blk = 12 * 8 * 16, 384
    q, k, v, do = oracle.seeded_qkv(1, 2, 2, S, S, seed=77)
    qb, kb, vb, dob = (t.to(torch.bfloat16) for t in (q, k, v, do))
    qg, kg, vg = (t.to(gpu).requires_grad_(True) for t in (qb, kb, vb))
    out = fba.ssta_3d_attention(qg, kg, vg, grid, tile, window=window, topk=topk, sink_blocks=1)
    out.backward(dob.to(gpu))
    idx = oracle.tile_order(grid, tile)
    mask = fba.create_ssta_3d_mask(qb[:, :, idx].to(gpu), kb[:, :, idx].to(gpu), grid, tile, window, topk, 1).cpu()
    assert mask.shape == (1, 2, 4, 4) and mask[..., 0].all() and mask.diagonal(dim1=-2, dim2=-1).all()
    assert (mask.sum(-1) >= topk).all()
    qt, kt, vt, dot = (t[:, :, idx].contiguous() for t in (qb, kb, vb, dob))
    o_ref, lse_ref = oracle.c_attention_forward(qt, kt, vt, mask, blk, blk)
    g_ref = oracle.c_attention_backward(qt, kt, vt, o_ref, lse_ref, dot, mask, blk, blk)
    inv = torch.empty_like(idx)
    inv[idx] = torch.arange(S)
    for name, got, want in (("o", out, o_ref), ("dq", qg.grad, g_ref[0]), ("dk", kg.grad, g_ref[1]), ("dv", vg.grad, g_ref[2])):
        mabs, rel = oracle.error_metrics(got.float(), want[:, :, inv])
        assert mabs <= 2e-2 and rel <= 1e-2, (name, mabs, rel)


@pytest.mark.parametrize("grid,tile,window", [((6, 16, 32), (2, 8, 8), (3, 1, 3)), ((4, 24, 16), (2, 8, 8), (1, 3, 1))])
def test_sliding_tile_attention_on_raster_latent(oracle, gpu, grid, tile, window):
    """ssta_3d_attention with the score-driven part switched off (topk 0, no sink) is pure sliding-tile attention.  On a
    latent in raster order it must equal dense attention under a TOKEN mask built from token coordinates alone
    (oracle.sta_token_mask): that pins the mask builder's window and axis order and its agreement with the tile
    permutation's enumeration, neither of which the mask the GPU built is consulted for.  Asymmetric tile grids, so a
    swapped axis fails."""
    import flex_block_attn_amd as fba

    S = grid[0] * grid[1] * grid[2]
    q, k, v, do = oracle.seeded_qkv(1, 2, 2, S, S, seed=S + window[0])
    qb, kb, vb, dob = (t.to(torch.bfloat16) for t in (q, k, v, do))
    token_mask = oracle.sta_token_mask(grid, tile, window, clamp=True)
    o_ref, lse_ref = oracle.dense_attention_explicit(qb, kb, vb, token_mask, 1, 1)
    g_ref = oracle.dense_attention_backward_explicit(qb, kb, vb, o_ref, lse_ref, dob, token_mask, 1, 1)
    qg, kg, vg = (t.to(gpu).requires_grad_(True) for t in (qb, kb, vb))
    out = fba.ssta_3d_attention(qg, kg, vg, grid, tile, window=window, topk=0, sink_blocks=0)
    out.backward(dob.to(gpu))
    for name, got, want in (("o", out, o_ref), ("dq", qg.grad, g_ref[0]), ("dk", kg.grad, g_ref[1]), ("dv", vg.grad, g_ref[2])):
        mabs, rel = oracle.error_metrics(got.float(), want)
        assert mabs <= 2e-2 and rel <= 1e-2, (name, mabs, rel)
