"""GPU parity at the full size of every benchmark configuration, number against number.

The product runs the whole configuration (all 24 heads, so that list rows, pair numbers and workspace offsets reach
their real magnitudes); single heads of the result, the first and the last, are then compared with the fp32 oracle
(`oracle.dense_attention_explicit` and its closed-form gradients) evaluated on the GPU on the same bf16 values and the
same mask, in chunks of query rows where a whole score matrix would not fit.  Chunking over query rows changes nothing
in the formula: O, LSE and dQ rows depend on their own query row only, dK and dV are sums over query rows.

Bounds as everywhere: max-abs 2e-2 and relative L2 1e-2, flat, for each of O, dQ, dK, dV.  The reference checks every
size of its sweeps the same way (benchmark/dynamic/random/scripts/random_fwd.py:186-200).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
REL_L2 = 1e-2


def _inputs(gpu, B, H, S, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return tuple(torch.randn((B, H, S, 128), generator=g).to(torch.bfloat16).to(gpu) for _ in range(4))


def _oracle_head(oracle, q, k, v, do, mask2d, qbs, kbs, chunk_blocks):
    """fp32 oracle for one head ([1, 1, S, 128] bf16 tensors on the GPU, mask [nQ, nK]), `chunk_blocks` query blocks at a
    time.  Returns fp32 (o, dq, dk, dv)."""
    Sq = q.shape[2]
    o = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    dq = torch.empty_like(o)
    dk = torch.zeros(k.shape, dtype=torch.float32, device=q.device)
    dv = torch.zeros_like(dk)
    rows = chunk_blocks * qbs
    for r0 in range(0, Sq, rows):
        r1 = min(Sq, r0 + rows)
        mc = mask2d[r0 // qbs: r1 // qbs]
        oc, lc = oracle.dense_attention_explicit(q[:, :, r0:r1], k, v, mc, qbs, kbs)
        dqc, dkc, dvc = oracle.dense_attention_backward_explicit(q[:, :, r0:r1], k, v, oc, lc, do[:, :, r0:r1], mc, qbs, kbs)
        o[:, :, r0:r1], dq[:, :, r0:r1] = oc, dqc
        dk += dkc
        dv += dvc
        del oc, lc, dqc, dkc, dvc
    return o, dq, dk, dv


def _compare(oracle, got, want, name, report):
    mabs, rel = oracle.error_metrics(got.float(), want)
    report[name] = (f"{mabs:.2e}", f"{rel:.2e}")
    assert mabs <= MAX_ABS, f"{name}: max-abs {mabs} > {MAX_ABS}"
    assert rel <= REL_L2, f"{name}: rel-L2 {rel} > {REL_L2}"


def _full_size_case(oracle, gpu, q, k, v, do, qbs, kbs, mask, heads, chunk_blocks, hand_over_modes=(None,)):
    import flex_block_attn_amd as fba

    lists = fba.lists_for(mask, qbs, kbs)
    o, lse = fba.forward_with_lists(q, k, v, qbs, kbs, lists)
    results = {}
    for mode in hand_over_modes:
        print(f"full-size parity: backward hand_over={mode}", flush=True)
        results[mode] = fba.backward_with_lists(q, k, v, o, lse, do, qbs, kbs, lists, hand_over=mode)
    torch.cuda.synchronize()
    for h in heads:
        m2 = mask if mask.dim() == 2 else mask[0, h]
        sl = slice(h, h + 1)
        o_ref, dq_ref, dk_ref, dv_ref = _oracle_head(oracle, q[:, sl], k[:, sl], v[:, sl], do[:, sl], m2, qbs, kbs, chunk_blocks)
        report = {}
        _compare(oracle, o[:, sl], o_ref, "o", report)
        for mode, (dq, dk, dv) in results.items():
            _compare(oracle, dq[:, sl], dq_ref, f"dq[{mode}]", report)
            _compare(oracle, dk[:, sl], dk_ref, f"dk[{mode}]", report)
            _compare(oracle, dv[:, sl], dv_ref, f"dv[{mode}]", report)
        print(f"    head {h}: {report}", flush=True)
        del o_ref, dq_ref, dk_ref, dv_ref
    return o, results


def test_random_sparse_full_size_against_oracle(oracle, gpu):
    """B1 H24 S30720 block 384, 32 of 80 key blocks per row, a mask per head: first and last head, the default backward,
    the whole-workspace hand-over and the recomputing backward."""
    from flex_block_attn_amd import masks

    q, k, v, do = _inputs(gpu, 1, 24, 30720, 31)
    m = masks.random_block_mask(1, 24, 80, 80, 32, 32).to(gpu)
    _full_size_case(oracle, gpu, q, k, v, do, 384, 384, m, heads=(0, 23), chunk_blocks=20, hand_over_modes=(None, True, False))


def test_full_attention_full_size_against_oracle(oracle, gpu):
    """B1 H24 S11520 block 384, all-ones 30 x 30 mask shared by the heads."""
    from flex_block_attn_amd import masks

    q, k, v, do = _inputs(gpu, 1, 24, 11520, 33)
    m = masks.full_block_mask(30, 30).to(gpu)
    _full_size_case(oracle, gpu, q, k, v, do, 384, 384, m, heads=(0, 23), chunk_blocks=30)


def test_sliding_tile_full_size_against_oracle(oracle, gpu):
    """B1 H24 S115200 = 300 tiles of 384 tokens, clamped 3x3x3 window, one mask for all heads; last head."""
    from flex_block_attn_amd import masks

    q, k, v, do = _inputs(gpu, 1, 24, 115200, 35)
    m = masks.sta_3d_block_mask((5, 6, 10), (3, 3, 3), clamp=True).to(gpu)
    _full_size_case(oracle, gpu, q, k, v, do, 384, 384, m, heads=(23,), chunk_blocks=10)


def test_asymmetric_score_mask_full_size_against_oracle(oracle, gpu):
    """B1 H24 S69120, q block 128 x k block 384, score-driven mask built on the GPU (band, sink, top-16); first and last
    head against the oracle under that same mask."""
    import flex_block_attn_amd as fba

    q, k, v, do = _inputs(gpu, 1, 24, 69120, 37)
    m = fba.create_ssta_mask(q, k, 128, 384, topk=16, band=1, sink_blocks=1)
    _full_size_case(oracle, gpu, q, k, v, do, 128, 384, m, heads=(0, 23), chunk_blocks=54)


def test_fine_blocks_full_size_against_oracle(oracle, gpu):
    """Tile lists at full size: B1 H24 S30720, independent 64 x 64 blocks, 40 % kept, a mask per head; the last head's
    tile pairs sit beyond 2^31 bytes in the dS workspace."""
    nb = 30720 // 64
    q, k, v, do = _inputs(gpu, 1, 24, 30720, 39)
    m = torch.rand((1, 24, nb, nb), generator=torch.Generator().manual_seed(40)) < 0.4
    m[..., torch.arange(nb), torch.arange(nb)] = True
    m = m.to(gpu)
    _full_size_case(oracle, gpu, q, k, v, do, 64, 64, m, heads=(23,), chunk_blocks=120, hand_over_modes=(None, False))


def test_deterministic_at_full_size(gpu):
    """B1 H24 S30720 block 384 on the hand-over path, twice: every output bit-equal, at a size where work-groups compete
    for compute units and the order in which they run differs between launches."""
    import flex_block_attn_amd as fba
    from flex_block_attn_amd import masks

    q, k, v, do = _inputs(gpu, 1, 24, 30720, 41)
    lists = fba.lists_for(masks.random_block_mask(1, 24, 80, 80, 32, 42).to(gpu), 384, 384)
    runs = []
    for _ in range(2):
        o, lse = fba.forward_with_lists(q, k, v, 384, 384, lists)
        runs.append((o, lse) + tuple(fba.backward_with_lists(q, k, v, o, lse, do, 384, 384, lists, hand_over=True)))
    for a, b in zip(*runs):
        assert torch.equal(a, b)
