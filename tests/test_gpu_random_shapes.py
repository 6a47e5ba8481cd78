"""Seeded random shapes, block sizes and masks: every kernel path against the oracle's explicit dense formula.

The formula (oracle.dense_attention_explicit / dense_attention_backward_explicit, fp32) is evaluated on the GPU by torch so
that many cases run in seconds; the same functions are pinned on the CPU by tests/test_oracle.py."""
import math
import os
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ABS, REL_L2 = 2e-2, 1e-2  # the operator's parity bar for N(0,1) inputs


def _draw_case(rng):
    """(B, Hq, Hkv, S, q_block, k_block) with S a common multiple of both blocks and of 128, at most 3072."""
    while True:
        qbs = rng.choice([128, 128, 256, 384, 384, 64, 32, 16])
        kbs = rng.choice([128, 384, 256] if qbs % 128 == 0 else [64, 128, 192])
        if qbs % 128 == 0 and rng.random() < 0.3:
            kbs = rng.choice([64, 192])  # tile lists through the key side
        if qbs % kbs and kbs % qbs:
            continue
        lcm = qbs * kbs // math.gcd(qbs, kbs)
        lcm = lcm * 128 // math.gcd(lcm, 128)
        if lcm > 3072:
            continue
        S = lcm * rng.randint(1, max(1, 1536 // lcm))
        Hkv = rng.choice([1, 2, 3])
        return rng.choice([1, 1, 2]), Hkv * rng.choice([1, 1, 2]), Hkv, S, qbs, kbs


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_against_the_dense_formula(oracle, gpu, seed):
    """Twelve cases per seed: block lists and tile lists, grouped kv heads, 2-D and per-head masks with an empty query
    row and an unselected key column thrown in, one in three with q scaled by 3 (peaked softmax).  Forward and both
    backward paths against the formula; dK / dV bit-equal between the two paths; on block lists the 32-key dK/dV kernel
    bit-equal to the default one."""
    import flex_block_attn_amd as fba

    rng = random.Random(1000 + seed)
    for case in range(12):
        B, Hq, Hkv, S, qbs, kbs = _draw_case(rng)
        nQ, nK = S // qbs, S // kbs
        density = rng.choice([0.15, 0.4, 0.7, 1.0])
        g = torch.Generator().manual_seed(rng.randint(0, 1 << 30))
        m = torch.rand((nQ, nK) if rng.random() < 0.3 else (B, Hq, nQ, nK), generator=g) < density
        if rng.random() < 0.5 and nQ > 1:
            m[..., rng.randrange(nQ), :] = False
        if rng.random() < 0.5 and nK > 1:
            m[..., :, rng.randrange(nK)] = False
        scale = rng.choice([1.0, 1.0, 3.0])
        q = (torch.randn((B, Hq, S, 128), generator=g) * scale).to(torch.bfloat16).to(gpu)
        do = torch.randn((B, Hq, S, 128), generator=g).to(torch.bfloat16).to(gpu)
        k, v = (torch.randn((B, Hkv, S, 128), generator=g).to(torch.bfloat16).to(gpu) for _ in range(2))
        md = m.to(gpu)
        tag = f"seed {seed} case {case}: B{B} Hq{Hq} Hkv{Hkv} S{S} q{qbs} k{kbs} mask {m.dim()}-D density {density} q x {scale}"
        print(tag, flush=True)
        o_ref, lse_ref = oracle.dense_attention_explicit(q, k, v, md, qbs, kbs)
        g_ref = oracle.dense_attention_backward_explicit(q, k, v, o_ref, lse_ref, do, md, qbs, kbs)
        lists = fba.lists_for(md, qbs, kbs)
        o, lse = fba.forward_with_lists(q, k, v, qbs, kbs, lists)
        grads = {ho: fba.backward_with_lists(q, k, v, o, lse, do, qbs, kbs, lists, hand_over=ho) for ho in (False, True)}
        for ho in (False, True):
            for name, got, want in zip(("o", "dq", "dk", "dv"), (o,) + tuple(grads[ho]), (o_ref,) + tuple(g_ref)):
                mabs, rel = oracle.error_metrics(got.float(), want)
                bound = MAX_ABS * max(1.0, float(want.abs().max()))  # results beyond unit scale: bf16 rounding alone is 2^-9 relative
                assert mabs <= bound and rel <= REL_L2, (tag, name, "hand-over" if ho else "recompute", mabs, rel)
        assert torch.equal(grads[False][1], grads[True][1]) and torch.equal(grads[False][2], grads[True][2]), tag
        if not lists.tiled:
            os.environ["FBA_DKDV_KEYS_PER_WAVE"] = "32"
            try:
                other = fba.backward_with_lists(q, k, v, o, lse, do, qbs, kbs, lists, hand_over=True)
            finally:
                os.environ.pop("FBA_DKDV_KEYS_PER_WAVE")
            assert all(torch.equal(a, b) for a, b in zip(other, grads[True])), (tag, "32-key and 64-key dK/dV kernels differ")
