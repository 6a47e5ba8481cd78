"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same seeded inputs.

Tolerances (stated by the task for floating point): every one of O, dQ, dK, dV within max-abs 2e-2 and relative
L2 1e-2 of the fp32 oracle.  Mask compaction is integer work and must be bit-exact.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
REL_L2 = 1e-2


def _run_case(oracle, gpu, B, Hq, Hkv, Sq, Skv, qbs, kbs, mask, seed=0, peaky=False, check_bwd=True):
    import flex_block_attn_amd as fba

    q, k, v, do = oracle.seeded_qkv(B, Hq, Hkv, Sq, Skv, seed=seed, peaky=peaky)
    qb, kb, vb, dob = (t.to(torch.bfloat16) for t in (q, k, v, do))
    # the oracle sees exactly the values the kernels see (bf16-rounded), in fp32
    o_ref, lse_ref = oracle.c_attention_forward(qb, kb, vb, mask, qbs, kbs)
    qg, kg, vg = (t.to(gpu).requires_grad_(check_bwd) for t in (qb, kb, vb))
    o = fba.flex_block_attn_func(qg, kg, vg, qbs, kbs, mask.to(gpu))
    res = {"o": oracle.error_metrics(o.float(), o_ref)}
    if check_bwd:
        dq_ref, dk_ref, dv_ref = oracle.c_attention_backward(qb, kb, vb, o_ref, lse_ref, dob, mask, qbs, kbs)
        o.backward(dob.to(gpu))
        res["dq"] = oracle.error_metrics(qg.grad.float(), dq_ref)
        res["dk"] = oracle.error_metrics(kg.grad.float(), dk_ref)
        res["dv"] = oracle.error_metrics(vg.grad.float(), dv_ref)
    print(f"B{B} Hq{Hq} Hkv{Hkv} Sq{Sq} Skv{Skv} q{qbs} k{kbs}:", {n: (f"{a:.2e}", f"{r:.2e}") for n, (a, r) in res.items()}, flush=True)
    for name, (mabs, rel) in res.items():
        assert mabs <= MAX_ABS, f"{name}: max-abs {mabs} > {MAX_ABS}"
        assert rel <= REL_L2, f"{name}: rel-L2 {rel} > {REL_L2}"
    return res


def test_mask_compaction_bit_exact(oracle, gpu):
    import flex_block_attn_amd as fba
    from flex_block_attn_amd import masks

    cases = [
        masks.bernoulli_block_mask(4, 4, 0.5, 0),
        masks.bernoulli_block_mask(80, 80, 0.4, 1),
        masks.bernoulli_block_mask(540, 180, 0.1, 2),
        masks.bernoulli_block_mask(1, 1, 1.0, 3),
        masks.bernoulli_block_mask(65, 129, 0.5, 4),
        torch.zeros((7, 9), dtype=torch.bool),
        torch.ones((30, 30), dtype=torch.bool),
        masks.random_block_mask(1, 24, 80, 80, 32, 5),
        masks.random_block_mask(2, 3, 17, 70, 5, 6),
    ]
    for m in cases:
        lists = fba.compact_block_mask(m.to(gpu))
        ref = oracle.compact_lists(m)
        ref_c = oracle.c_compact_lists(m)
        for got, want, want_c, name in zip((lists.q_cnt, lists.q_idx, lists.k_cnt, lists.k_idx), ref, ref_c, ("q_cnt", "q_idx", "k_cnt", "k_idx")):
            assert (want == want_c).all()
            assert got.dtype == torch.int32
            assert (got.cpu().numpy() == want).all(), f"{name} differs for mask {tuple(m.shape)}"


def test_config1_cpu_reference_shape(oracle, gpu):
    """B=1, H=2, S=1536, block 384 (4x4 Bernoulli(0.5) mask with the diagonal forced on)."""
    from flex_block_attn_amd import masks

    _run_case(oracle, gpu, 1, 2, 2, 1536, 1536, 384, 384, masks.bernoulli_block_mask(4, 4, 0.5, 0))


def test_full_mask_small(oracle, gpu):
    _run_case(oracle, gpu, 1, 2, 2, 768, 768, 384, 384, torch.ones((2, 2), dtype=torch.bool))


def test_per_head_mask_and_q128(oracle, gpu):
    from flex_block_attn_amd import masks

    _run_case(oracle, gpu, 2, 3, 3, 768, 1152, 128, 384, masks.random_block_mask(2, 3, 6, 3, 2, 7))
