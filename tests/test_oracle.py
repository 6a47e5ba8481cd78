"""Pins the CPU oracle (oracle/attn_oracle.py, oracle/attn_ref.c) before anything is compared against it.

The reference holds no golden vectors for this path; its one known-answer relation is "equals
F.scaled_dot_product_attention on the dense expanded mask" (test/test_flex_block_attn.py:48-51, :139).  The checks
below are chosen so that a plausible mistake fails one of them: three independent restatements must agree; special
masks must reduce to textbook attention; tiny cases are brute-forced with Python loops; gradients are checked against
fp64 finite differences and against identities that a dropped term or a transposed operand breaks.
"""
import math
import os

import numpy as np
import pytest
import torch

TOL = 2e-5  # fp32 agreement between restatements


def _mask(kind, nQ, nK, seed=0, B=1, H=1):
    g = torch.Generator(device="cpu").manual_seed(seed)
    if kind == "full":
        return torch.ones((nQ, nK), dtype=torch.bool)
    if kind == "diag":
        return torch.eye(nQ, nK, dtype=torch.bool)
    if kind == "rand2d":
        m = torch.rand((nQ, nK), generator=g) < 0.5
        m[torch.arange(nQ), (torch.arange(nQ) * nK) // nQ] = True
        return m
    if kind == "rand4d":
        m = torch.rand((B, H, nQ, nK), generator=g) < 0.5
        m[..., torch.arange(nQ), (torch.arange(nQ) * nK) // nQ] = True
        return m
    raise ValueError(kind)


CASES = [
    # B, Hq, Hkv, Sq, Skv, qbs, kbs, mask kind
    (1, 2, 2, 64, 64, 16, 16, "rand2d"),
    (2, 2, 2, 64, 96, 16, 32, "rand4d"),
    (1, 4, 2, 32, 64, 16, 16, "rand4d"),  # grouped-query heads
    (1, 1, 1, 48, 48, 16, 16, "full"),
]


@pytest.mark.parametrize("case", CASES)
def test_three_restatements_agree(oracle, case):
    B, Hq, Hkv, Sq, Skv, qbs, kbs, kind = case
    q, k, v, do = oracle.seeded_qkv(B, Hq, Hkv, Sq, Skv, D=32, seed=1)
    m = _mask(kind, Sq // qbs, Skv // kbs, seed=2, B=B, H=Hq)
    o_e, lse_e = oracle.dense_attention_explicit(q, k, v, m, qbs, kbs)
    o_s, dq_s, dk_s, dv_s = oracle.sdpa_dense(q, k, v, m, qbs, kbs, do)
    o_c, lse_c = oracle.c_attention_forward(q, k, v, m, qbs, kbs)
    assert oracle.error_metrics(o_e, o_s)[0] < TOL
    assert oracle.error_metrics(o_c, o_s)[0] < TOL
    assert oracle.error_metrics(lse_c, lse_e)[0] < TOL
    g_e = oracle.dense_attention_backward_explicit(q, k, v, o_e, lse_e, do, m, qbs, kbs)
    g_c = oracle.c_attention_backward(q, k, v, o_c, lse_c, do, m, qbs, kbs)
    for ge, gc, gs in zip(g_e, g_c, (dq_s, dk_s, dv_s)):
        assert ge.shape == gs.shape and gc.shape == gs.shape
        assert oracle.error_metrics(ge, gs)[0] < 5 * TOL
        assert oracle.error_metrics(gc, gs)[0] < 5 * TOL


def test_full_mask_is_plain_attention(oracle):
    q, k, v, _ = oracle.seeded_qkv(1, 2, 2, 64, 64, D=32, seed=3)
    m = torch.ones((4, 4), dtype=torch.bool)
    o, lse = oracle.c_attention_forward(q, k, v, m, 16, 16)
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v)
    assert oracle.error_metrics(o, want)[0] < TOL
    s = torch.matmul(q, k.transpose(-1, -2)) / math.sqrt(32)
    assert oracle.error_metrics(lse, torch.logsumexp(s, -1))[0] < TOL


def test_block_diagonal_is_independent_attentions(oracle):
    q, k, v, _ = oracle.seeded_qkv(1, 1, 1, 64, 64, D=32, seed=4)
    o, _ = oracle.c_attention_forward(q, k, v, torch.eye(4, dtype=torch.bool), 16, 16)
    for i in range(4):
        sl = slice(16 * i, 16 * i + 16)
        want = torch.nn.functional.scaled_dot_product_attention(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        assert oracle.error_metrics(o[:, :, sl], want)[0] < TOL


def test_rectangular_blocks_single_selection(oracle):
    """q_block 16, kv_block 32: query block i attends key block (i // 2) only."""
    q, k, v, _ = oracle.seeded_qkv(1, 1, 1, 64, 64, D=32, seed=5)
    m = torch.zeros((4, 2), dtype=torch.bool)
    for i in range(4):
        m[i, i // 2] = True
    o, _ = oracle.c_attention_forward(q, k, v, m, 16, 32)
    for i in range(4):
        qs, ks = slice(16 * i, 16 * i + 16), slice(32 * (i // 2), 32 * (i // 2) + 32)
        want = torch.nn.functional.scaled_dot_product_attention(q[:, :, qs], k[:, :, ks], v[:, :, ks])
        assert oracle.error_metrics(o[:, :, qs], want)[0] < TOL


def test_brute_force_tiny(oracle):
    """Pure-Python loops over every (query, key, channel) on a case small enough to read."""
    B, H, S, D, bs = 1, 1, 8, 4, 2
    q, k, v, do = oracle.seeded_qkv(B, H, H, S, S, D=D, seed=6)
    m = _mask("rand2d", S // bs, S // bs, seed=7)
    o_c, lse_c = oracle.c_attention_forward(q, k, v, m, bs, bs)
    dq_c, dk_c, dv_c = oracle.c_attention_backward(q, k, v, o_c, lse_c, do, m, bs, bs)
    Q, K, V, DO = (t[0, 0].double().tolist() for t in (q, k, v, do))
    scale = 1.0 / math.sqrt(D)
    O = [[0.0] * D for _ in range(S)]
    P = [[0.0] * S for _ in range(S)]
    for i in range(S):
        sc = {j: scale * sum(Q[i][c] * K[j][c] for c in range(D)) for j in range(S) if m[i // bs, j // bs]}
        mx = max(sc.values())
        den = sum(math.exp(x - mx) for x in sc.values())
        for j, x in sc.items():
            P[i][j] = math.exp(x - mx) / den
            for c in range(D):
                O[i][c] += P[i][j] * V[j][c]
        assert abs(lse_c[0, 0, i].item() - (mx + math.log(den))) < 1e-5
    dQ = [[0.0] * D for _ in range(S)]
    dK = [[0.0] * D for _ in range(S)]
    dV = [[0.0] * D for _ in range(S)]
    for i in range(S):
        delta = sum(DO[i][c] * O[i][c] for c in range(D))
        for j in range(S):
            dp = sum(DO[i][c] * V[j][c] for c in range(D))
            ds = P[i][j] * (dp - delta) * scale
            for c in range(D):
                dQ[i][c] += ds * K[j][c]
                dK[j][c] += ds * Q[i][c]
                dV[j][c] += P[i][j] * DO[i][c]
    for got, want in ((o_c, O), (dq_c, dQ), (dk_c, dK), (dv_c, dV)):
        assert (got[0, 0].double() - torch.tensor(want, dtype=torch.float64)).abs().max().item() < 1e-5


def test_gradients_match_finite_differences_fp64(oracle):
    B, Hq, Hkv, S, D, bs = 1, 2, 1, 8, 4, 4
    q, k, v, do = (t.double() for t in oracle.seeded_qkv(B, Hq, Hkv, S, S, D=D, seed=8))
    m = _mask("rand2d", S // bs, S // bs, seed=9)

    def loss(q_, k_, v_):
        o, _ = oracle.dense_attention_explicit(q_, k_, v_, m, bs, bs, dtype=torch.float64)
        return (o * do).sum().item()

    o, lse = oracle.dense_attention_explicit(q, k, v, m, bs, bs, dtype=torch.float64)
    grads = oracle.dense_attention_backward_explicit(q, k, v, o, lse, do, m, bs, bs, dtype=torch.float64)
    eps = 1e-6
    for which, (x, g) in enumerate(zip((q, k, v), grads)):
        flat = x.reshape(-1)
        for pos in range(0, flat.numel(), 7):
            xp, xm = flat.clone(), flat.clone()
            xp[pos] += eps
            xm[pos] -= eps
            args_p = [q, k, v]
            args_m = [q, k, v]
            args_p[which] = xp.reshape(x.shape)
            args_m[which] = xm.reshape(x.shape)
            num = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(num - g.reshape(-1)[pos].item()) < 1e-6, (which, pos)


def test_gradient_identities(oracle):
    """sum(q o dq) = sum(k o dk) per head (both equal sum_ij dS_ij S_ij); dK = dV = 0 for a key block nobody selects;
    gradients are linear in dO."""
    B, H, S, D, bs = 1, 2, 64, 32, 16
    q, k, v, do = oracle.seeded_qkv(B, H, H, S, S, D=D, seed=10)
    m = _mask("rand2d", 4, 4, seed=11)
    m[:, 2] = False
    o, lse = oracle.c_attention_forward(q, k, v, m, bs, bs)
    dq, dk, dv = oracle.c_attention_backward(q, k, v, o, lse, do, m, bs, bs)
    lhs, rhs = (q * dq).sum((-1, -2)), (k * dk).sum((-1, -2))
    assert (lhs - rhs).abs().max().item() < 1e-3 * lhs.abs().max().item() + 1e-4
    assert dk[:, :, 32:48].abs().max().item() == 0.0 and dv[:, :, 32:48].abs().max().item() == 0.0
    dq2, dk2, dv2 = oracle.c_attention_backward(q, k, v, o, lse, 2 * do, m, bs, bs)
    for a, b2 in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert oracle.error_metrics(b2, 2 * a)[0] < 1e-5


def test_key_block_permutation_invariance(oracle):
    B, H, S, D, bs = 1, 1, 64, 32, 16
    q, k, v, _ = oracle.seeded_qkv(B, H, H, S, S, D=D, seed=12)
    m = _mask("rand2d", 4, 4, seed=13)
    perm = torch.tensor([2, 0, 3, 1])
    tok = (perm[:, None] * bs + torch.arange(bs)[None, :]).reshape(-1)
    o1, lse1 = oracle.c_attention_forward(q, k, v, m, bs, bs)
    o2, lse2 = oracle.c_attention_forward(q, k[:, :, tok], v[:, :, tok], m[:, perm], bs, bs)
    assert oracle.error_metrics(o2, o1)[0] < TOL and oracle.error_metrics(lse2, lse1)[0] < TOL


def test_empty_query_block(oracle):
    """A query block that selects nothing: O = 0, LSE = -inf, dQ = 0 (the reference divides 0/0 there)."""
    q, k, v, do = oracle.seeded_qkv(1, 1, 1, 32, 32, D=16, seed=14)
    m = torch.tensor([[True, False], [False, False]])
    o, lse = oracle.c_attention_forward(q, k, v, m, 16, 16)
    assert o[0, 0, 16:].abs().max().item() == 0.0 and torch.isinf(lse[0, 0, 16:]).all() and (lse[0, 0, 16:] < 0).all()
    o_e, lse_e = oracle.dense_attention_explicit(q, k, v, m, 16, 16)
    assert torch.equal(torch.isinf(lse_e), torch.isinf(lse)) and oracle.error_metrics(o_e, o)[0] < TOL
    dq, dk, dv = oracle.c_attention_backward(q, k, v, o, lse, do, m, 16, 16)
    assert dq[0, 0, 16:].abs().max().item() == 0.0
    assert torch.isfinite(dq).all() and torch.isfinite(dk).all() and torch.isfinite(dv).all()


def test_mask_expansion(oracle):
    m = _mask("rand2d", 3, 5, seed=15)
    dense = oracle.expand_block_mask(m, 4, 2)
    dense_c = oracle.c_expand_block_mask(m, 4, 2)
    assert dense.shape == (12, 10) and torch.equal(dense, dense_c)
    for i in range(12):
        for j in range(10):
            assert dense[i, j] == m[i // 4, j // 2]


@pytest.mark.parametrize("shape", [(4, 4), (1, 1), (7, 9), (80, 80), (65, 129), (2, 3, 17, 70)])
def test_compaction_lists(oracle, shape):
    g = torch.Generator(device="cpu").manual_seed(sum(shape))
    m = torch.rand(shape, generator=g) < 0.4
    q_cnt, q_idx, k_cnt, k_idx = oracle.compact_lists(m)
    c = oracle.c_compact_lists(m)
    for a, b in zip((q_cnt, q_idx, k_cnt, k_idx), c):
        assert a.dtype == np.int32 and np.array_equal(a, b)
    m3 = m.reshape(-1, shape[-2], shape[-1])
    assert q_cnt.sum() == k_cnt.sum() == int(m.sum())
    for b in range(m3.shape[0]):
        nz = torch.nonzero(m3[b])  # row-major: ascending (i, j)
        for i in range(shape[-2]):
            want = nz[nz[:, 0] == i][:, 1].numpy()
            assert np.array_equal(q_idx[b, i, : q_cnt[b, i]], want)
            assert (q_idx[b, i, q_cnt[b, i] :] == -1).all()
        nzt = torch.nonzero(m3[b].t())
        for j in range(shape[-1]):
            want = nzt[nzt[:, 0] == j][:, 1].numpy()
            assert np.array_equal(k_idx[b, j, : k_cnt[b, j]], want)
            assert (k_idx[b, j, k_cnt[b, j] :] == -1).all()


@pytest.mark.parametrize("qbs,kbs,nQ,nK", [(16, 64, 16, 4), (64, 128, 4, 2), (48, 192, 8, 2), (128, 64, 2, 4), (384, 192, 1, 2), (32, 64, 8, 6)])
def test_tile_lists_describe_the_dense_mask(oracle, qbs, kbs, nQ, nK):
    """The tile lists, decoded back, must rebuild exactly the element-level mask: every predicate bit stands for a
    region inside which the dense mask is constant, and regions without an entry are all False."""
    g = torch.Generator().manual_seed(qbs + kbs)
    m = torch.rand((2, nQ, nK), generator=g) < 0.45
    dense = oracle.expand_block_mask(m, qbs, kbs).numpy()
    qt_cnt, qt_ent, kt_cnt, kt_ent = oracle.tile_lists(m[:, None], qbs, kbs)
    Sq, Skv = nQ * qbs, nK * kbs
    for b in range(2):
        from_q = np.zeros((Sq, Skv), bool)
        for T in range(Sq // 128):
            ents = qt_ent[b, T, : qt_cnt[b, T]]
            assert (qt_ent[b, T, qt_cnt[b, T]:] == -1).all() and (np.diff(ents >> 8) > 0).all()
            for e in ents:
                for grp in range(8):
                    if (e >> grp) & 1:
                        from_q[128 * T + 16 * grp: 128 * T + 16 * grp + 16, (e >> 8) * kbs: ((e >> 8) + 1) * kbs] = True
        from_k = np.zeros((Sq, Skv), bool)
        for U in range(Skv // 128):
            ents = kt_ent[b, U, : kt_cnt[b, U]]
            assert (kt_ent[b, U, kt_cnt[b, U]:] == -1).all() and (np.diff(ents >> 8) > 0).all()
            for e in ents:
                for w in range(4):
                    for f in range(2):
                        if (e >> (2 * w + f)) & 1:
                            r0, c0 = 32 * (e >> 8) + 16 * f, 128 * U + 32 * w
                            from_k[r0: r0 + 16, c0: c0 + 32] = True
        assert (from_q == dense[b]).all() and (from_k == dense[b]).all()


def test_ssta_mask_against_library_topk(oracle):
    """Row sets against torch.topk on distinct scores; counts and forced entries follow from the definition."""
    g = torch.Generator().manual_seed(12)
    q = torch.randn((2, 4, 12 * 32, 16), generator=g)
    k = torch.randn((2, 2, 6 * 64, 16), generator=g)
    qm, km = oracle.block_mean(q, 32), oracle.block_mean(k, 64)
    assert torch.allclose(qm[1, 3, 5], q[1, 3, 160:192].double().mean(0))
    sc = oracle.ssta_scores(qm, km)
    assert torch.allclose(sc[1, 3, 5, 2], (qm[1, 3, 5] * km[1, 1, 2]).sum())  # q head 3 reads kv head 1
    topk = 3
    m = oracle.ssta_mask(sc, 32, 64, topk, band=-1, sink=0)
    want = torch.zeros_like(m).scatter_(-1, sc.topk(topk, dim=-1).indices, True)
    assert torch.equal(m, want) and (m.sum(-1) == topk).all()
    full = oracle.ssta_mask(sc, 32, 64, topk, band=1, sink=1)
    i = torch.arange(12)[:, None]
    j = torch.arange(6)[None, :]
    forced = ((j - i // 2).abs() <= 1) | (j < 1)
    assert torch.equal(full, m | forced[None, None])
    base = torch.rand((12, 6), generator=g) < 0.3
    assert torch.equal(oracle.ssta_mask(sc, 32, 64, topk, -1, 0, base), m | base[None, None])
    # ties go to the lower index; asking for more blocks than exist selects all of them
    flat = torch.zeros((1, 1, 2, 5), dtype=torch.float64)
    assert oracle.ssta_mask(flat, 64, 64, 2, -1, 0)[0, 0].tolist() == [[True, True, False, False, False]] * 2
    assert oracle.ssta_mask(flat, 64, 64, 9, -1, 0).all()


def test_tile_order_is_the_einops_rearrangement(oracle):
    import einops

    grid, tile = (4, 6, 4), (2, 3, 2)
    x = torch.arange(4 * 6 * 4)
    want = einops.rearrange(x, "(nt tt nh th nw tw) -> (nt nh nw tt th tw)", nt=2, tt=2, nh=2, th=3, nw=2, tw=2)
    idx = oracle.tile_order(grid, tile)
    assert torch.equal(x[idx], want) and sorted(idx.tolist()) == list(range(96))


def test_pair_numbering(oracle):
    """oracle.pair_numbering: the numbers are 0..n-1 in key-major list order (checked against numpy's cumsum and against
    the lists themselves), and the query-major table points back at the same pair."""
    for shape, p, seed in (((5, 7), 0.5, 0), ((2, 3, 6, 4), 0.4, 1), ((3, 3), 0.0, 2), ((1, 2, 4, 4), 1.0, 3)):
        m = torch.rand(shape, generator=torch.Generator().manual_seed(seed)) < p
        q_cnt, q_idx, k_cnt, k_idx = oracle.compact_lists(m)
        pair_base, q_slot = oracle.pair_numbering(q_cnt, q_idx, k_cnt, k_idx)
        M, nK = k_cnt.shape
        nQ = q_cnt.shape[1]
        assert np.array_equal(pair_base, np.concatenate([[0], np.cumsum(k_cnt.reshape(-1))]).astype(np.int32))
        assert pair_base[-1] == int(m.sum())
        seen = []
        for mm in range(M):
            for I in range(nQ):
                for e in range(nK):
                    n = q_slot[mm, I, e]
                    if e >= q_cnt[mm, I]:
                        assert n == -1
                        continue
                    J = q_idx[mm, I, e]
                    pos = n - pair_base[mm * nK + J]
                    assert 0 <= pos < k_cnt[mm, J] and k_idx[mm, J, pos] == I
                    seen.append(int(n))
        assert sorted(seen) == list(range(int(m.sum())))


def test_tile_pair_numbering(oracle):
    """oracle.tile_pair_numbering against the token-level mask: a (query tile, key tile) pair is numbered exactly when
    the dense mask (numpy's kron) has an allowed element inside that 128 x 128 square, the numbers run 0..n-1 in
    key-major order, and every entry of the key-major tile list carries the number of the square its slab lies in."""
    for shape, qb, kb, p, seed in (((8, 4), 32, 64, 0.3, 0), ((2, 2, 16, 2), 16, 192, 0.2, 1), ((4, 4), 64, 64, 0.0, 2),
                                   ((1, 2, 8, 6), 48, 64, 0.5, 3), ((2, 4), 128, 64, 1.0, 4)):
        m = torch.rand(shape, generator=torch.Generator().manual_seed(seed)) < p
        nQ, nK = shape[-2:]
        Sq, Skv = nQ * qb, nK * kb
        if Sq % 128 or Skv % 128:
            continue
        n_qt, n_kt = Sq // 128, Skv // 128
        pair_base, table, kt_slot = oracle.tile_pair_numbering(m, qb, kb)
        dense = np.kron(m.numpy().reshape(-1, nQ, nK), np.ones((qb, kb), bool))
        M = dense.shape[0]
        squares = dense.reshape(M, n_qt, 128, n_kt, 128).any(axis=(2, 4))  # [M, T, U]
        assert np.array_equal(table >= 0, squares)
        order = [table[b, T, U] for b in range(M) for U in range(n_kt) for T in range(n_qt) if squares[b, T, U]]
        assert order == list(range(len(order))) and pair_base[-1] == len(order)
        assert np.array_equal(pair_base[:-1], np.concatenate([[0], np.cumsum(squares.transpose(0, 2, 1).reshape(-1, n_qt).sum(1))[:-1]]))
        _, _, kt_cnt, kt_ent = oracle.tile_lists(m, qb, kb)
        for b in range(M):
            for U in range(n_kt):
                for e in range(kt_ent.shape[2]):
                    if e < kt_cnt[b, U]:
                        assert kt_slot[b, U, e] == table[b, (kt_ent[b, U, e] >> 8) // 4, U] >= 0
                    else:
                        assert kt_slot[b, U, e] == -1


def test_sliding_tile_mask_restatement(oracle):
    """Pins oracle.sta_window / sta_3d_mask / sta_token_mask: hand-computed windows, a hand-listed row of an asymmetric
    grid, the Kronecker product of 1-D band matrices (numpy's kron fixes the T-major, W-minor enumeration: swapping two
    axes fails it), and the token-level mask against the block mask expanded through the tile permutation."""
    w = oracle.sta_window
    assert w(0, 10, 3, True) == (0, 2) and w(9, 10, 3, True) == (7, 9) and w(4, 10, 3, True) == (3, 5)
    assert w(0, 10, 3, False) == (0, 1) and w(9, 10, 3, False) == (8, 9) and w(4, 10, 3, False) == (3, 5)
    assert w(1, 10, 5, True) == (0, 4) and w(1, 10, 5, False) == (0, 3) and w(8, 10, 5, True) == (5, 9)
    assert w(0, 2, 3, True) == (0, 1) and w(1, 2, 3, True) == (0, 1) and w(0, 1, 3, True) == (0, 0) and w(0, 1, 3, False) == (0, 0)
    assert w(3, 6, 1, True) == (3, 3)

    # tiles (2, 3, 5), clipped 3x3x3 window: tile (1, 2, 3) has index (1*3+2)*5+3 = 28 and keeps t in {0,1}, h in {1,2},
    # w in {2,3,4}
    m = oracle.sta_3d_mask((2, 3, 5), (3, 3, 3), clamp=False)
    want = sorted((t * 3 + h) * 5 + x for t in (0, 1) for h in (1, 2) for x in (2, 3, 4))
    assert want == [7, 8, 9, 12, 13, 14, 22, 23, 24, 27, 28, 29]
    assert m[28].nonzero().flatten().tolist() == want
    # same tile, clamped: t in {0,1} (axis shorter than the window), h slides to {0,1,2}, w in {2,3,4}
    mc = oracle.sta_3d_mask((2, 3, 5), (3, 3, 3), clamp=True)
    assert mc[28].nonzero().flatten().tolist() == sorted((t * 3 + h) * 5 + x for t in (0, 1) for h in (0, 1, 2) for x in (2, 3, 4))

    def band(n, wd, clamp):  # 1-D window as a matrix: centre clipped into the grid (clamped) or left alone (clipped)
        i = np.arange(n)
        if clamp and n <= wd:
            return np.ones((n, n), bool)
        c = np.clip(i, wd // 2, n - 1 - wd // 2) if clamp else i
        return np.abs(c[:, None] - i[None, :]) <= wd // 2

    for tiles, window in (((2, 3, 5), (3, 3, 3)), ((5, 6, 10), (3, 3, 3)), ((3, 1, 4), (1, 3, 5)), ((4, 2, 3), (5, 1, 3))):
        for clamp in (False, True):
            kron = np.kron(np.kron(band(tiles[0], window[0], clamp), band(tiles[1], window[1], clamp)), band(tiles[2], window[2], clamp))
            got = oracle.sta_3d_mask(tiles, window, clamp)
            assert np.array_equal(got.numpy(), kron.astype(bool)), (tiles, window, clamp)
    full = oracle.sta_3d_mask((5, 6, 10), (3, 3, 3), True)
    assert (full.sum(-1) == 27).all()
    assert int(oracle.sta_3d_mask((5, 6, 10), (3, 3, 3), False).sum()) == 13 * 16 * 28

    # token-level mask from raster coordinates == block mask expanded to tokens and carried back through the tile order
    grid, tile, window = (4, 6, 10), (2, 3, 2), (3, 1, 3)
    tiles = tuple(g // t for g, t in zip(grid, tile))
    blk = tile[0] * tile[1] * tile[2]
    idx = oracle.tile_order(grid, tile)
    for clamp in (False, True):
        dense_tiled = oracle.expand_block_mask(oracle.sta_3d_mask(tiles, window, clamp), blk, blk)
        raster = torch.zeros_like(dense_tiled)
        raster[idx[:, None], idx[None, :]] = dense_tiled
        assert torch.equal(oracle.sta_token_mask(grid, tile, window, clamp), raster)


def test_golden_fixtures_match_oracle(oracle):
    """The committed fixtures are what the oracle computes today (guards both against drift)."""
    gdir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    names = sorted(f for f in os.listdir(gdir) if f.endswith(".npz"))
    assert len(names) >= 4
    for name in names:
        z = np.load(os.path.join(gdir, name))
        q, k, v, do = (torch.from_numpy(z[n]).view(torch.bfloat16).float() for n in ("q", "k", "v", "do"))
        m = torch.from_numpy(z["mask"])
        qbs, kbs = int(z["q_block"]), int(z["kv_block"])
        o_s, dq_s, dk_s, dv_s = oracle.sdpa_dense(q, k, v, m, qbs, kbs, do)
        rows_ok = torch.isfinite(torch.from_numpy(z["lse"]))  # SDPA yields NaN on rows without keys
        sel = rows_ok.unsqueeze(-1).expand_as(o_s)
        assert (torch.from_numpy(z["o"])[sel] - o_s[sel]).abs().max().item() < 5 * TOL
        if rows_ok.all():
            scale = max(1.0, float(dq_s.abs().max()))
            for n, want in (("dq", dq_s), ("dk", dk_s), ("dv", dv_s)):
                assert (torch.from_numpy(z[n]) - want).abs().max().item() < 2e-4 * scale, (name, n)
        lists = oracle.compact_lists(m)
        for n, want in zip(("q_cnt", "q_idx", "k_cnt", "k_idx"), lists):
            assert np.array_equal(z[n], want)
