"""CPU oracle for the block-sparse attention operator — TEST INFRASTRUCTURE ONLY.

Nothing in the product imports this module: only tests/, `__graft_entry__.smoke()` and the `cpu_baseline` leg of
bench.py may.  It restates the reference's dense path in three independent ways so that each can check the others:

  * `dense_attention_explicit`  the textbook formula written out with matmul / exp / sum in fp32 or fp64, plus
    closed-form gradients (`dense_attention_backward_explicit`);
  * `sdpa_dense`                the library routine the reference itself uses as its dense path,
    `F.scaled_dot_product_attention(q, k, v, attn_mask=dense bool mask)` (test/test_flex_block_attn.py:48-51,
    benchmark/utils/utils.py:132-138), with gradients from autograd;
  * the plain-C restatement in attn_ref.c (double accumulation, OpenMP), reached through `c_*` wrappers.

Semantics restated (reference file:line):
  allowed(i, j) = block_mask[b, h, i // q_block, j // kv_block]          benchmark/utils/utils.py:105-119
  O = softmax(Q K^T / sqrt(128) | allowed) V                             flex_block_attn_h100.cu:177, :199-221, :292
  delta = rowsum(dO o O)                                                 flex_block_attn_h100.cu:375-379
  P = exp(S/sqrt(D) - LSE); dV = P^T dO; dP = dO V^T;
  dS = P o (dP - delta)/sqrt(D); dQ = dS K; dK = dS^T Q                  flex_block_attn_h100.cu:498-537, :750-753
  kv head of q head h = h // (Hq / Hkv); dK, dV summed over the group    flex_block_attn_h100.cu:80, :615, :555-556
  work lists = ascending nonzero indices per mask row / column           flex_block_attn_h100.cu:134-135, :672

Parity status: O and LSE are pinned by SDPA, by the explicit formula, by special cases and by brute force
(tests/test_oracle.py).  dQ, dK, dV have no assertion anywhere in the reference (its dQ check is commented out,
test/test_flex_block_attn.py:140, and its benchmark comparison is vacuous); they are pinned here by autograd of
SDPA, by the closed form and by fp64 finite differences.
"""
import ctypes
import math
import os

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
C_LIB_PATH = os.path.join(_HERE, "libattn_ref.so")


# ---------------------------------------------------------------------------------------------------------------
# masks and work lists
# ---------------------------------------------------------------------------------------------------------------
def expand_block_mask(block_mask, q_block, kv_block):
    """[..., nQ, nK] bool -> [..., nQ*q_block, nK*kv_block] bool (benchmark/utils/utils.py:105-119)."""
    return block_mask.repeat_interleave(q_block, dim=-2).repeat_interleave(kv_block, dim=-1)


def compact_lists(block_mask):
    """Work lists of a bool mask [nQ, nK] or [B, H, nQ, nK] by brute force on the host.

    Returns int32 numpy arrays (q_cnt [M,nQ], q_idx [M,nQ,nK], k_cnt [M,nK], k_idx [M,nK,nQ]), M = B*H or 1;
    lists ascending, padded with -1.
    """
    m = block_mask.detach().cpu().numpy().astype(bool)
    nQ, nK = m.shape[-2:]
    m = m.reshape(-1, nQ, nK)
    M = m.shape[0]
    q_cnt = np.zeros((M, nQ), np.int32)
    q_idx = np.full((M, nQ, nK), -1, np.int32)
    k_cnt = np.zeros((M, nK), np.int32)
    k_idx = np.full((M, nK, nQ), -1, np.int32)
    for b in range(M):
        for i in range(nQ):
            js = np.nonzero(m[b, i])[0]
            q_cnt[b, i] = len(js)
            q_idx[b, i, : len(js)] = js
        for j in range(nK):
            is_ = np.nonzero(m[b, :, j])[0]
            k_cnt[b, j] = len(is_)
            k_idx[b, j, : len(is_)] = is_
    return q_cnt, q_idx, k_cnt, k_idx


def pair_numbering(q_cnt, q_idx, k_cnt, k_idx):
    """Numbers of the selected block pairs in key-major list order (include/fba.h, fba_pair_slots), by plain loops:
    pair (m, J, e) = (pairs of all list rows before (m, J)) + e; returns (pair_base [M*nK + 1] with the total last,
    q_slot [M, nQ, nK] = number of the pair (I, q_idx[m, I, e]), -1 beyond q_cnt)."""
    M, nK = k_cnt.shape
    nQ = q_cnt.shape[1]
    pair_base = np.zeros((M * nK + 1,), np.int32)
    number = {}
    n = 0
    for m in range(M):
        for J in range(nK):
            pair_base[m * nK + J] = n
            for e in range(int(k_cnt[m, J])):
                number[(m, int(k_idx[m, J, e]), J)] = n
                n += 1
    pair_base[M * nK] = n
    q_slot = np.full((M, nQ, nK), -1, np.int32)
    for m in range(M):
        for I in range(nQ):
            for e in range(int(q_cnt[m, I])):
                q_slot[m, I, e] = number[(m, I, int(q_idx[m, I, e]))]
    return pair_base, q_slot


def tile_lists(block_mask, q_block, kv_block):
    """Brute-force tile lists (include/fba.h, fba_tile_lists) of a bool mask [nQ, nK] or [B, H, nQ, nK]: for every
    128-row query tile the key blocks selected by any of its eight 16-row groups, with one predicate bit per group; for
    every 128-row key tile the 32-row query slabs that touch it, with one bit per (32-key wave, 16-row half-slab).
    Everything follows from allowed(i, j) = mask[i // q_block, j // kv_block]."""
    m = block_mask.detach().cpu().numpy().astype(bool)
    nQ, nK = m.shape[-2:]
    m = m.reshape(-1, nQ, nK)
    M, Sq, Skv = m.shape[0], nQ * q_block, nK * kv_block
    n_qt, n_kt, n_qs = Sq // 128, Skv // 128, Sq // 32
    qt_cnt = np.zeros((M, n_qt), np.int32)
    qt_ent = np.full((M, n_qt, nK), -1, np.int32)
    kt_cnt = np.zeros((M, n_kt), np.int32)
    kt_ent = np.full((M, n_kt, n_qs), -1, np.int32)
    for b in range(M):
        for T in range(n_qt):
            for J in range(nK):
                bits = sum(int(m[b, (128 * T + 16 * g) // q_block, J]) << g for g in range(8))
                if bits:
                    qt_ent[b, T, qt_cnt[b, T]] = (J << 8) | bits
                    qt_cnt[b, T] += 1
        for U in range(n_kt):
            for s_ in range(n_qs):
                bits = 0
                for w in range(4):
                    for f in range(2):
                        bits |= int(m[b, (32 * s_ + 16 * f) // q_block, (128 * U + 32 * w) // kv_block]) << (2 * w + f)
                if bits:
                    kt_ent[b, U, kt_cnt[b, U]] = (s_ << 8) | bits
                    kt_cnt[b, U] += 1
    return qt_cnt, qt_ent, kt_cnt, kt_ent


def tile_pair_numbering(block_mask, q_block, kv_block):
    """Numbers of the (128-row query tile T, 128-key tile U) pairs that hold at least one allowed (row, key), in
    key-major order (include/fba.h, fba_tile_slots), straight from allowed(i, j) = mask[i // q_block, j // kv_block]:
    returns (pair_base [M * n_kt + 1] with the total last, slot_table [M, n_qt, n_kt] (-1 where nothing is allowed),
    kt_slot [M, n_kt, n_qs] = the pair number of every entry of the key-major tile list (-1 beyond its count))."""
    m = block_mask.detach().cpu().numpy().astype(bool)
    nQ, nK = m.shape[-2:]
    m = m.reshape(-1, nQ, nK)
    M, Sq, Skv = m.shape[0], nQ * q_block, nK * kv_block
    n_qt, n_kt, n_qs = Sq // 128, Skv // 128, Sq // 32
    pair_base = np.zeros((M * n_kt + 1,), np.int32)
    slot_table = np.full((M, n_qt, n_kt), -1, np.int32)
    kt_slot = np.full((M, n_kt, n_qs), -1, np.int32)
    n = 0
    for b in range(M):
        for U in range(n_kt):
            pair_base[b * n_kt + U] = n
            cols = sorted({j // kv_block for j in range(128 * U, 128 * U + 128, 32)})
            for T in range(n_qt):
                rows = sorted({i // q_block for i in range(128 * T, 128 * T + 128, 16)})
                if m[b][np.ix_(rows, cols)].any():
                    slot_table[b, T, U] = n
                    n += 1
            e = 0
            for s_ in range(n_qs):  # entries of the key-major tile list: slabs with an allowed (row, key) in this key tile
                rows = sorted({i // q_block for i in range(32 * s_, 32 * s_ + 32, 16)})
                if m[b][np.ix_(rows, cols)].any():
                    kt_slot[b, U, e] = slot_table[b, s_ // 4, U]
                    e += 1
    pair_base[M * n_kt] = n
    return pair_base, slot_table, kt_slot


def block_mean(x, block):
    """(B, H, S, D) -> (B, H, S / block, D) float64 means of consecutive row blocks (include/fba.h, fba_block_mean)."""
    B, H, S, D = x.shape
    return x.double().reshape(B, H, S // block, block, D).mean(3)


def ssta_scores(q_mean, k_mean):
    """<q_mean[b,h,i], k_mean[b, h // (Hq/Hkv), j]> in float64 -> (B, Hq, nQ, nK)."""
    Hq = q_mean.shape[1]
    return torch.matmul(q_mean.double(), _repeat_heads(k_mean.double(), Hq).transpose(-1, -2))


def _repeat_heads(x, Hq):
    return x if x.shape[1] == Hq else x.repeat_interleave(Hq // x.shape[1], dim=1)


def ssta_mask(scores, q_block, kv_block, topk, band, sink, base=None):
    """Bool (B, H, nQ, nK) by plain loops over rows (include/fba.h, fba_ssta_mask): the `topk` largest scores of each
    row, ties to the lower index; key blocks within `band` of the one holding the query block's first row; the first
    `sink` key blocks; `base` [nQ, nK] if given."""
    sc = scores.numpy()
    B, H, nQ, nK = sc.shape
    out = np.zeros((B, H, nQ, nK), bool)
    for b in range(B):
        for h in range(H):
            for i in range(nQ):
                order = sorted(range(nK), key=lambda j: (-sc[b, h, i, j], j))
                out[b, h, i, order[: min(topk, nK)]] = True
                diag = (i * q_block) // kv_block
                for j in range(nK):
                    if abs(j - diag) <= band or j < sink:
                        out[b, h, i, j] = True
    if base is not None:
        out |= base.numpy().astype(bool)[None, None]
    return torch.from_numpy(out)


def tile_order(grid, tile):
    """Raster index of every token, listed in tile order (include/fba.h, fba_tile_permute): x_tiled = x[..., idx, :]."""
    T, H, W = grid
    tT, tH, tW = tile
    idx = []
    for bt in range(T // tT):
        for bh in range(H // tH):
            for bw in range(W // tW):
                for it in range(tT):
                    for ih in range(tH):
                        for iw in range(tW):
                            idx.append(((bt * tT + it) * H + bh * tH + ih) * W + bw * tW + iw)
    return torch.tensor(idx, dtype=torch.long)


def sta_window(c, n, w, clamp):
    """Inclusive range [lo, hi] of key tiles along one axis for the query tile at coordinate c of n, window extent w
    (odd).  Clipped: the part of [c - w//2, c + w//2] inside the grid.  Clamped: that interval is first slid inwards
    until it lies inside the grid (then cut to the grid if the axis is shorter than the window), so an interior and a
    border tile see equally many tiles."""
    lo, hi = c - w // 2, c + w // 2
    if clamp:
        if lo < 0:
            lo, hi = 0, hi - lo
        if hi > n - 1:
            lo, hi = lo - (hi - (n - 1)), n - 1
    return max(lo, 0), min(hi, n - 1)


def sta_3d_mask(tiles, window, clamp=True):
    """Sliding-tile block mask by plain loops over tile coordinates: tile (t, h, w) has index (t * nh + h) * nw + w
    (T-major, W-minor); query tile a keeps key tile b iff b lies inside a's window on every axis.  Bool [n, n]."""
    nt, nh, nw = tiles
    n = nt * nh * nw
    out = np.zeros((n, n), bool)
    for qt in range(nt):
        t0, t1 = sta_window(qt, nt, window[0], clamp)
        for qh in range(nh):
            h0, h1 = sta_window(qh, nh, window[1], clamp)
            for qw in range(nw):
                w0, w1 = sta_window(qw, nw, window[2], clamp)
                a = (qt * nh + qh) * nw + qw
                for kt in range(t0, t1 + 1):
                    for kh in range(h0, h1 + 1):
                        for kw in range(w0, w1 + 1):
                            out[a, (kt * nh + kh) * nw + kw] = True
    return torch.from_numpy(out)


def sta_token_mask(grid, tile, window, clamp=True):
    """Token-level sliding-tile mask for a latent in RASTER order, from token coordinates alone: token i =
    (t * H + h) * W + w attends token j iff the tile holding j lies inside the window of the tile holding i on every
    axis.  Bool [T*H*W, T*H*W]; independent of any tile enumeration or token permutation."""
    T, H, W = grid
    tiles = (T // tile[0], H // tile[1], W // tile[2])
    coords = np.stack(np.meshgrid(np.arange(T), np.arange(H), np.arange(W), indexing="ij"), -1).reshape(-1, 3)
    ok = np.ones((len(coords), len(coords)), bool)
    for ax in range(3):
        tc = coords[:, ax] // tile[ax]  # tile coordinate of every token along this axis
        lohi = np.array([sta_window(int(c), tiles[ax], window[ax], clamp) for c in range(tiles[ax])])
        lo, hi = lohi[tc, 0], lohi[tc, 1]
        ok &= (tc[None, :] >= lo[:, None]) & (tc[None, :] <= hi[:, None])
    return torch.from_numpy(ok)


# ---------------------------------------------------------------------------------------------------------------
# restatement 1: explicit formula
# ---------------------------------------------------------------------------------------------------------------
def _broadcast_kv(x, Hq):
    """[B, Hkv, S, D] -> [B, Hq, S, D], q head h reading kv head h // (Hq / Hkv)."""
    Hkv = x.shape[1]
    return x if Hkv == Hq else x.repeat_interleave(Hq // Hkv, dim=1)


def dense_attention_explicit(q, k, v, block_mask, q_block, kv_block, dtype=torch.float32):
    """Returns (o, lse) in `dtype`; rows with no allowed key give o = 0, lse = -inf."""
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    Hq, D = q.shape[1], q.shape[3]
    kk, vv = _broadcast_kv(k, Hq), _broadcast_kv(v, Hq)
    allowed = expand_block_mask(block_mask.to(q.device), q_block, kv_block)
    s = torch.matmul(q, kk.transpose(-1, -2)) / math.sqrt(D)
    s = s.masked_fill(~allowed, float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse.unsqueeze(-1).clamp_min(torch.finfo(dtype).min))
    p = torch.where(torch.isfinite(lse).unsqueeze(-1), p, torch.zeros_like(p))
    return torch.matmul(p, vv), lse


def dense_attention_backward_explicit(q, k, v, o, lse, do, block_mask, q_block, kv_block, dtype=torch.float32):
    """Closed-form gradients (dq, dk, dv) in `dtype`."""
    q, k, v, o, lse, do = (t.to(dtype) for t in (q, k, v, o, lse, do))
    B, Hq, Sq, D = q.shape
    Hkv, Skv = k.shape[1], k.shape[2]
    kk, vv = _broadcast_kv(k, Hq), _broadcast_kv(v, Hq)
    allowed = expand_block_mask(block_mask.to(q.device), q_block, kv_block)
    s = torch.matmul(q, kk.transpose(-1, -2)) / math.sqrt(D)
    p = torch.exp(s - lse.reshape(B, Hq, Sq, 1))
    p = torch.where(allowed & torch.isfinite(lse.reshape(B, Hq, Sq, 1)), p, torch.zeros_like(p))
    delta = (do * o).sum(-1, keepdim=True)
    dv = torch.matmul(p.transpose(-1, -2), do)
    dp = torch.matmul(do, vv.transpose(-1, -2))
    ds = p * (dp - delta) / math.sqrt(D)
    dq = torch.matmul(ds, kk)
    dk = torch.matmul(ds.transpose(-1, -2), q)
    if Hkv != Hq:
        g = Hq // Hkv
        dk = dk.reshape(B, Hkv, g, Skv, D).sum(2)
        dv = dv.reshape(B, Hkv, g, Skv, D).sum(2)
    return dq, dk, dv


# ---------------------------------------------------------------------------------------------------------------
# restatement 2: the library routine the reference calls
# ---------------------------------------------------------------------------------------------------------------
def sdpa_dense(q, k, v, block_mask, q_block, kv_block, do=None):
    """F.scaled_dot_product_attention on the expanded mask, in the dtype of q.  With `do`, also returns
    (dq, dk, dv) from autograd."""
    Hq = q.shape[1]
    allowed = expand_block_mask(block_mask.to(q.device), q_block, kv_block)
    if do is None:
        return F.scaled_dot_product_attention(q, _broadcast_kv(k, Hq), _broadcast_kv(v, Hq), attn_mask=allowed)
    q_, k_, v_ = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    o = F.scaled_dot_product_attention(q_, _broadcast_kv(k_, Hq), _broadcast_kv(v_, Hq), attn_mask=allowed)
    o.backward(do)
    return o.detach(), q_.grad, k_.grad, v_.grad


# ---------------------------------------------------------------------------------------------------------------
# restatement 3: plain C (attn_ref.c)
# ---------------------------------------------------------------------------------------------------------------
_clib = None


def c_lib():
    global _clib
    if _clib is None:
        if not os.path.exists(C_LIB_PATH):
            raise ImportError(f"{C_LIB_PATH} missing: run `python oracle/build_oracle.py`")
        lib = ctypes.CDLL(C_LIB_PATH)
        P, I, L = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
        lib.oracle_num_threads.restype = I
        lib.oracle_set_num_threads.argtypes = [I]
        lib.oracle_expand_block_mask.argtypes = [P, I, I, I, I, P]
        lib.oracle_mask_compact.argtypes = [P, L, I, I, P, P, P, P]
        lib.oracle_attn_fwd.argtypes = [P, P, P, P, L, I, I, I, I, I, I, I, I, P, P]
        lib.oracle_bwd_delta.argtypes = [P, P, L, I, P]
        lib.oracle_attn_bwd.argtypes = [P, P, P, P, P, P, P, L, I, I, I, I, I, I, I, I, P, P, P]
        _clib = lib
    return _clib


def _f32(t):
    return np.ascontiguousarray(t.detach().cpu().to(torch.float32).numpy())


def _u8(t):
    return np.ascontiguousarray(t.detach().cpu().numpy().astype(np.uint8))


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def c_compact_lists(block_mask):
    m = _u8(block_mask)
    nQ, nK = m.shape[-2:]
    M = 1 if m.ndim == 2 else m.shape[0] * m.shape[1]
    q_cnt = np.empty((M, nQ), np.int32)
    q_idx = np.empty((M, nQ, nK), np.int32)
    k_cnt = np.empty((M, nK), np.int32)
    k_idx = np.empty((M, nK, nQ), np.int32)
    c_lib().oracle_mask_compact(_p(m), M, nQ, nK, _p(q_cnt), _p(q_idx), _p(k_cnt), _p(k_idx))
    return q_cnt, q_idx, k_cnt, k_idx


def c_expand_block_mask(block_mask, q_block, kv_block):
    m = _u8(block_mask)
    nQ, nK = m.shape
    out = np.empty((nQ * q_block, nK * kv_block), np.uint8)
    c_lib().oracle_expand_block_mask(_p(m), nQ, nK, q_block, kv_block, _p(out))
    return torch.from_numpy(out.astype(bool))


def c_attention_forward(q, k, v, block_mask, q_block, kv_block):
    """fp32 (o, lse) from attn_ref.c."""
    qa, ka, va, m = _f32(q), _f32(k), _f32(v), _u8(block_mask)
    B, Hq, Sq, D = qa.shape
    Hkv, Skv = ka.shape[1], ka.shape[2]
    M = 1 if m.ndim == 2 else B * Hq
    o = np.empty_like(qa)
    lse = np.empty((B, Hq, Sq), np.float32)
    c_lib().oracle_attn_fwd(_p(qa), _p(ka), _p(va), _p(m), M, B, Hq, Hkv, Sq, Skv, D, q_block, kv_block, _p(o), _p(lse))
    return torch.from_numpy(o), torch.from_numpy(lse)


def c_attention_backward(q, k, v, o, lse, do, block_mask, q_block, kv_block):
    """fp32 (dq, dk, dv) from attn_ref.c."""
    qa, ka, va, oa, la, da, m = _f32(q), _f32(k), _f32(v), _f32(o), _f32(lse), _f32(do), _u8(block_mask)
    B, Hq, Sq, D = qa.shape
    Hkv, Skv = ka.shape[1], ka.shape[2]
    M = 1 if m.ndim == 2 else B * Hq
    dq, dk, dv = np.empty_like(qa), np.empty_like(ka), np.empty_like(va)
    c_lib().oracle_attn_bwd(
        _p(qa), _p(ka), _p(va), _p(oa), _p(la), _p(da), _p(m), M, B, Hq, Hkv, Sq, Skv, D, q_block, kv_block, _p(dq), _p(dk), _p(dv)
    )
    return torch.from_numpy(dq), torch.from_numpy(dk), torch.from_numpy(dv)


# ---------------------------------------------------------------------------------------------------------------
# shared helpers for parity tests
# ---------------------------------------------------------------------------------------------------------------
def seeded_qkv(B, Hq, Hkv, Sq, Skv, D=128, seed=0, peaky=False):
    """fp32 q, k, v, do from a CPU generator.  `peaky` reproduces the reference test's input distribution: a random
    direction times a N(0.1, 10) magnitude per row (test/test_flex_block_attn.py:58-64)."""
    g = torch.Generator(device="cpu").manual_seed(seed)

    def draw(shape):
        t = torch.randn(shape, generator=g)
        if peaky:
            mag = torch.randn(shape[:-1] + (1,), generator=g) * 10.0 + 0.1
            t = t * mag / t.norm(dim=-1, keepdim=True)
        return t

    return draw((B, Hq, Sq, D)), draw((B, Hkv, Skv, D)), draw((B, Hkv, Skv, D)), torch.randn((B, Hq, Sq, D), generator=g)


def error_metrics(got, ref):
    """(max-abs error, relative L2 error) of `got` against `ref`, computed in fp64."""
    g, r = got.detach().double().cpu(), ref.detach().double().cpu()
    return (g - r).abs().max().item(), ((g - r).norm() / r.norm().clamp_min(1e-30)).item()
