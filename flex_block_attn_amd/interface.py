"""Operator surface of flex-block-attn on MI355X.

Same names, argument order and return arity as the reference's flex_block_attn/flex_block_attn_interface.py
(`flex_block_attn_func` :91-106, `FlexBlockAttnFunc` :14-89, `_flex_block_attn_forward` :6-8,
`_flex_block_attn_backward` :10-12).  The compiled half is libfba_gfx950.so, reached through ctypes with raw device
pointers and the current HIP stream; PyTorch only provides device memory and autograd plumbing.

What differs from the reference, deliberately:
  * the bool block mask is turned into index lists once, on the GPU (`compact_block_mask`), at its true
    (q_block x kv_block) granularity; the coarse / fine mask pair of flex_block_attn_interface.py:38-66 is not needed;
  * backward reuses the key-major lists emitted by the same compaction instead of transposing the masks
    (flex_block_attn_interface.py:85-86);
  * dq, dk, dv come back in the dtype of q (bf16) rather than fp32 (flex_block_attn_h100.cu:1077-1088);
  * `lse` is the natural-log softmax denominator, shape (B, H, Sq, 1); the reference's value at that position is
    -sqrt(128) times it (flex_block_attn_h100.cu:303-307) and is only ever consumed by its own backward.
"""
import ctypes
import math
import os
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib

HEAD_DIM = 128


@dataclass
class BlockLists:
    """Active-block index lists of one block mask (see include/fba.h, fba_mask_compact).

    With `tiled` set the four tensors are tile lists instead (fba_tile_lists: qt_cnt, qt_ent, kt_cnt, kt_ent), which the
    kernels need when a block size is not a multiple of 128."""

    q_cnt: torch.Tensor  # [mask_bh, nQ] int32
    q_idx: torch.Tensor  # [mask_bh, nQ, nK] int32, ascending, -1 padded
    k_cnt: torch.Tensor  # [mask_bh, nK] int32
    k_idx: torch.Tensor  # [mask_bh, nK, nQ] int32, ascending, -1 padded
    mask_bh: int
    nQ: int
    nK: int
    tiled: bool = False
    # pair numbering for the dS hand-over of backward, filled by `number_pairs`.  Block lists (fba_pair_slots):
    # pair_base [mask_bh * nK + 1], q_slot [mask_bh, nQ, nK].  Tile lists (fba_tile_slots): pair_base
    # [mask_bh * Skv/128 + 1], q_slot [mask_bh, Sq/128, Skv/128] (the slot table), k_slot [mask_bh, Skv/128, Sq/32].
    pair_base: Optional[torch.Tensor] = None  # int32; the last entry is the number of listed pairs
    q_slot: Optional[torch.Tensor] = None     # int32
    k_slot: Optional[torch.Tensor] = None     # int32, tile lists only
    _count: Optional[tuple] = None            # (pinned host copy of pair_base at head boundaries, event after the copy)

    def pair_bounds(self):
        """pair_base at the head boundaries of the mask ([mask_bh + 1] ints, first 0, last = number of listed pairs), read
        from the host copy that `number_pairs` requested; waits for that copy only, not for work enqueued after it."""
        host, event = self._count
        event.synchronize()
        return host.tolist()

    def listed_pairs(self):
        """Number of pairs in the lists (sum of k_cnt)."""
        return int(self.pair_bounds()[-1])

    def transposed(self):
        """Lists of the transposed mask (query and key roles swapped); no device work.  Block lists only."""
        if self.tiled:
            raise ValueError("tile lists cannot be transposed")
        return BlockLists(self.k_cnt, self.k_idx, self.q_cnt, self.q_idx, self.mask_bh, self.nK, self.nQ)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require_device(t, name):
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor (the HIP kernels have no CPU fallback)")


def compact_block_mask(block_mask, with_pair_numbers=False):
    """bool block mask [nQ, nK] or [B, H, nQ, nK] (GPU) -> BlockLists, via the compaction kernel.  `with_pair_numbers`
    also numbers the pairs right away (what the dS hand-over of backward needs; see `number_pairs`)."""
    if block_mask.dtype != torch.bool:
        raise TypeError(f"block_mask must be a bool tensor, got {block_mask.dtype}")
    if block_mask.dim() not in (2, 4):
        raise ValueError(f"block_mask must have 2 or 4 dimensions, got {block_mask.dim()}")
    _require_device(block_mask, "block_mask")
    m = block_mask.contiguous()
    nQ, nK = m.shape[-2], m.shape[-1]
    mask_bh = 1 if m.dim() == 2 else m.shape[0] * m.shape[1]
    dev = m.device
    q_cnt = torch.empty((mask_bh, nQ), dtype=torch.int32, device=dev)
    q_idx = torch.empty((mask_bh, nQ, nK), dtype=torch.int32, device=dev)
    k_cnt = torch.empty((mask_bh, nK), dtype=torch.int32, device=dev)
    k_idx = torch.empty((mask_bh, nK, nQ), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("fba_mask_compact", _ptr(m), mask_bh, nQ, nK, _ptr(q_cnt), _ptr(q_idx), _ptr(k_cnt), _ptr(k_idx), _stream())
    lists = BlockLists(q_cnt, q_idx, k_cnt, k_idx, mask_bh, nQ, nK)
    # numbered right away when a backward pass will follow: the host copy of the pair count is then ordered before
    # whatever the caller enqueues next, and backward finds it without waiting for the forward kernel
    return number_pairs(lists) if with_pair_numbers else lists


def needs_tile_lists(q_block_size, kv_block_size):
    """The kernels work on 128-row tiles: block sizes that are not multiples of 128 go through tile lists."""
    return q_block_size % 128 != 0 or kv_block_size % 128 != 0


def tile_block_mask(block_mask, q_block_size, kv_block_size, with_pair_numbers=False):
    """bool block mask -> tile lists (a BlockLists with `tiled` set), via fba_tile_lists.  `with_pair_numbers` also
    numbers the tile pairs right away (see `number_pairs`)."""
    if block_mask.dtype != torch.bool:
        raise TypeError(f"block_mask must be a bool tensor, got {block_mask.dtype}")
    if block_mask.dim() not in (2, 4):
        raise ValueError(f"block_mask must have 2 or 4 dimensions, got {block_mask.dim()}")
    _require_device(block_mask, "block_mask")
    m = block_mask.contiguous()
    nQ, nK = m.shape[-2], m.shape[-1]
    Sq, Skv = nQ * q_block_size, nK * kv_block_size
    if Sq % 128 or Skv % 128:
        raise _lib.FbaError(_lib.FBA_ERR_UNSUPPORTED, f"tile lists need sequence lengths that are multiples of 128, got {Sq} and {Skv}")
    mask_bh = 1 if m.dim() == 2 else m.shape[0] * m.shape[1]
    i32 = dict(dtype=torch.int32, device=m.device)
    qt_cnt = torch.empty((mask_bh, Sq // 128), **i32)
    qt_ent = torch.empty((mask_bh, Sq // 128, nK), **i32)
    kt_cnt = torch.empty((mask_bh, Skv // 128), **i32)
    kt_ent = torch.empty((mask_bh, Skv // 128, Sq // 32), **i32)
    with torch.cuda.device(m.device):
        _lib.call("fba_tile_lists", _ptr(m), mask_bh, nQ, nK, q_block_size, kv_block_size, _ptr(qt_cnt), _ptr(qt_ent),
                  _ptr(kt_cnt), _ptr(kt_ent), _stream())
    lists = BlockLists(qt_cnt, qt_ent, kt_cnt, kt_ent, mask_bh, nQ, nK, tiled=True)
    return number_pairs(lists) if with_pair_numbers else lists


def lists_for(block_mask, q_block_size, kv_block_size, with_pair_numbers=False):
    """The list flavour the kernels need for these block sizes."""
    if needs_tile_lists(q_block_size, kv_block_size):
        return tile_block_mask(block_mask, q_block_size, kv_block_size, with_pair_numbers)
    return compact_block_mask(block_mask, with_pair_numbers)


def _check_qkv(q, k, v):
    """Tensor contract of the extension (flex_block_attn_h100.cu:820-858)."""
    for name, t in (("q", q), ("k", k), ("v", v)):
        _require_device(t, name)
        if t.dtype != torch.bfloat16:
            raise TypeError(f"{name} must be bfloat16, got {t.dtype}")
        if t.dim() != 4:
            raise ValueError(f"{name} must have shape (batch, heads, seq, head_dim)")
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
    B, Hq, Sq, D = q.shape
    Bk, Hkv, Skv, Dk = k.shape
    if D != HEAD_DIM or Dk != HEAD_DIM or v.shape[3] != HEAD_DIM:
        raise ValueError("head_dim must be 128")
    if Bk != B or v.shape[0] != B:
        raise ValueError("q, k, v batch dimensions must match")
    if v.shape[1] != Hkv or v.shape[2] != Skv:
        raise ValueError("k and v must have the same shape")
    if Hq % Hkv != 0:
        raise ValueError("q heads must be a multiple of kv heads")
    return B, Hq, Hkv, Sq, Skv


def _check_blocks(q, k, q_block_size, kv_block_size, block_mask):
    """Block-size and mask-shape rules (flex_block_attn_interface.py:18-32)."""
    assert q_block_size % 16 == 0, f"q_block_size ({q_block_size}) must be divisible by 16"
    assert kv_block_size % 64 == 0, f"kv_block_size ({kv_block_size}) must be divisible by 64"
    assert kv_block_size % q_block_size == 0 or q_block_size % kv_block_size == 0, (
        f"kv_block_size ({kv_block_size}) must be divisible by q_block_size ({q_block_size}), or vice versa."
    )
    q_seq_len, kv_seq_len = q.shape[2], k.shape[2]
    assert q_seq_len % q_block_size == 0, f"q_seq_len ({q_seq_len}) must be divisible by q_block_size ({q_block_size})"
    assert kv_seq_len % kv_block_size == 0, f"kv_seq_len ({kv_seq_len}) must be divisible by kv_block_size ({kv_block_size})"
    if block_mask.dim() not in (2, 4):
        raise ValueError(f"block_mask must have 2 or 4 dimensions, got {block_mask.dim()}")
    q_block_num, kv_block_num = block_mask.shape[-2], block_mask.shape[-1]
    assert q_block_size * q_block_num == q_seq_len, (
        f"q_block_size ({q_block_size}) * q_block_num ({q_block_num}) must equal q_seq_len ({q_seq_len})"
    )
    assert kv_block_size * kv_block_num == kv_seq_len, (
        f"kv_block_size ({kv_block_size}) * kv_block_num ({kv_block_num}) must equal kv_seq_len ({kv_seq_len})"
    )
    if block_mask.dim() == 4 and tuple(block_mask.shape[:2]) != (q.shape[0], q.shape[1]):
        raise ValueError(
            f"4-D block_mask must be [batch, heads, q_blocks, kv_blocks] = [{q.shape[0]}, {q.shape[1]}, ...], "
            f"got {tuple(block_mask.shape)}"
        )


def _check_lists(lists, q, B, Hq, Sq, Skv, q_block_size, kv_block_size):
    """The kernels index the list tensors by raw pointer: metadata, dtype, device, layout and exact shapes must fit."""
    if lists.nQ * q_block_size != Sq or lists.nK * kv_block_size != Skv:
        raise ValueError("block lists do not match the sequence lengths and block sizes")
    if lists.tiled != needs_tile_lists(q_block_size, kv_block_size):
        raise ValueError("wrong list flavour for these block sizes (see lists_for)")
    if lists.mask_bh not in (1, B * Hq):
        raise ValueError("block lists do not match batch * heads")
    M = lists.mask_bh
    if lists.tiled:
        shapes = ((M, Sq // 128), (M, Sq // 128, lists.nK), (M, Skv // 128), (M, Skv // 128, Sq // 32))
    else:
        shapes = ((M, lists.nQ), (M, lists.nQ, lists.nK), (M, lists.nK), (M, lists.nK, lists.nQ))
    names, tensors = ["q_cnt", "q_idx", "k_cnt", "k_idx"], [lists.q_cnt, lists.q_idx, lists.k_cnt, lists.k_idx]
    if lists.pair_base is not None and lists.tiled:
        names += ["pair_base", "q_slot", "k_slot"]
        tensors += [lists.pair_base, lists.q_slot, lists.k_slot]
        shapes += ((M * (Skv // 128) + 1,), (M, Sq // 128, Skv // 128), (M, Skv // 128, Sq // 32))
    elif lists.pair_base is not None:
        names += ["pair_base", "q_slot"]
        tensors += [lists.pair_base, lists.q_slot]
        shapes += ((M * lists.nK + 1,), (M, lists.nQ, lists.nK))
    for name, t, shape in zip(names, tensors, shapes):
        if t.dtype != torch.int32 or t.device != q.device or not t.is_contiguous() or tuple(t.shape) != shape:
            raise ValueError(f"block lists: {name} must be a contiguous int32 tensor of shape {shape} on {q.device}, "
                             f"got {tuple(t.shape)} {t.dtype} on {t.device}")


# Workspace for tail splitting (see include/fba.h), allocated per call from torch's caching allocator; MiB, 0 switches
# splitting off, unset: what the library's planner can use at most.
SPLIT_WORKSPACE_MIB = os.environ.get("FBA_SPLIT_WORKSPACE_MIB")


def _split_workspace(device):
    """(tensor or None, pointer, bytes) of a fresh tail-splitting workspace on `device`."""
    n = _lib.load().fba_split_workspace_bytes() if SPLIT_WORKSPACE_MIB is None else int(float(SPLIT_WORKSPACE_MIB) * 2 ** 20)
    if n <= 0:
        return None, None, 0
    ws = torch.empty((n,), dtype=torch.uint8, device=device)
    return ws, _ptr(ws), n


def forward_with_lists(q, k, v, q_block_size, kv_block_size, lists):
    """Forward on compacted lists -> (o [B,H,Sq,128] bf16, lse [B,H,Sq,1] fp32)."""
    B, Hq, Hkv, Sq, Skv = _check_qkv(q, k, v)
    _check_lists(lists, q, B, Hq, Sq, Skv, q_block_size, kv_block_size)
    o = torch.empty_like(q)
    lse = torch.empty((B, Hq, Sq, 1), dtype=torch.float32, device=q.device)
    args = (_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(lists.q_cnt), _ptr(lists.q_idx), lists.mask_bh,
            B, Hq, Hkv, Sq, Skv, HEAD_DIM, q_block_size, kv_block_size)
    with torch.cuda.device(q.device):
        _ws, ws_ptr, ws_bytes = _split_workspace(q.device)
        _lib.call("fba_fwd_tiled" if lists.tiled else "fba_fwd", *args, ws_ptr, ws_bytes, _stream())
    return o, lse


def number_pairs(lists):
    """Pair numbering for the dS hand-over, kept on `lists`: block pairs of block lists (fba_pair_slots), pairs of
    128-row tiles of tile lists (fba_tile_slots).  The number of listed pairs, which sizes the workspace, is copied to
    pinned host memory asynchronously; `lists.listed_pairs()` waits for that copy alone."""
    if lists.pair_base is None:
        dev = lists.k_cnt.device
        i32 = dict(dtype=torch.int32, device=dev)
        host = torch.empty((lists.mask_bh + 1,), dtype=torch.int32, pin_memory=True)
        k_slot = None
        with torch.cuda.device(dev):
            if lists.tiled:
                n_qt, n_kt = lists.q_cnt.shape[1], lists.k_cnt.shape[1]
                pair_base = torch.empty((lists.mask_bh * n_kt + 1,), **i32)
                q_slot = torch.empty((lists.mask_bh, n_qt, n_kt), **i32)
                k_slot = torch.empty((lists.mask_bh, n_kt, 4 * n_qt), **i32)
                _lib.call("fba_tile_slots", _ptr(lists.k_cnt), _ptr(lists.k_idx), lists.mask_bh, n_qt, n_kt, _ptr(pair_base),
                          _ptr(k_slot), _ptr(q_slot), _stream())
            else:
                pair_base = torch.empty((lists.mask_bh * lists.nK + 1,), **i32)
                q_slot = torch.empty((lists.mask_bh, lists.nQ, lists.nK), **i32)
                _lib.call("fba_pair_slots", _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.k_cnt), _ptr(lists.k_idx), lists.mask_bh,
                          lists.nQ, lists.nK, _ptr(pair_base), _ptr(q_slot), _stream())
            host.copy_(pair_base[:: lists.k_cnt.shape[1]], non_blocking=True)  # one entry per head of the mask, and the total
            event = torch.cuda.Event()
            event.record()
        lists.pair_base, lists.q_slot, lists.k_slot, lists._count = pair_base, q_slot, k_slot, (host, event)
    return lists


# Largest dS workspace backward allocates on its own: at most DS_WORKSPACE_LIMIT_GIB, and at most DS_WORKSPACE_FACTOR
# times the bytes of the call's own tensors (q, k, v, o, dO, dq, dk, dv), so that backward memory stays proportional to
# the sequence length like the reference's.  A backward pass whose selected pairs need more is run in chunks of heads
# through a workspace within the limit (every head's dS is independent); when not even one kv head fits, or the
# allocation fails, backward recomputes S and dP in the dQ kernel instead (fba_bwd), which needs no workspace.  The
# default of 20 GiB lets the benchmark shapes with 24 heads run in chunks of at least 8 heads, one per XCD (chunks of
# fewer heads are slower per head); FBA_DS_WORKSPACE_LIMIT_GIB=8 costs them up to 9 % of backward.
# (The limit deliberately reads no allocator or driver state: hipMemGetInfo takes milliseconds, and torch's memory
# counters build a dictionary of a few hundred entries per call, enough to trigger a full pass of Python's cyclic garbage
# collector, 40 ms in a process that has torch loaded, every few dozen calls.)
DS_WORKSPACE_LIMIT_GIB = float(os.environ.get("FBA_DS_WORKSPACE_LIMIT_GIB", "20"))
DS_WORKSPACE_FACTOR = float(os.environ.get("FBA_DS_WORKSPACE_FACTOR", "6"))


def ds_workspace_limit(q, k):
    """Bytes of dS workspace the default backward may allocate for these q and k/v shapes."""
    own = (5 * q.numel() + 4 * k.numel()) * 2  # q, o, dO, dq and k, v, dk, dv (bf16)
    return int(min(DS_WORKSPACE_LIMIT_GIB * 2 ** 30, DS_WORKSPACE_FACTOR * own))


def _unit_pairs(lists, B, Hq, Hkv):
    """Listed pairs of every (batch, kv head): the heads of a GQA group share their kv head's launch."""
    bounds = number_pairs(lists).pair_bounds()
    group = Hq // Hkv
    if lists.mask_bh == 1:
        return [bounds[-1] * group] * (B * Hkv), bounds
    return [bounds[(u + 1) * group] - bounds[u * group] for u in range(B * Hkv)], bounds


def ds_workspace_bytes(lists, B, Hq, q_block_size, kv_block_size):
    """(pairs over all heads, bytes of dS workspace) the hand-over backward needs for all heads of these lists at once."""
    listed = number_pairs(lists).listed_pairs()
    pairs = listed * (B * Hq if lists.mask_bh == 1 else 1)
    return pairs, pairs * (128 * 128 if lists.tiled else q_block_size * kv_block_size) * 2


XCDS = 8  # a launch that gives every XCD whole heads of its own runs faster per head than one that makes XCDs share heads


def plan_head_chunks(unit_pairs, pair_bytes, limit_bytes):
    """Cuts the (batch, kv head) units into consecutive chunks of equal length whose dS fits `limit_bytes`: as few chunks
    as the total needs, shortened while some chunk is still too large, and then, if a chunk holds more than one unit per
    XCD, shortened to a multiple of the XCD count (twelve heads per chunk cost dK/dV 3 % against eight).  Returns
    [(first unit, end unit, pairs)], or None when a single unit does not fit."""
    n = len(unit_pairs)
    total = sum(unit_pairs) * pair_bytes
    if total == 0:
        return [(0, n, 0)]

    def cut(per):
        return [(u, min(n, u + per), sum(unit_pairs[u: u + per])) for u in range(0, n, per)]

    def fits(chunks):
        return all(c[2] * pair_bytes <= limit_bytes for c in chunks)

    limit_bytes = int(limit_bytes)
    per = -(-n // max(1, -(-total // max(1, limit_bytes)))) if limit_bytes > 0 else 0
    while per >= 1 and not fits(cut(per)):
        per -= 1
    if per < 1:
        return None
    if per < n and per > XCDS and per % XCDS and fits(cut(per - per % XCDS)):
        per -= per % XCDS
    return cut(per)


def _offset(t, elements):
    """Device pointer `elements` elements into tensor t (may point below t for the shifted dS workspace)."""
    return ctypes.c_void_p(t.data_ptr() + elements * t.element_size())


def backward_with_lists(q, k, v, o, lse, do, q_block_size, kv_block_size, lists, hand_over=None):
    """Backward on compacted lists -> (dq, dk, dv), bf16, shaped like q, k, v.

    hand_over=None (default): the key-major kernel stores dS once and dQ is formed from it (ten products per block
    pair instead of fourteen), in chunks of heads through a workspace of at most `ds_workspace_limit(q, k)` bytes; if not
    even one kv head fits, as False.  True: the same with one workspace for all heads, whatever its size (fba_bwd_handover /
    fba_bwd_tiled_handover in one call).  False: dQ recomputes S and dP (fba_bwd or fba_bwd_tiled, no workspace)."""
    B, Hq, Hkv, Sq, Skv = _check_qkv(q, k, v)
    _check_lists(lists, q, B, Hq, Sq, Skv, q_block_size, kv_block_size)
    if do.dtype != torch.bfloat16:
        do = do.to(torch.bfloat16)
    do = do.contiguous()
    o = o.contiguous()
    if o.shape != q.shape or do.shape != q.shape:
        raise ValueError("o and do must have the shape of q")
    if lse.dtype != torch.float32 or lse.numel() != B * Hq * Sq:
        raise ValueError("lse must be float32 with B*H*Sq elements")
    lse = lse.contiguous()
    dq = torch.empty_like(q)
    dk = torch.empty_like(k)
    dv = torch.empty_like(v)
    pair_bytes = (128 * 128 if lists.tiled else q_block_size * kv_block_size) * 2
    chunks = ds_ws = None
    if hand_over or hand_over is None:
        unit_pairs, bounds = _unit_pairs(lists, B, Hq, Hkv)
        if sum(unit_pairs) > 0:
            chunks = [(0, B * Hkv, sum(unit_pairs))] if hand_over else plan_head_chunks(unit_pairs, pair_bytes, ds_workspace_limit(q, k))
        if chunks is not None:
            try:
                ds_ws = torch.empty((max(c[2] for c in chunks) * pair_bytes,), dtype=torch.uint8, device=q.device)
            except torch.OutOfMemoryError:
                if hand_over:
                    raise
                chunks = None
    group = Hq // Hkv
    M = lists.mask_bh
    with torch.cuda.device(q.device):
        _ws, sp_ptr, sp_bytes = _split_workspace(q.device)
        if chunks is None:
            stats = torch.empty((2, B, Hq, Sq), dtype=torch.float32, device=q.device)
            common = (_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(stats), _ptr(dq), _ptr(dk), _ptr(dv),
                      _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.k_cnt), _ptr(lists.k_idx), M,
                      B, Hq, Hkv, Sq, Skv, HEAD_DIM, q_block_size, kv_block_size)
            if lists.tiled:
                _lib.call("fba_bwd_tiled", *common, sp_ptr, sp_bytes, _stream())
            else:
                _lib.call("fba_bwd", *common, sp_ptr, sp_bytes, _stream())
            return dq, dk, dv
        # one launch sequence per chunk of kv heads [u0, u1): every pointer moves to the chunk's first head, the chunk is
        # described as a batch of one, and the workspace pointer is moved back by the pairs of the heads in front of the
        # chunk, so that the absolute pair numbers of the lists land inside the workspace
        stats = torch.empty((2, max(c[1] - c[0] for c in chunks) * group * Sq), dtype=torch.float32, device=q.device)
        n_qt, n_kt = Sq // 128, Skv // 128
        for u0, u1, pairs in chunks:
            h0, nh, nu = u0 * group, (u1 - u0) * group, u1 - u0
            m0 = h0 if M > 1 else 0  # first row of the per-head list tensors
            qo, ko = h0 * Sq * HEAD_DIM, u0 * Skv * HEAD_DIM
            ws_ptr = ctypes.c_void_p(ds_ws.data_ptr() - (bounds[h0] * pair_bytes if M > 1 else 0))
            shape = (nh if M > 1 else 1, 1, nh, nu, Sq, Skv, HEAD_DIM, q_block_size, kv_block_size)
            if lists.tiled:
                _lib.call(
                    "fba_bwd_tiled_handover", _offset(q, qo), _offset(k, ko), _offset(v, ko), _offset(o, qo), _offset(do, qo), _offset(lse, h0 * Sq),
                    _ptr(stats), ws_ptr, pairs * pair_bytes, _offset(dq, qo), _offset(dk, ko), _offset(dv, ko),
                    _offset(lists.q_cnt, m0 * n_qt), _offset(lists.q_idx, m0 * n_qt * lists.nK), _offset(lists.k_cnt, m0 * n_kt),
                    _offset(lists.k_idx, m0 * n_kt * 4 * n_qt), _offset(lists.pair_base, m0 * n_kt), _offset(lists.k_slot, m0 * n_kt * 4 * n_qt),
                    _offset(lists.q_slot, m0 * n_qt * n_kt), pairs, *shape, sp_ptr, sp_bytes, _stream(),
                )
            else:
                nQ, nK = lists.nQ, lists.nK
                _lib.call(
                    "fba_bwd_handover", _offset(q, qo), _offset(k, ko), _offset(v, ko), _offset(o, qo), _offset(do, qo), _offset(lse, h0 * Sq),
                    _ptr(stats), ws_ptr, pairs * pair_bytes, _offset(dq, qo), _offset(dk, ko), _offset(dv, ko),
                    _offset(lists.q_cnt, m0 * nQ), _offset(lists.q_idx, m0 * nQ * nK), _offset(lists.k_cnt, m0 * nK), _offset(lists.k_idx, m0 * nK * nQ),
                    _offset(lists.pair_base, m0 * nK), _offset(lists.q_slot, m0 * nQ * nK), pairs, *shape, sp_ptr, sp_bytes, _stream(),
                )
    return dq, dk, dv


def _flex_block_attn_forward(q, k, v, q_block_size, kv_block_size, block_mask, small_block_mask, use_small_block_mode):
    """Drop-in for flex_block_attn_interface.py:6-8.  `small_block_mask` is the mask at (q_block x kv_block)
    granularity (it equals `block_mask` when the two block sizes agree); `block_mask`, the max-pooled copy the
    reference's kernel needs, is accepted and ignored."""
    fine = small_block_mask if use_small_block_mode else block_mask
    _check_blocks(q, k, q_block_size, kv_block_size, fine)
    lists = lists_for(fine, q_block_size, kv_block_size)
    return forward_with_lists(q, k, v, q_block_size, kv_block_size, lists)


def _flex_block_attn_backward(q, k, v, o, lse, do, q_block_size, kv_block_size, block_mask, small_block_mask, use_small_block_mode):
    """Drop-in for flex_block_attn_interface.py:10-12.  As in the reference, both masks arrive TRANSPOSED
    ([..., kv_blocks, q_blocks], flex_block_attn_interface.py:85-86)."""
    fine_t = small_block_mask if use_small_block_mode else block_mask
    if fine_t.dim() not in (2, 4):
        raise ValueError(f"block_mask must have 2 or 4 dimensions, got {fine_t.dim()}")
    if needs_tile_lists(q_block_size, kv_block_size):
        lists = tile_block_mask(fine_t.transpose(-1, -2).contiguous(), q_block_size, kv_block_size)
    else:
        lists = compact_block_mask(fine_t).transposed()
    return backward_with_lists(q, k, v, o, lse, do, q_block_size, kv_block_size, lists)


class FlexBlockAttnFunc(torch.autograd.Function):
    """autograd wrapper, same signature as flex_block_attn_interface.py:14-89."""

    @staticmethod
    def forward(ctx, q, k, v, q_block_size, kv_block_size, block_mask, is_grad_enabled):
        _check_blocks(q, k, q_block_size, kv_block_size, block_mask)
        is_grad = is_grad_enabled and any(x.requires_grad for x in [q, k, v])
        lists = lists_for(block_mask, q_block_size, kv_block_size, with_pair_numbers=is_grad)
        o, lse = forward_with_lists(q, k, v, q_block_size, kv_block_size, lists)
        if is_grad:
            ctx.save_for_backward(q, k, v, o, lse)
            ctx.q_block_size = q_block_size
            ctx.kv_block_size = kv_block_size
            ctx.lists = lists  # integer index tensors built here, no part of the autograd graph
        return o

    @staticmethod
    def backward(ctx, dout, *args):
        q, k, v, o, lse = ctx.saved_tensors
        dq, dk, dv = backward_with_lists(q, k, v, o, lse, dout, ctx.q_block_size, ctx.kv_block_size, ctx.lists)
        return dq, dk, dv, None, None, None, None


def flex_block_attn_func(q, k, v, q_block_size, kv_block_size, block_mask):
    """Block-sparse attention: softmax(q k^T / sqrt(128)) v restricted, per query block, to the key blocks that
    `block_mask` selects.

    q: (batch, heads, q_seq_len, 128) bf16; k, v: (batch, kv_heads, kv_seq_len, 128) bf16; block_mask: bool
    [q_seq_len / q_block_size, kv_seq_len / kv_block_size] or [batch, heads, ...]. Returns o shaped like q.
    """
    pad_q = _pad_rows(q.shape[2], q_block_size, kv_block_size)
    pad_k = _pad_rows(k.shape[2], kv_block_size, q_block_size)
    if pad_q == 0 and pad_k == 0:
        return FlexBlockAttnFunc.apply(q, k, v, q_block_size, kv_block_size, block_mask, torch.is_grad_enabled())
    # The kernels work on 128-row tiles.  A sequence that is not a multiple of 128 (possible only with block sizes that
    # are not) is padded with rows that no block selects; the padded query rows come back as zeros and are cut off.
    _check_blocks(q, k, q_block_size, kv_block_size, block_mask)
    F = torch.nn.functional
    qp = F.pad(q, (0, 0, 0, pad_q))
    kp, vp = F.pad(k, (0, 0, 0, pad_k)), F.pad(v, (0, 0, 0, pad_k))
    mp = F.pad(block_mask, (0, pad_k // kv_block_size, 0, pad_q // q_block_size), value=False)
    o = FlexBlockAttnFunc.apply(qp, kp, vp, q_block_size, kv_block_size, mp, torch.is_grad_enabled())
    return o[:, :, : q.shape[2]]


def _pad_rows(seq_len, block, other_block):
    """Rows to append so that a sequence cut into `block`-row blocks becomes a whole number of 128-row tiles (0 when
    both block sizes are multiples of 128: the kernels then never see a partial tile)."""
    if not needs_tile_lists(block, other_block) or seq_len % 128 == 0:
        return 0
    unit = block * 128 // math.gcd(block, 128)
    return -seq_len % unit
