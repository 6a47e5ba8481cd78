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
    _count: Optional[tuple] = None            # (pinned host copy of pair_base[-1], event recorded after the copy)

    def listed_pairs(self):
        """Number of pairs in the lists (sum of k_cnt), read from the host copy that `number_pairs` requested; waits
        for that copy only, not for work enqueued after it."""
        host, event = self._count
        event.synchronize()
        return int(host.item())

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


def forward_with_lists(q, k, v, q_block_size, kv_block_size, lists):
    """Forward on compacted lists -> (o [B,H,Sq,128] bf16, lse [B,H,Sq,1] fp32)."""
    B, Hq, Hkv, Sq, Skv = _check_qkv(q, k, v)
    _check_lists(lists, q, B, Hq, Sq, Skv, q_block_size, kv_block_size)
    o = torch.empty_like(q)
    lse = torch.empty((B, Hq, Sq, 1), dtype=torch.float32, device=q.device)
    with torch.cuda.device(q.device):
        _lib.call(
            "fba_fwd_tiled" if lists.tiled else "fba_fwd", _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), _ptr(lists.q_cnt), _ptr(lists.q_idx), lists.mask_bh,
            B, Hq, Hkv, Sq, Skv, HEAD_DIM, q_block_size, kv_block_size, _stream(),
        )
    return o, lse


def number_pairs(lists):
    """Pair numbering for the dS hand-over, kept on `lists`: block pairs of block lists (fba_pair_slots), pairs of
    128-row tiles of tile lists (fba_tile_slots).  The number of listed pairs, which sizes the workspace, is copied to
    pinned host memory asynchronously; `lists.listed_pairs()` waits for that copy alone."""
    if lists.pair_base is None:
        dev = lists.k_cnt.device
        i32 = dict(dtype=torch.int32, device=dev)
        host = torch.empty((1,), dtype=torch.int32, pin_memory=True)
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
            host.copy_(pair_base[-1:], non_blocking=True)
            event = torch.cuda.Event()
            event.record()
        lists.pair_base, lists.q_slot, lists.k_slot, lists._count = pair_base, q_slot, k_slot, (host, event)
    return lists


# Largest dS workspace backward may allocate on its own (GiB); beyond it, or when the allocation fails, backward
# recomputes S and dP in the dQ kernel instead (fba_bwd).
DS_WORKSPACE_LIMIT_GIB = float(os.environ.get("FBA_DS_WORKSPACE_LIMIT_GIB", "64"))


def ds_workspace_bytes(lists, B, Hq, q_block_size, kv_block_size):
    """(pairs over all heads, bytes of dS workspace) the hand-over backward needs for these lists."""
    listed = number_pairs(lists).listed_pairs()
    pairs = listed * (B * Hq if lists.mask_bh == 1 else 1)
    return pairs, pairs * (128 * 128 if lists.tiled else q_block_size * kv_block_size) * 2


def backward_with_lists(q, k, v, o, lse, do, q_block_size, kv_block_size, lists, hand_over=None):
    """Backward on compacted lists -> (dq, dk, dv), bf16, shaped like q, k, v.

    hand_over=True: the key-major kernel stores dS once and dQ is formed from it (fba_bwd_handover or
    fba_bwd_tiled_handover, ten products per block pair); False: dQ recomputes S and dP (fba_bwd or fba_bwd_tiled,
    fourteen products, no workspace); None: hand over when the workspace fits DS_WORKSPACE_LIMIT_GIB and can be
    allocated."""
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
    stats = torch.empty((2, B, Hq, Sq), dtype=torch.float32, device=q.device)
    pairs = ws_bytes = 0
    ds_ws = None
    if hand_over or hand_over is None:
        pairs, ws_bytes = ds_workspace_bytes(lists, B, Hq, q_block_size, kv_block_size)
        if ws_bytes > 0 and (hand_over or ws_bytes <= DS_WORKSPACE_LIMIT_GIB * 2 ** 30):
            try:
                ds_ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=q.device)
            except torch.OutOfMemoryError:
                if hand_over:
                    raise
    hand_over = ds_ws is not None
    with torch.cuda.device(q.device):
        if hand_over and lists.tiled:
            _lib.call(
                "fba_bwd_tiled_handover", _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(stats), _ptr(ds_ws), ws_bytes,
                _ptr(dq), _ptr(dk), _ptr(dv), _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.k_cnt), _ptr(lists.k_idx),
                _ptr(lists.pair_base), _ptr(lists.k_slot), _ptr(lists.q_slot), pairs, lists.mask_bh,
                B, Hq, Hkv, Sq, Skv, HEAD_DIM, q_block_size, kv_block_size, _stream(),
            )
        elif hand_over:
            _lib.call(
                "fba_bwd_handover", _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(stats), _ptr(ds_ws), ws_bytes,
                _ptr(dq), _ptr(dk), _ptr(dv), _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.k_cnt), _ptr(lists.k_idx),
                _ptr(lists.pair_base), _ptr(lists.q_slot), pairs, lists.mask_bh,
                B, Hq, Hkv, Sq, Skv, HEAD_DIM, q_block_size, kv_block_size, _stream(),
            )
        else:
            _lib.call(
                "fba_bwd_tiled" if lists.tiled else "fba_bwd", _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(stats), _ptr(dq), _ptr(dk), _ptr(dv),
                _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.k_cnt), _ptr(lists.k_idx), lists.mask_bh,
                B, Hq, Hkv, Sq, Skv, HEAD_DIM, q_block_size, kv_block_size, _stream(),
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
