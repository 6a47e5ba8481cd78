"""Host-side checks that need no GPU: the C ABI loads and exports every declared symbol, argument validation fails the
way the header says, the Python operator surface mirrors the reference's checks, and the mask helpers behave."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from flex_block_attn_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from flex_block_attn_amd import build

        build.build_library()
    return _lib


def test_every_declared_symbol_is_exported(lib):
    header = open(os.path.join(ROOT, "include", "fba.h")).read()
    declared = set(re.findall(r"\b(fba_[a-z_0-9]+)\s*\(", header))
    assert declared == set(lib.SIGNATURES), "include/fba.h and the ctypes table disagree"
    handle = lib.load()
    for name in declared:
        assert getattr(handle, name) is not None
    assert handle.fba_version() == lib.ABI_VERSION


def _null():
    return ctypes.c_void_p(0)


def _fake(addr=0x1000):
    return ctypes.c_void_p(addr)


def test_c_abi_argument_validation(lib):
    h = lib.load()
    f = _fake()
    # fba_fwd(q,k,v,o,lse,q_cnt,q_idx, mask_bh, B,Hq,Hkv,Sq,Skv,D,q_block,k_block, split_ws,split_ws_bytes, stream)
    ok_shape = (1, 1, 2, 2, 256, 256, 128, 128, 128)

    def fwd(*shape, q=f):
        return h.fba_fwd(q, f, f, f, f, f, f, *shape, _null(), 0, _null())

    bad = [
        ((1, 1, 2, 2, 256, 256, 64, 128, 128), "head_dim"),
        ((1, 1, 3, 2, 256, 256, 128, 128, 128), "multiple of Hkv"),
        ((1, 1, 2, 2, 256, 256, 128, 24, 128), "q_block"),
        ((1, 1, 2, 2, 256, 256, 128, 128, 96), "k_block"),
        ((1, 1, 2, 2, 256, 384, 128, 128, 192), "divide"),
        ((1, 1, 2, 2, 200, 256, 128, 128, 128), "Sq"),
        ((1, 1, 2, 2, 256, 200, 128, 128, 128), "Skv"),
        ((3, 1, 2, 2, 256, 256, 128, 128, 128), "mask_bh"),
        ((1, 0, 2, 2, 256, 256, 128, 128, 128), "positive"),
    ]
    for shape, needle in bad:
        assert fwd(*shape) == lib.FBA_ERR_INVALID, shape
        assert needle in h.fba_last_error().decode(), (shape, h.fba_last_error())
    assert fwd(*ok_shape, q=_null()) == lib.FBA_ERR_INVALID and b"q is null" in h.fba_last_error()
    assert fwd(*ok_shape, q=_fake(0x1008)) == lib.FBA_ERR_INVALID and b"aligned" in h.fba_last_error()
    # a shape the operator allows but no kernel variant covers yet is reported as such, not computed wrongly
    assert fwd(1, 1, 2, 2, 256, 256, 128, 64, 128) == lib.FBA_ERR_UNSUPPORTED
    assert b"q_block" in h.fba_last_error()
    # ... and the tile-list entry points take it, as long as the sequence lengths are multiples of 128
    assert h.fba_fwd_tiled(f, f, f, f, f, f, f, 1, 1, 2, 2, 192, 192, 128, 64, 64, _null(), 0, _null()) == lib.FBA_ERR_UNSUPPORTED
    assert b"multiples of 128" in h.fba_last_error()
    assert h.fba_fwd_tiled(_null(), f, f, f, f, f, f, 1, 1, 2, 2, 256, 256, 128, 64, 64, _null(), 0, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_tile_lists(f, 1, 3, 3, 64, 64, f, f, f, f, _null()) == lib.FBA_ERR_UNSUPPORTED
    assert h.fba_tile_lists(f, 1, 4, 4, 24, 64, f, f, f, f, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_tile_lists(f, 1, 4, 4, 64, 64, f, _null(), f, f, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_bwd_tiled(*([f] * 14), 1, 1, 2, 2, 256, 256, 128, 64, 96, _null(), 0, _null()) == lib.FBA_ERR_INVALID
    # tile-pair numbering and the tile-list backward that hands dS over
    assert h.fba_tile_slots(f, f, 0, 2, 2, f, f, f, _null()) == lib.FBA_ERR_INVALID and b"positive" in h.fba_last_error()
    assert h.fba_tile_slots(f, f, 1, 2, 2, f, _null(), f, _null()) == lib.FBA_ERR_INVALID
    tho = [f] * 8 + [2 * 32768] + [f] * 10
    assert h.fba_bwd_tiled_handover(*tho, 3, 1, 1, 2, 2, 256, 256, 128, 64, 64, _null(), 0, _null()) == lib.FBA_ERR_INVALID
    assert b"3 tile pairs" in h.fba_last_error()
    assert h.fba_bwd_tiled_handover(*tho, 2, 1, 1, 2, 2, 192, 192, 128, 64, 64, _null(), 0, _null()) == lib.FBA_ERR_UNSUPPORTED
    tho[18] = _null()  # slot_table
    assert h.fba_bwd_tiled_handover(*tho, 2, 1, 1, 2, 2, 256, 256, 128, 64, 64, _null(), 0, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_mask_compact(f, 0, 4, 4, f, f, f, f, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_mask_compact(_null(), 1, 4, 4, f, f, f, f, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_bwd_stats(f, f, f, f, 16, 64, _null()) == lib.FBA_ERR_INVALID
    # caller-side helpers
    assert h.fba_block_mean(f, f, 4, 256, 24, 128, _null()) == lib.FBA_ERR_INVALID and b"multiple of 16" in h.fba_last_error()
    assert h.fba_block_mean(f, f, 4, 256, 96, 128, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_block_mean(f, f, 4, 256, 64, 64, _null()) == lib.FBA_ERR_INVALID and b"head_dim" in h.fba_last_error()
    assert h.fba_block_mean(_null(), f, 4, 256, 64, 128, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_ssta_mask(f, f, _null(), f, 1, 3, 2, 4, 4, 128, 128, 2, 1, 1, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_ssta_mask(f, f, _null(), f, 1, 2, 2, 4, 5000, 128, 128, 2, 1, 1, _null()) == lib.FBA_ERR_UNSUPPORTED
    assert h.fba_ssta_mask(f, f, _null(), _null(), 1, 2, 2, 4, 4, 128, 128, 2, 1, 1, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_ssta_mask(f, f, _null(), f, 1, 2, 2, 4, 4, 128, 128, -1, 1, 1, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_tile_permute(f, _fake(0x2000), 1, 6, 8, 9, 6, 8, 8, 128, 1, _null()) == lib.FBA_ERR_INVALID and b"divide" in h.fba_last_error()
    assert h.fba_tile_permute(f, f, 1, 6, 8, 8, 6, 8, 8, 128, 1, _null()) == lib.FBA_ERR_INVALID and b"alias" in h.fba_last_error()
    assert h.fba_probe_mfma(_null(), f, 0, 10, _null()) == lib.FBA_ERR_INVALID and h.fba_probe_mfma(_null(), _null(), 4, 10, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_probe_read(f, 32768 + 16, f, 4, _null()) == lib.FBA_ERR_INVALID and h.fba_probe_read(_null(), 32768, f, 4, _null()) == lib.FBA_ERR_INVALID
    assert h.fba_probe_read(f, 32768, f, 0, _null()) == lib.FBA_ERR_INVALID
    # FbaError carries the code and the library's message
    with pytest.raises(lib.FbaError) as ei:
        lib.call("fba_mask_compact", f, 0, 4, 4, f, f, f, f, _null())
    assert ei.value.code == lib.FBA_ERR_INVALID and "positive" in ei.value.message
    # a 4-D mask is indexed by the QUERY head: with grouped kv heads a mask with one slice per kv head is rejected
    assert h.fba_fwd(f, f, f, f, f, f, f, 2, 1, 4, 2, 256, 256, 128, 128, 128, _null(), 0, _null()) == lib.FBA_ERR_INVALID
    assert b"mask_bh" in h.fba_last_error()
    assert h.fba_bwd(*([f] * 14), 2, 1, 4, 2, 256, 256, 128, 128, 128, _null(), 0, _null()) == lib.FBA_ERR_INVALID and b"mask_bh" in h.fba_last_error()
    # backward validates every argument before its first launch: a bad gradient pointer is reported, nothing is enqueued
    bwd_args = [f] * 14
    bwd_args[7] = _null()  # dq
    assert h.fba_bwd(*bwd_args, 1, 1, 2, 2, 256, 256, 128, 128, 128, _null(), 0, _null()) == lib.FBA_ERR_INVALID and b"dq is null" in h.fba_last_error()
    # the tail-splitting workspace is optional; when given it must be 16-byte aligned with a size that is not negative
    assert h.fba_fwd(f, f, f, f, f, f, f, *ok_shape, _fake(0x1008), 1 << 20, _null()) == lib.FBA_ERR_INVALID and b"split_ws" in h.fba_last_error()
    assert h.fba_fwd(f, f, f, f, f, f, f, *ok_shape, f, -1, _null()) == lib.FBA_ERR_INVALID and b"split_ws_bytes" in h.fba_last_error()
    assert h.fba_split_workspace_bytes() >= 32 * 2 ** 20


def test_operator_surface_names():
    import flex_block_attn
    import flex_block_attn_amd as fba

    for name in ("flex_block_attn_func", "_flex_block_attn_forward", "_flex_block_attn_backward"):
        assert getattr(flex_block_attn, name) is getattr(fba, name)
    # the reference's module path (flex_block_attn/__init__.py:1-5 imports from .flex_block_attn_interface)
    from flex_block_attn.flex_block_attn_interface import FlexBlockAttnFunc, _flex_block_attn_backward, _flex_block_attn_forward, flex_block_attn_func

    assert FlexBlockAttnFunc is fba.FlexBlockAttnFunc and flex_block_attn_func is fba.flex_block_attn_func
    assert _flex_block_attn_forward is fba._flex_block_attn_forward and _flex_block_attn_backward is fba._flex_block_attn_backward
    from benchmark.utils import utils as ref_path  # the module path the reference's scripts import from

    assert ref_path.create_sparse_mask is fba.masks.create_sparse_mask and ref_path.generate_selected_blocks is fba.masks.generate_selected_blocks
    q, k, v = ref_path.generate_input(1, 8, 2, 128, "cpu")
    assert q.shape == (1, 8, 2, 128) and q.dtype == torch.bfloat16 and q.requires_grad
    import inspect

    assert list(inspect.signature(fba.flex_block_attn_func).parameters) == ["q", "k", "v", "q_block_size", "kv_block_size", "block_mask"]
    assert list(inspect.signature(fba._flex_block_attn_forward).parameters) == [
        "q", "k", "v", "q_block_size", "kv_block_size", "block_mask", "small_block_mask", "use_small_block_mode"]
    assert list(inspect.signature(fba._flex_block_attn_backward).parameters) == [
        "q", "k", "v", "o", "lse", "do", "q_block_size", "kv_block_size", "block_mask", "small_block_mask", "use_small_block_mode"]


def test_shape_rules_match_reference_asserts():
    """Same conditions as flex_block_attn_interface.py:18-32, raised before anything touches a device."""
    from flex_block_attn_amd.interface import _check_blocks

    q = torch.zeros((1, 2, 768, 128), dtype=torch.bfloat16)
    k = torch.zeros((1, 2, 768, 128), dtype=torch.bfloat16)
    m = torch.ones((2, 2), dtype=torch.bool)
    _check_blocks(q, k, 384, 384, m)
    with pytest.raises(AssertionError, match="divisible by 16"):
        _check_blocks(q, k, 24, 384, m)
    with pytest.raises(AssertionError, match="divisible by 64"):
        _check_blocks(q, k, 384, 96, m)
    with pytest.raises(AssertionError, match="vice versa"):
        _check_blocks(q, k, 48, 64, torch.ones((16, 12), dtype=torch.bool))
    with pytest.raises(AssertionError, match="q_seq_len"):
        _check_blocks(q, k, 512, 256, m)
    with pytest.raises(AssertionError, match="q_block_num"):
        _check_blocks(q, k, 384, 384, torch.ones((3, 2), dtype=torch.bool))
    with pytest.raises(AssertionError, match="kv_block_num"):
        _check_blocks(q, k, 384, 384, torch.ones((2, 3), dtype=torch.bool))
    with pytest.raises(ValueError, match="2 or 4"):
        _check_blocks(q, k, 384, 384, torch.ones((1, 2, 2), dtype=torch.bool))
    with pytest.raises(ValueError, match="4-D block_mask"):
        _check_blocks(q, k, 384, 384, torch.ones((1, 3, 2, 2), dtype=torch.bool))


def test_no_cpu_fallback():
    """CPU tensors are rejected: the product has no path that avoids the HIP kernels."""
    import flex_block_attn_amd as fba

    q = torch.zeros((1, 1, 128, 128), dtype=torch.bfloat16)
    m = torch.ones((1, 1), dtype=torch.bool)
    with pytest.raises(ValueError, match="GPU tensor"):
        fba.flex_block_attn_func(q, q, q, 128, 128, m)
    with pytest.raises(ValueError, match="GPU tensor"):
        fba.compact_block_mask(m)
    with pytest.raises(TypeError, match="bool"):
        fba.compact_block_mask(m.to(torch.uint8))


def test_tensor_contract():
    from flex_block_attn_amd.interface import _check_qkv

    good = torch.zeros((1, 2, 256, 128), dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="GPU tensor"):
        _check_qkv(good, good, good)


def test_mask_helpers():
    from flex_block_attn_amd import masks

    q = torch.zeros((1, 1, 1536, 128))
    sel = masks.generate_selected_blocks(q, 384, 0.5, seed=3)
    assert len(sel) == 4 * 2 and sel == masks.generate_selected_blocks(q, 384, 0.5, seed=3)
    for i in range(4):
        cols = [j for (r, j) in sel if r == i]
        assert len(cols) == 2 and len(set(cols)) == 2
    bm = masks.create_sparse_mask(q, 384, sel)
    assert bm.shape == (4, 4) and bm.dtype == torch.bool and int(bm.sum()) == 8
    dense = masks.create_torch_mask(q, 384, sel)
    assert dense.shape == (1536, 1536) and torch.equal(dense[::384, ::384], bm)
    assert torch.equal(dense, masks.expand_block_mask(bm, 384, 384))
    swa = masks.generate_swa_selected_blocks(q, 384, 2)
    assert set(swa) == {(i, j) for i in range(4) for j in range(4) if abs(i - j) < 2}
    assert torch.equal(masks.create_sparse_mask(q, 384, swa), masks.swa_block_mask(4, 4, 2))

    r = masks.random_block_mask(1, 3, 80, 80, 32, seed=0)
    assert r.shape == (1, 3, 80, 80) and (r.sum(-1) == 32).all() and r.diagonal(dim1=-2, dim2=-1).all()
    assert torch.equal(r, masks.random_block_mask(1, 3, 80, 80, 32, seed=0))
    assert not torch.equal(r[0, 0], r[0, 1])

    sta = masks.sta_3d_block_mask((5, 6, 10), (3, 3, 3), clamp=True)
    assert sta.shape == (300, 300) and (sta.sum(-1) == 27).all() and sta.diagonal().all()
    clipped = masks.sta_3d_block_mask((5, 6, 10), (3, 3, 3), clamp=False)
    assert int(clipped.sum()) == 5824 and torch.equal(clipped, clipped.t())


@pytest.mark.parametrize("tiles,window", [((5, 6, 10), (3, 3, 3)), ((2, 3, 5), (3, 3, 3)), ((1, 2, 2), (3, 3, 3)), ((3, 1, 4), (1, 3, 5)),
                                          ((4, 2, 3), (5, 1, 3)), ((2, 2, 7), (1, 1, 5))])
@pytest.mark.parametrize("clamp", [False, True])
def test_sliding_tile_mask_against_oracle(oracle, tiles, window, clamp):
    """masks.sta_3d_block_mask against the oracle's loop restatement over (t, h, w) tile coordinates, on asymmetric
    grids (a swapped axis or another tile enumeration changes the result), with axes shorter than the window."""
    from flex_block_attn_amd import masks

    got = masks.sta_3d_block_mask(tiles, window, clamp=clamp)
    want = oracle.sta_3d_mask(tiles, window, clamp=clamp)
    assert got.dtype == torch.bool and torch.equal(got, want)
    swapped = oracle.sta_3d_mask((tiles[0], tiles[2], tiles[1]), (window[0], window[2], window[1]), clamp=clamp)
    if tiles[1] != tiles[2] and (tiles[1] > 1 and tiles[2] > 1):
        assert not torch.equal(got, swapped)  # the comparison does tell the axes apart


def test_block_lists_transposed_view():
    from flex_block_attn_amd.interface import BlockLists

    a, b, c, d = (torch.zeros(1) for _ in range(4))
    t = BlockLists(a, b, c, d, 1, 3, 5).transposed()
    assert t.q_cnt is c and t.q_idx is d and t.k_cnt is a and t.k_idx is b and (t.nQ, t.nK) == (5, 3)
    with pytest.raises(ValueError, match="transposed"):
        BlockLists(a, b, c, d, 1, 3, 5, tiled=True).transposed()


def test_list_flavour_follows_block_sizes():
    from flex_block_attn_amd.interface import _pad_rows, needs_tile_lists

    assert _pad_rows(30720, 384, 384) == 0 and _pad_rows(256, 64, 64) == 0 and _pad_rows(1536, 128, 384) == 0
    assert _pad_rows(192, 64, 64) == 64 and _pad_rows(80, 16, 64) == 48 and _pad_rows(144, 48, 192) == 240
    assert _pad_rows(576, 192, 48) == 192 and _pad_rows(192, 64, 128) == 64 and _pad_rows(384, 128, 64) == 0

    assert not needs_tile_lists(128, 128) and not needs_tile_lists(384, 256)
    assert needs_tile_lists(64, 128) and needs_tile_lists(128, 192) and needs_tile_lists(16, 64)


def test_benchmark_harness_tables(tmp_path):
    """CSV layout and block selection of the sweep harness follow the reference scripts (utils.py:31-59, :69-92)."""
    from flex_block_attn_amd import benchmark

    f = tmp_path / "t.csv"
    benchmark.append_to_csv({"batch_size": 1, "seq_len": 768, "ptm_attn_executes": 0.5}, str(f))
    benchmark.append_to_csv({"batch_size": 1, "seq_len": 1536, "ptm_attn_executes": 0.7}, str(f))
    assert f.read_text().splitlines() == ["batch_size,seq_len,ptm_attn_executes", "1,768,0.5", "1,1536,0.7"]
    q = torch.zeros((1, 1, 3840, 128))
    sel = benchmark.selected_blocks("random", q, 384, 0.6, seed=0)
    assert len(sel) == 10 * 6  # sparse_rate is the KEPT fraction in the reference's scripts
    swa = benchmark.selected_blocks("swa", q, 384, 0.2, seed=0)
    assert set(swa) == {(i, j) for i in range(10) for j in range(10) if abs(i - j) < 2}
    assert len(benchmark.selected_blocks("full", q, 384, 0.0, seed=0)) == 100
    assert benchmark.SEQ_LENS[0] == 11520 and benchmark.SEQ_LENS[-1] == 84480 and benchmark.SPARSE_RATES == (0.2, 0.4, 0.6, 0.8)


def test_block_lists_are_validated_before_any_launch():
    """A BlockLists whose tensors do not fit the call (shape, dtype, layout) is rejected on the host: the kernels index
    them by raw pointer."""
    from flex_block_attn_amd.interface import BlockLists, _check_lists

    q = torch.zeros((1, 2, 256, 128), dtype=torch.bfloat16)
    i32 = dict(dtype=torch.int32)

    def lists(q_idx_shape=(1, 2, 2), dtype=torch.int32, mask_bh=1):
        return BlockLists(torch.zeros((mask_bh, 2), **i32), torch.zeros(q_idx_shape, dtype=dtype), torch.zeros((mask_bh, 2), **i32),
                          torch.zeros((mask_bh, 2, 2), **i32), mask_bh, 2, 2)

    _check_lists(lists(), q, 1, 2, 256, 256, 128, 128)
    _check_lists(lists((2, 2, 2), mask_bh=2), q, 1, 2, 256, 256, 128, 128)
    with pytest.raises(ValueError, match="q_idx"):
        _check_lists(lists((1, 2, 3)), q, 1, 2, 256, 256, 128, 128)
    with pytest.raises(ValueError, match="q_idx"):
        _check_lists(lists(dtype=torch.int64), q, 1, 2, 256, 256, 128, 128)
    with pytest.raises(ValueError, match="batch \\* heads"):
        _check_lists(lists((3, 2, 2), mask_bh=3), q, 1, 2, 256, 256, 128, 128)
    bad = lists()
    bad.k_idx = torch.zeros((1, 2, 4), **i32)[:, :, ::2]
    with pytest.raises(ValueError, match="k_idx"):
        _check_lists(bad, q, 1, 2, 256, 256, 128, 128)
    with pytest.raises(ValueError, match="sequence lengths"):
        _check_lists(lists(), q, 1, 2, 512, 256, 128, 128)
    numbered = lists()
    numbered.pair_base, numbered.q_slot = torch.zeros((3,), **i32), torch.zeros((1, 2, 2), **i32)
    _check_lists(numbered, q, 1, 2, 256, 256, 128, 128)
    numbered.pair_base = torch.zeros((4,), **i32)
    with pytest.raises(ValueError, match="pair_base"):
        _check_lists(numbered, q, 1, 2, 256, 256, 128, 128)
    tiled = BlockLists(torch.zeros((1, 2), **i32), torch.zeros((1, 2, 4), **i32), torch.zeros((1, 2), **i32), torch.zeros((1, 2, 8), **i32), 1, 4, 4, tiled=True)
    _check_lists(tiled, q, 1, 2, 256, 256, 64, 64)
    tiled.k_idx = torch.zeros((1, 2, 4), **i32)
    with pytest.raises(ValueError, match="k_idx"):
        _check_lists(tiled, q, 1, 2, 256, 256, 64, 64)
    tiled.k_idx = torch.zeros((1, 2, 8), **i32)
    tiled.pair_base, tiled.q_slot, tiled.k_slot = torch.zeros((3,), **i32), torch.zeros((1, 2, 2), **i32), torch.zeros((1, 2, 8), **i32)
    _check_lists(tiled, q, 1, 2, 256, 256, 64, 64)
    tiled.k_slot = torch.zeros((1, 2, 4), **i32)
    with pytest.raises(ValueError, match="k_slot"):
        _check_lists(tiled, q, 1, 2, 256, 256, 64, 64)


def test_no_alloc_backward_rejects_oversized_problems(lib):
    """fba_bwd_noalloc serves at most 2^22 query rows from its built-in workspace and says so beyond that, before it
    touches a device."""
    h = lib.load()
    f = _fake()
    rc = h.fba_bwd_noalloc(*([f] * 13), 1, 1, 64, 64, 128 * 1024, 128 * 1024, 128, 128, 128, _null())
    assert rc == lib.FBA_ERR_UNSUPPORTED and b"exceed the built-in workspace" in h.fba_last_error()


def test_build_check_finds_a_write_in_front_of_an_asm_matrix_instruction():
    """build.find_asm_mfma_hazards: a vector instruction that writes an A / B operand of an accumulation-register matrix
    instruction at most a few instructions earlier is reported, also across a label (the block may be fallen into);
    writes of other registers, writes further away and the compiler's own (vector-register) matrix instructions are not."""
    from flex_block_attn_amd.build import find_asm_mfma_hazards

    mfma = "v_mfma_f32_32x32x16_bf16 a[224:239], v[54:57], v[50:53], a[224:239]"
    bad = "\n".join(["v_mov_b64_e32 v[50:51], s[40:41]", "s_waitcnt lgkmcnt(6)", mfma])
    assert [(w.split()[0], d) for w, _m, d in find_asm_mfma_hazards(bad)] == [("v_mov_b64_e32", 2)]
    assert find_asm_mfma_hazards("\n".join(["v_cvt_pk_bf16_f32 v57, v1, v2", mfma]))[0][2] == 1
    assert find_asm_mfma_hazards("\n".join(["v_mov_b32_e32 v58, 0", "ds_read_b64_tr_b16 v[54:55], v9", mfma])) == []
    far = "\n".join(["v_mov_b32_e32 v50, 0"] + ["s_nop 0"] * 4 + [mfma])
    assert find_asm_mfma_hazards(far) == []
    assert len(find_asm_mfma_hazards("\n".join(["v_mov_b32_e32 v50, 0", ".LBB0_7:", mfma]))) == 1
    assert find_asm_mfma_hazards("\n".join(["v_mov_b32_e32 v50, 0", "v_mfma_f32_32x32x16_bf16 v[0:15], v[54:57], v[50:53], v[0:15]"])) == []
