"""fba_bwd_noalloc (backward with the statistics workspace inside the library's device image) against fba_bwd, through
the C ABI: bit-identical gradients on two calls in a row, the second on a smaller input, so that what the first call
left in the shared workspace cannot leak into the second."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(gpu, B, H, Hkv, S, bs, keep, seed, check_device_free=True):
    import flex_block_attn_amd as fba
    from flex_block_attn_amd import _lib, interface, masks
    from flex_block_attn_amd.interface import _ptr, _stream

    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn((B, H, S, 128), generator=g).to(torch.bfloat16).to(gpu)
    k, v = (torch.randn((B, Hkv, S, 128), generator=g).to(torch.bfloat16).to(gpu) for _ in range(2))
    do = torch.randn((B, H, S, 128), generator=g).to(torch.bfloat16).to(gpu)
    nb = S // bs
    lists = fba.compact_block_mask(masks.random_block_mask(B, H, nb, nb, keep, seed).to(gpu))
    o, lse = fba.forward_with_lists(q, k, v, bs, bs, lists)
    # fba_bwd with a torch-allocated stats buffer and, like fba_bwd_noalloc, without a tail-splitting workspace (splitting
    # changes the order of the fp32 sums of the split tiles)
    saved, interface.SPLIT_WORKSPACE_MIB = interface.SPLIT_WORKSPACE_MIB, "0"
    try:
        want = fba.backward_with_lists(q, k, v, o, lse, do, bs, bs, lists, hand_over=False)
    finally:
        interface.SPLIT_WORKSPACE_MIB = saved
    got = tuple(torch.full_like(t, float("nan")) for t in (q, k, v))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]  # device-wide: would also see a hipMalloc made behind torch's back
    print(f"no-alloc case B{B} H{H} Hkv{Hkv} S{S} block {bs} keep {keep} seed {seed}", flush=True)
    _lib.call("fba_bwd_noalloc", _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(got[0]), _ptr(got[1]), _ptr(got[2]),
              _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.k_cnt), _ptr(lists.k_idx), lists.mask_bh, B, H, Hkv, S, S, 128, bs, bs, _stream())
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    # (the first call on a device maps the library's built-in 32 MiB array, which then stays until the process ends)
    assert not check_device_free or torch.cuda.mem_get_info()[0] == free_before
    for name, a, b in zip(("dq", "dk", "dv"), got, want):
        assert torch.equal(a, b), f"{name} of fba_bwd_noalloc differs from fba_bwd"


def test_no_alloc_backward_matches_backward(gpu):
    _case(gpu, 1, 4, 2, 3072, 384, 4, seed=1, check_device_free=False)   # 12288 query rows
    _case(gpu, 1, 2, 2, 768, 128, 3, seed=2)    # a smaller problem on the same workspace
    _case(gpu, 2, 3, 3, 1536, 384, 2, seed=3)
