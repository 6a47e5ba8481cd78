"""Forward and backward on precompacted lists captured into a HIP graph (torch.cuda.graph) and replayed."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("hand_over,shape", [(False, (4, 1536, 384)), (True, (4, 1536, 384)), (True, (9, 16384, 128))])
def test_step_replays_from_a_captured_graph(gpu, hand_over, shape):
    """The library's launches record into a stream capture (no allocation, synchronisation or host read-back inside the
    C ABI), so a whole step on precompacted lists can be replayed as one graph.  Three replays with eager work and
    synchronisations in between, on fresh inputs written into the captured tensors, each compared bit for bit with the
    eager result on the same inputs.  The third case is large enough (1152 key tiles) for the dK/dV work-groups to claim
    their tiles from counters that a small launch inside the captured sequence zeroes on every replay."""
    import flex_block_attn_amd as fba
    from flex_block_attn_amd import interface, masks

    B, (H, S, bs) = 1, shape
    g = torch.Generator(device="cpu").manual_seed(3)
    new = lambda: torch.randn((B, H, S, 128), generator=g).to(torch.bfloat16).to(gpu)
    q, k, v, do = new(), new(), new(), new()
    mask = masks.random_block_mask(B, H, S // bs, S // bs, max(2, S // bs // 10), seed=1).to(gpu)
    lists = fba.compact_block_mask(mask, with_pair_numbers=True)
    lists.listed_pairs()  # the pair count reaches the host before the capture; nothing inside it waits

    def step():
        o, lse = interface.forward_with_lists(q, k, v, bs, bs, lists)
        dq, dk, dv = interface.backward_with_lists(q, k, v, o, lse, do, bs, bs, lists, hand_over=hand_over)
        return o, dq, dk, dv

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture: first-use attributes, allocator pools
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    for rep in range(3):
        for t in (q, k, v, do):
            t.copy_(new())
        want = [x.clone() for x in step()]
        torch.cuda.synchronize()
        for x in out:
            x.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "dq", "dk", "dv"), out, want):
            assert torch.equal(a, b), (rep, name)
