"""Writes tests/golden/*.npz: small seeded cases with the CPU oracle's outputs.

    python tests/golden/make_golden.py

The reference ships no vectors for this path (its only known-answer relation is "equals dense masked SDPA"), so the
fixtures are produced by this repository's oracle after it has been pinned against SDPA, the closed forms and finite
differences (tests/test_oracle.py).  Each file holds the inputs as bf16 bit patterns (int16), the block mask and block
sizes, and the fp32 outputs o, lse, dq, dk, dv plus the compacted index lists.  The GPU parity tests replay them.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import attn_oracle as A  # noqa: E402

CASES = {
    # name: (B, Hq, Hkv, Sq, Skv, q_block, kv_block, mask kind, seed, peaky)
    "square_2x2": (1, 1, 1, 256, 256, 128, 128, "bernoulli", 11, False),
    "band_q128_k384": (1, 1, 1, 384, 768, 128, 384, "band", 12, False),
    "gqa_cross": (1, 2, 1, 128, 256, 128, 128, "per_head", 13, False),
    "peaky_with_empty_row": (1, 1, 1, 384, 384, 128, 128, "empty_row", 14, True),
}


def build_mask(kind, B, Hq, nQ, nK, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    if kind == "bernoulli":
        m = torch.rand((nQ, nK), generator=g) < 0.5
        m[torch.arange(nQ), (torch.arange(nQ) * nK) // nQ] = True
    elif kind == "band":
        i = torch.arange(nQ)[:, None] * nK // nQ
        j = torch.arange(nK)[None, :]
        m = (i - j).abs() < 2
    elif kind == "per_head":
        m = torch.rand((B, Hq, nQ, nK), generator=g) < 0.5
        m[..., torch.arange(nQ), (torch.arange(nQ) * nK) // nQ] = True
    elif kind == "empty_row":
        m = torch.rand((nQ, nK), generator=g) < 0.6
        m[torch.arange(nQ), torch.arange(nQ) % nK] = True
        m[1, :] = False  # a query block that selects nothing
        m[:, 2] = False  # a key block nobody selects
        m[0, 0] = True
    else:
        raise ValueError(kind)
    return m


def make_case(name):
    B, Hq, Hkv, Sq, Skv, qbs, kbs, kind, seed, peaky = CASES[name]
    q, k, v, do = A.seeded_qkv(B, Hq, Hkv, Sq, Skv, seed=seed, peaky=peaky)
    q, k, v, do = (t.to(torch.bfloat16).to(torch.float32) for t in (q, k, v, do))
    mask = build_mask(kind, B, Hq, Sq // qbs, Skv // kbs, seed)
    o, lse = A.c_attention_forward(q, k, v, mask, qbs, kbs)
    dq, dk, dv = A.c_attention_backward(q, k, v, o, lse, do, mask, qbs, kbs)
    q_cnt, q_idx, k_cnt, k_idx = A.compact_lists(mask)
    bits = lambda t: t.to(torch.bfloat16).view(torch.int16).numpy()  # inputs are stored as their exact bf16 bit patterns
    return dict(
        q=bits(q), k=bits(k), v=bits(v), do=bits(do), mask=mask.numpy(), q_block=np.int32(qbs), kv_block=np.int32(kbs),
        o=o.numpy(), lse=lse.numpy(), dq=dq.numpy(), dk=dk.numpy(), dv=dv.numpy(),
        q_cnt=q_cnt, q_idx=q_idx, k_cnt=k_cnt, k_idx=k_idx,
    )


if __name__ == "__main__":
    from oracle import build_oracle

    build_oracle.build_oracle()
    for name in CASES:
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **make_case(name))
        print(path, os.path.getsize(path) // 1024, "KiB")
