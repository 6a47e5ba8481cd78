"""Sweep harness that writes the tables of the reference's benchmark scripts for this implementation.

    python -m flex_block_attn_amd.benchmark --mode random --out results/

Modes, sweeps and CSV layout follow benchmark/{dynamic/random,static/swa,full}/scripts/*.py and *.sh: batch 1, one
head, head_dim 128, block 384, seq_len 11520 ... 84480, sparse rates 0.2 ... 0.8 (random_fwd.sh:4-11); one row per
configuration with the reference's leading columns (batch_size, seq_len, num_heads, head_dim, block_size,
sparse_rate) and its columns for this operator, `ptm_attn_masks`, `ptm_attn_executes` (forward, ms), `ptm_attn_bwd`
(backward through autograd of the scripts' own loss expression, ms) and `ptm_fwd_memory` / `ptm_bwd_memory` (peak bytes
allocated, as torch reports them), so that rows can be set beside the published H800/H20 tables.  Times are means over
`--rep` calls measured with HIP events on the launch stream.
"""
import argparse
import csv
import os

import torch

from . import masks
from .interface import flex_block_attn_func

SEQ_LENS = (11520, 19200, 30720, 38400, 46080, 53760, 61440, 69120, 76800, 84480)
SPARSE_RATES = (0.2, 0.4, 0.6, 0.8)


def append_to_csv(row, filename):
    """Append a dict as one CSV line, writing the header when the file is new (benchmark/utils/utils.py:31-59)."""
    new = not os.path.isfile(filename)
    with open(filename, "a", newline="", encoding="utf-8") as f:
        w = csv.DictWriter(f, fieldnames=list(row.keys()))
        if new:
            w.writeheader()
        w.writerow(row)


def mean_ms(fn, warmup, rep):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(rep)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in evs) / rep


def selected_blocks(mode, q, block_size, sparse_rate, seed):
    """Block pairs per mode, with the reference scripts' reading of `sparse_rate`: random KEEPS int(n * sparse_rate)
    key blocks per row (random_fwd.py:62 passes it as the kept percentage of utils.py:69-83); swa keeps
    |i - j| < int(n * sparse_rate) (swa_fwd.py:63-65); full keeps everything."""
    n = q.shape[2] // block_size
    if mode == "random":
        return masks.generate_selected_blocks(q, block_size, sparse_rate, seed=seed)
    if mode == "swa":
        return masks.generate_swa_selected_blocks(q, block_size, int(n * sparse_rate))
    return [(i, j) for i in range(n) for j in range(n)]


def run_one(mode, batch, seq_len, heads, block_size, sparse_rate, warmup, rep, seed=0):
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(seed)
    q, k, v = (torch.randn((batch, heads, seq_len, 128), generator=g).to(torch.bfloat16).to(dev).requires_grad_(True) for _ in range(3))
    sel = selected_blocks(mode, q, block_size, sparse_rate, seed)
    mask_ms = mean_ms(lambda: masks.create_sparse_mask(q, block_size, sel), 1, max(2, rep // 4))
    mask = masks.create_sparse_mask(q, block_size, sel)
    with torch.no_grad():
        fwd_ms = mean_ms(lambda: flex_block_attn_func(q, k, v, block_size, block_size, mask), warmup, rep)
    torch.cuda.reset_peak_memory_stats()
    out = flex_block_attn_func(q, k, v, block_size, block_size, mask)
    torch.cuda.synchronize()
    fwd_mem = torch.cuda.max_memory_allocated()
    # the reference's scripts time backward on this expression (random_bwd.py:114-122): the result in (batch, seq, heads,
    # dim) layout, made contiguous, summed, squared
    res = out.transpose(1, 2).contiguous()
    loss = res.sum() * res.sum()
    bwd_ms = mean_ms(lambda: loss.backward(retain_graph=True), warmup, rep)
    torch.cuda.reset_peak_memory_stats()
    loss.backward(retain_graph=True)
    torch.cuda.synchronize()
    bwd_mem = torch.cuda.max_memory_allocated()
    head = {"batch_size": batch, "seq_len": seq_len, "num_heads": heads, "head_dim": 128, "block_size": block_size}
    if mode != "full":
        head["sparse_rate"] = sparse_rate
    pairs = int(mask.sum().item()) * batch * heads
    flops = float(block_size) ** 2 * 128 * pairs
    return head, {"ptm_attn_masks": mask_ms, "ptm_attn_executes": fwd_ms}, {"ptm_attn_bwd": bwd_ms}, \
        {"ptm_fwd_memory": fwd_mem, "ptm_bwd_memory": bwd_mem}, \
        {"fwd_TFLOP/s": 4 * flops / fwd_ms * 1e-9, "bwd_TFLOP/s": 10 * flops / bwd_ms * 1e-9}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--mode", choices=["random", "swa", "full"], default="random")
    ap.add_argument("--batch-size", type=int, default=1)
    ap.add_argument("--num-heads", type=int, default=1)
    ap.add_argument("--block-size", type=int, default=384)
    ap.add_argument("--seq-lens", default=",".join(map(str, SEQ_LENS)))
    ap.add_argument("--sparse-rates", default=",".join(map(str, SPARSE_RATES)))
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--rep", type=int, default=10)
    ap.add_argument("--out", default=".")
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("the benchmark needs a GPU")
    os.makedirs(a.out, exist_ok=True)
    rates = [0.0] if a.mode == "full" else [float(x) for x in a.sparse_rates.split(",")]
    for seq_len in (int(x) for x in a.seq_lens.split(",")):
        for rate in rates:
            head, fwd, bwd, mem, rate_info = run_one(a.mode, a.batch_size, seq_len, a.num_heads, a.block_size, rate, a.warmup, a.rep)
            append_to_csv({**head, **fwd}, os.path.join(a.out, f"{a.mode}_fwd_results_{a.block_size}.csv"))
            append_to_csv({**head, **bwd}, os.path.join(a.out, f"{a.mode}_bwd_results_{a.block_size}.csv"))
            append_to_csv({**head, **mem}, os.path.join(a.out, f"{a.mode}_memory_results_{a.block_size}.csv"))
            print({**head, **fwd, **bwd, **mem, **rate_info}, flush=True)


if __name__ == "__main__":
    main()
