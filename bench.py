#!/usr/bin/env python3
"""Benchmark of the block-sparse attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload random|full|sta|ssta] [--no-cpu]

One step = mask compaction + forward + backward (statistics, dK/dV, dQ) on synthetic inputs already resident in HBM; the
ssta workload also builds its mask from q and k inside the step (block means, scores, top-k).
Default workload: B=1, H=24, S=30720, head_dim 128, bf16, 384-token blocks (80x80), an independent random mask per
(batch, head) keeping 32 of 80 key blocks per query-block row with the diagonal forced on.
FLOPs count selected block pairs only: forward 4*Bq*Bk*D, backward 10*Bq*Bk*D per pair.
Prints ONE JSON line on stdout (everything else goes to stderr).
"""
import argparse
import ctypes
import gc
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0
D = 128

PROFILES = os.path.join(ROOT, "profiles")


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` from the tracked rocprofv3 counter summary of this workload
    (profiles/traffic_<workload>.json: 2 x FETCH_SIZE + WRITE_SIZE KiB, scaled by what a plain copy of known size reads),
    or None when no summary exists or a kernel source is newer than it (a stale figure is worse than none)."""
    path = os.path.join(PROFILES, f"traffic_{workload}.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        rec = json.load(f)
    csrc = os.path.join(ROOT, "flex_block_attn_amd", "csrc")
    for src in rec.get("sources", {}).get(kernel, []):
        if _file_digest(os.path.join(csrc, src)) != rec["digests"].get(src):
            return None
    return rec.get("traffic_bytes", {}).get(kernel)


def _file_digest(path):
    import hashlib

    try:
        with open(path, "rb") as f:
            return hashlib.sha256(f.read()).hexdigest()[:16]
    except OSError:
        return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_workload(name, device, inputs="random"):
    from flex_block_attn_amd import masks

    if name == "random":
        B, H, S, qbs, kbs = 1, 24, 30720, 384, 384
        mask = masks.random_block_mask(B, H, S // qbs, S // kbs, 32, seed=0)
        desc = "dynamic random sparse: B1 H24 S30720 D128 bf16, block 384 (80x80), per-(b,h) mask, 32 of 80 key blocks kept per row (sparsity 0.6), diagonal on"
    elif name == "full":
        B, H, S, qbs, kbs = 1, 24, 11520, 384, 384
        mask = masks.full_block_mask(S // qbs, S // kbs)
        desc = "full attention: B1 H24 S11520 D128 bf16, block 384 (30x30), all-ones 2-D mask"
    elif name == "sta":
        B, H, S, qbs, kbs = 1, 24, 115200, 384, 384
        mask = masks.sta_3d_block_mask((5, 6, 10), (3, 3, 3), clamp=True)
        desc = "3-D sliding-tile mask: B1 H24 S115200 D128 bf16, 300 tiles of 6x8x8=384 tokens, 3x3x3 tile window (clamped), 2-D mask"
    elif name == "ssta":
        B, H, S, qbs, kbs = 1, 24, 69120, 128, 384
        mask = None  # built on the GPU from q and k inside every step
        desc = ("asymmetric score-driven mask: B1 H24 S69120 D128 bf16, q block 128 (540) x k block 384 (180); mask = key block of the "
                "diagonal +-1, key block 0, top-16 key blocks by mean-pooled q . mean-pooled k, built on the GPU inside the step")
    else:
        raise SystemExit(f"unknown workload {name}")
    g = torch.Generator(device="cpu").manual_seed(1234)
    shape = (B, H, S, D)
    q, k, v, do = (torch.randn(shape, generator=g, dtype=torch.float32).to(torch.bfloat16).to(device) for _ in range(4))
    if inputs == "zeros":  # same instruction stream, no data toggling: shows how much of the time is the power limit
        for t in (q, k, v, do):
            t.zero_()
    if mask is None:
        import flex_block_attn_amd as fba

        mask_fn = lambda: fba.create_ssta_mask(q, k, qbs, kbs, topk=16, band=1, sink_blocks=1)
        mask = mask_fn()
    else:
        mask = mask.to(device)
        mask_fn = None
    return dict(B=B, H=H, S=S, qbs=qbs, kbs=kbs, mask=mask, mask_fn=mask_fn, q=q, k=k, v=v, do=do, desc=desc,
                nnz=int(mask.sum().item()) * (1 if mask.dim() == 4 else B * H))


def time_events(fn, warmup, iters):
    """Per-call durations (ms) of fn on torch's current stream, from HIP events around each call."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in evs]


def cpu_baseline(seconds_budget=12.0):
    """The reference's CPU path (dense-mask scaled_dot_product_attention + backward, fp32) as restated by the oracle,
    on this machine's host cores: B1 H2 S1536 D128, 4x4 Bernoulli(0.5) block mask with the diagonal on."""
    from oracle import attn_oracle
    from flex_block_attn_amd import masks

    cores = os.cpu_count() or 1
    threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(threads)
    B, H, S, bs = 1, 2, 1536, 384
    q, k, v, do = attn_oracle.seeded_qkv(B, H, H, S, S, seed=0)
    mask = masks.bernoulli_block_mask(S // bs, S // bs, 0.5, 0)
    attn_oracle.sdpa_dense(q, k, v, mask, bs, bs, do)  # warm-up
    times = []
    t_end = time.perf_counter() + seconds_budget
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 200):
        t0 = time.perf_counter()
        attn_oracle.sdpa_dense(q, k, v, mask, bs, bs, do)
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    dense_flops = 14.0 * S * S * D * H * B
    return {
        "value": dense_flops / med * 1e-12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"oracle sdpa_dense fwd+bwd fp32, B1 H2 S1536 D128 block 384 dense-expanded 4x4 mask, dense FLOPs 14*S^2*D*H, median of {len(times)} runs ({med * 1e3:.1f} ms each), host has {cores} cpus",
    }


def sustained_mfma_tflops(dev, data):
    """TFLOP/s of a register-only loop of v_mfma_f32_32x32x16_bf16 (fba_probe_mfma) on N(0,1) or all-zero operands."""
    from flex_block_attn_amd import _lib
    from flex_block_attn_amd.interface import _ptr, _stream

    wgs, iters = 2048, 100000
    src = torch.randn((1024,), generator=torch.Generator(device="cpu").manual_seed(7)).to(dev) if data == "normal" else None
    sink = torch.empty((wgs * 256,), dtype=torch.float32, device=dev)
    ms = statistics.median(time_events(lambda: _lib.call("fba_probe_mfma", _ptr(src) if src is not None else None, _ptr(sink), wgs, iters, _stream()), 1, 3))
    return wgs * 4.0 * iters * 4 * 32768 / (ms * 1e-3) * 1e-12


def streaming_read_gbs(dev):
    """GB/s at which a kernel that only reads (fba_probe_read: streaming 16-byte loads, nothing stored) pulls 4 GiB from device memory."""
    from flex_block_attn_amd import _lib
    from flex_block_attn_amd.interface import _ptr, _stream

    nbytes = 4 << 30
    src = torch.empty((nbytes,), dtype=torch.uint8, device=dev).fill_(1)
    sink = torch.zeros((1,), dtype=torch.int32, device=dev)
    ms = statistics.median(time_events(lambda: _lib.call("fba_probe_read", _ptr(src), nbytes, _ptr(sink), 2048, _stream()), 1, 5))
    return nbytes / (ms * 1e-3) * 1e-9


def probe_atomics():
    """fp32 atomic adds of 512-byte rows (one query row of dQ) at random rows of a [24 * 30720, 128] fp32 buffer, through
    torch's index_add_ (a gather of src rows + one hardware atomic add per element), against a plain copy of the same bytes.
    The reference's backward adds its dQ partials this way (flex_block_attn_h100.cu:707-708); with 128-key tiles that is
    36 GB of adds per launch of the default workload."""
    dev = torch.device("cuda:0")
    rows, n = 24 * 30720, 4 * 1024 * 1024
    g = torch.Generator(device="cpu").manual_seed(0)
    dst = torch.zeros((rows, D), dtype=torch.float32, device=dev)
    src = torch.randn((n, D), generator=g, dtype=torch.float32).to(dev)
    idx = torch.randint(0, rows, (n,), generator=g).to(dev)
    out = torch.empty_like(src)
    add_ms = statistics.median(time_events(lambda: dst.index_add_(0, idx, src), 2, 5))
    copy_ms = statistics.median(time_events(lambda: out.copy_(src), 2, 5))
    nbytes = src.numel() * 4
    res = {"probe": "fp32 atomic adds, 512-byte rows at random rows of a 377 MB buffer (torch index_add_)", "bytes_added": nbytes,
           "atomic_add_ms": add_ms, "atomic_add_GB/s": nbytes / add_ms * 1e-6, "plain_copy_ms": copy_ms, "plain_copy_GB/s": nbytes / copy_ms * 1e-6,
           "dq_partial_bytes_per_launch_128_key_tiles": 4.0 * 61440 * 384 * 128 * 3, "dq_partial_bytes_per_launch_384_key_owner": 4.0 * 61440 * 384 * 128}
    print(json.dumps(res), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="random")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--recompute", action="store_true", help="backward without the dS workspace (fba_bwd: dQ recomputes S and dP)")
    ap.add_argument("--inputs", choices=["random", "zeros"], default="random",
                    help="zeros: all-zero q, k, v, dO (a probe of the power limit, not a benchmark figure)")
    ap.add_argument("--fwd-tile-rows", choices=["128", "384"], default=None,
                    help="query rows per forward work-group where both kernels apply (measurement of the two forward variants)")
    ap.add_argument("--dkdv-keys-per-wave", choices=["32", "64"], default=None,
                    help="keys per wave of the dK/dV kernel on block lists: 32 (two waves per SIMD, the default) or 64 (one wave per "
                         "SIMD, accumulators in accumulation registers); measurement of the two variants")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy three times, as the known-size yardstick for rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--probe-atomics", action="store_true",
                    help="instead of the benchmark, measure the throughput of fp32 atomic adds into a dQ-sized buffer (what a fused "
                         "backward with reducing stores, as in the reference, would be bound by) and print it")
    args = ap.parse_args()
    if args.probe_atomics:
        return probe_atomics()
    if args.fwd_tile_rows:
        os.environ["FBA_FWD_TILE_ROWS"] = args.fwd_tile_rows
    if args.dkdv_keys_per_wave:
        os.environ["FBA_DKDV_KEYS_PER_WAVE"] = args.dkdv_keys_per_wave
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU only: every box in this build has a single MI355X (use --gpus 1)")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")

    import flex_block_attn_amd as fba
    from flex_block_attn_amd import _lib, interface
    from flex_block_attn_amd.interface import _ptr, _stream

    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = build_workload(args.workload, dev, args.inputs)
    B, H, S, qbs, kbs = w["B"], w["H"], w["S"], w["qbs"], w["kbs"]
    q, k, v, do, mask = w["q"], w["k"], w["v"], w["do"], w["mask"]
    nnz = w["nnz"]
    pair_flops = float(qbs) * kbs * D
    fl_fwd, fl_bwd = 4.0 * pair_flops * nnz, 10.0 * pair_flops * nnz
    log(f"workload: {w['desc']}; nnz block pairs = {nnz}; fwd {fl_fwd * 1e-12:.3f} TFLOP, bwd {fl_bwd * 1e-12:.3f} TFLOP")

    mask_fn = w["mask_fn"]

    def step():
        lists = fba.compact_block_mask(mask_fn() if mask_fn else mask, with_pair_numbers=not args.recompute)
        o, lse = fba.forward_with_lists(q, k, v, qbs, kbs, lists)
        return fba.backward_with_lists(q, k, v, o, lse, do, qbs, kbs, lists, hand_over=False if args.recompute else None)

    # ---- whole-step timing (the contract's K timed steps) -------------------------------------------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # Python's cyclic garbage collector is kept out of the timed region, as timeit does: a full pass over a process with
    # torch loaded takes about 40 ms (two steps) and says nothing about the GPU path
    gc.collect()
    gc.disable()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    gc.enable()
    value = (fl_fwd + fl_bwd) / (ms_per_step * 1e-3) * 1e-12
    # peak memory of one step above what is resident before it (q, k, v, dO, mask): outputs, lists, statistics, the dS
    # workspace of the chunked hand-over, the tail-splitting workspace
    torch.cuda.reset_peak_memory_stats()
    resident = torch.cuda.memory_allocated()
    step()
    torch.cuda.synchronize()
    step_peak_bytes = torch.cuda.max_memory_allocated() - resident

    # ---- per-kernel timing with HIP events on the launch stream -------------------------------------------
    lists = fba.compact_block_mask(mask)
    o, lse = fba.forward_with_lists(q, k, v, qbs, kbs, lists)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    stats = torch.empty((2, B, H, S), dtype=torch.float32, device=dev)
    o2, lse2 = torch.empty_like(o), torch.empty_like(lse)
    common = (lists.mask_bh, B, H, H, S, S, D, qbs, kbs)
    _sp, sp_ptr, sp_bytes = interface._split_workspace(dev)  # tail-splitting workspace, as the operator passes it
    kernels = {
        "mask_compact": lambda: _lib.call("fba_mask_compact", _ptr(mask), lists.mask_bh, lists.nQ, lists.nK, _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.k_cnt), _ptr(lists.k_idx), _stream()),
        "fwd": lambda: _lib.call("fba_fwd", _ptr(q), _ptr(k), _ptr(v), _ptr(o2), _ptr(lse2), _ptr(lists.q_cnt), _ptr(lists.q_idx), *common, sp_ptr, sp_bytes, _stream()),
        "bwd_stats": lambda: _lib.call("fba_bwd_stats", _ptr(o), _ptr(do), _ptr(lse), _ptr(stats), B * H * S, D, _stream()),
        "bwd_dkdv": lambda: _lib.call("fba_bwd_dkdv", _ptr(q), _ptr(k), _ptr(v), _ptr(do), _ptr(stats), _ptr(dk), _ptr(dv), _ptr(lists.k_cnt), _ptr(lists.k_idx), *common, sp_ptr, sp_bytes, _stream()),
        "bwd_dq": lambda: _lib.call("fba_bwd_dq", _ptr(q), _ptr(k), _ptr(v), _ptr(do), _ptr(stats), _ptr(dq), _ptr(lists.q_cnt), _ptr(lists.q_idx), *common, sp_ptr, sp_bytes, _stream()),
    }
    if mask_fn:
        q_mean, k_mean = fba.block_mean(q, qbs), fba.block_mean(k, kbs)
        mask2 = torch.empty_like(mask)
        kernels["block_mean_q"] = lambda: _lib.call("fba_block_mean", _ptr(q), _ptr(q_mean), B * H, S, qbs, D, _stream())
        kernels["block_mean_k"] = lambda: _lib.call("fba_block_mean", _ptr(k), _ptr(k_mean), B * H, S, kbs, D, _stream())
        kernels["ssta_mask"] = lambda: _lib.call("fba_ssta_mask", _ptr(q_mean), _ptr(k_mean), None, _ptr(mask2), B, H, H, S // qbs, S // kbs, qbs, kbs, 16, 1, 1, _stream())
    # the hand-over backward: dK/dV + dS store, then dQ from the stored dS.  The step runs it in chunks of heads through a
    # bounded workspace; the two kernels are timed here on all heads at once (one workspace for everything)
    pairs, ws_bytes = interface.ds_workspace_bytes(lists, B, H, qbs, kbs)
    hand_over = 0 < ws_bytes <= 64 * 2 ** 30 and not args.recompute
    if hand_over:
        ds_ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
        ho = (pairs, lists.mask_bh, B, H, H, S, S, D, qbs, kbs)
        kernels["bwd_dkdv_handover"] = lambda: _lib.call("fba_bwd_dkdv_handover", _ptr(q), _ptr(k), _ptr(v), _ptr(do), _ptr(stats), _ptr(dk), _ptr(dv), _ptr(ds_ws), ws_bytes, _ptr(lists.k_cnt), _ptr(lists.k_idx), _ptr(lists.pair_base), *ho, sp_ptr, sp_bytes, _stream())
        kernels["bwd_dq_from_ds"] = lambda: _lib.call("fba_bwd_dq_from_ds", _ptr(k), _ptr(ds_ws), ws_bytes, _ptr(dq), _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.q_slot), _ptr(lists.pair_base), *ho, sp_ptr, sp_bytes, _stream())
        kernels["pair_slots"] = lambda: _lib.call("fba_pair_slots", _ptr(lists.q_cnt), _ptr(lists.q_idx), _ptr(lists.k_cnt), _ptr(lists.k_idx), lists.mask_bh, lists.nQ, lists.nK, _ptr(lists.pair_base), _ptr(lists.q_slot), _stream())
    iters = max(5, args.steps)
    kms = {}
    for name, fn in kernels.items():
        ts = time_events(fn, max(2, args.warmup), iters)
        kms[name] = {"mean_ms": sum(ts) / len(ts), "median_ms": statistics.median(ts)}
        log(f"kernel {name}: mean {kms[name]['mean_ms']:.4f} ms, median {kms[name]['median_ms']:.4f} ms")

    # executed MFMA FLOPs per selected block pair: forward 2 products, dK/dV kernel 4 (S, dP, dV, dK), recomputing dQ
    # kernel 3, dQ from stored dS 1.  The last is bound by memory: it reads every dS element once (2 bytes per
    # (query, key) of a selected pair), K once and writes dQ.
    kernel_flops = {"fwd": 4.0 * pair_flops * nnz, "bwd_dkdv": 8.0 * pair_flops * nnz, "bwd_dq": 6.0 * pair_flops * nnz}
    if hand_over:
        kernel_flops["bwd_dkdv_handover"] = 8.0 * pair_flops * nnz
    rooflines = {}
    for name, fl in kernel_flops.items():
        ach = fl / (kms[name]["mean_ms"] * 1e-3) * 1e-12
        rooflines[name] = {"bound": "mfma", "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": ach / PEAK_BF16_TFLOPS,
                           "traffic": measured_traffic(args.workload, name), "ms": kms[name]["mean_ms"]}
    if hand_over:
        ds_bytes = 2.0 * qbs * kbs * nnz + 2.0 * B * H * S * D * 2
        ach = ds_bytes / (kms["bwd_dq_from_ds"]["mean_ms"] * 1e-3) * 1e-9
        rooflines["bwd_dq_from_ds"] = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS,
                                       "traffic": measured_traffic(args.workload, "bwd_dq_from_ds"), "ms": kms["bwd_dq_from_ds"]["mean_ms"]}
    in_step = [n for n in rooflines if n not in (("bwd_dkdv", "bwd_dq") if hand_over else ("bwd_dkdv_handover", "bwd_dq_from_ds"))]
    dominant = max(in_step, key=lambda n: kms[n]["mean_ms"])
    roofline = dict(rooflines[dominant])
    roofline["kernel"] = dominant
    # what a bare MFMA loop sustains right now on this GPU, on N(0,1) operands and on zeros (the clock follows the data)
    sustained = {d: sustained_mfma_tflops(dev, d) for d in ("normal", "zeros")}
    log(f"bare MFMA loop: {sustained['normal']:.0f} TFLOP/s on N(0,1) operands, {sustained['zeros']:.0f} on zeros (nominal peak {PEAK_BF16_TFLOPS:.0f})")
    if roofline["bound"] == "mfma":
        roofline["sustained_peak"] = sustained["normal"]
        roofline["frac_of_sustained"] = roofline["achieved"] / sustained["normal"]
    # ... and what a kernel that only reads pulls from device memory: the yardstick of the kernel that reads dS back
    read_gbs = streaming_read_gbs(dev)
    log(f"read-only streaming kernel: {read_gbs:.0f} GB/s (nominal peak {PEAK_HBM_GBS:.0f})")
    if hand_over:
        rooflines["bwd_dq_from_ds"]["streaming_read_GB/s"] = read_gbs
        rooflines["bwd_dq_from_ds"]["frac_of_streaming_read"] = rooflines["bwd_dq_from_ds"]["achieved"] / read_gbs

    mask_bytes = mask.numel() + 4 * (2 * nnz // (1 if mask.dim() == 4 else B * H) + lists.mask_bh * (lists.nQ + lists.nK))
    compaction = {"ms": kms["mask_compact"]["mean_ms"], "algorithmic_bytes": mask_bytes, "GB/s": mask_bytes / (kms["mask_compact"]["mean_ms"] * 1e-3) * 1e-9, "peak_GB/s": PEAK_HBM_GBS}
    bwd_recompute_ms = kms["bwd_stats"]["mean_ms"] + kms["bwd_dkdv"]["mean_ms"] + kms["bwd_dq"]["mean_ms"]
    bwd_ms = kms["bwd_stats"]["mean_ms"] + kms["bwd_dkdv_handover"]["mean_ms"] + kms["bwd_dq_from_ds"]["mean_ms"] if hand_over else bwd_recompute_ms
    detail = {
        "fwd_ms": kms["fwd"]["mean_ms"], "fwd_TFLOP/s": fl_fwd / (kms["fwd"]["mean_ms"] * 1e-3) * 1e-12,
        "bwd_ms": bwd_ms, "bwd_TFLOP/s": fl_bwd / (bwd_ms * 1e-3) * 1e-12,
        "bwd_path": "dS hand-over (fba_bwd_handover)" if hand_over else "recompute (fba_bwd)",
        "bwd_recompute_ms": bwd_recompute_ms, "ds_workspace_GB": ws_bytes * 1e-9,
        "step_peak_memory_GB": step_peak_bytes * 1e-9, "step_ds_workspace_limit_GB": interface.ds_workspace_limit(q, k) * 1e-9,
        "fwd+bwd_kernels_TFLOP/s": (fl_fwd + fl_bwd) / ((bwd_ms + kms["fwd"]["mean_ms"]) * 1e-3) * 1e-12,
        "frac_of_bf16_peak": value / PEAK_BF16_TFLOPS,
        "kernels_ms": {n: kms[n]["mean_ms"] for n in kms},
        "rooflines": rooflines,
        "bare_mfma_loop_TFLOP/s": sustained,
        "streaming_read_GB/s": read_gbs,
        "mask_compaction": compaction,
    }
    if mask_fn:
        pooled = 2.0 * B * H * S * D * 2 + 4.0 * B * H * (S // qbs + S // kbs) * D
        pool_ms = kms["block_mean_q"]["mean_ms"] + kms["block_mean_k"]["mean_ms"]
        detail["mask_build"] = {"block_mean_ms": pool_ms, "block_mean_algorithmic_bytes": pooled, "block_mean_GB/s": pooled / (pool_ms * 1e-3) * 1e-9,
                                "ssta_mask_ms": kms["ssta_mask"]["mean_ms"], "peak_GB/s": PEAK_HBM_GBS}

    if args.calibrate_copy:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        log("calibration: 3 device copies of 268435456 bytes (read 256 MiB + write 256 MiB each)")

    cpu = None if args.no_cpu else cpu_baseline()
    out = {
        "metric": "fwd+bwd effective TFLOP/s (selected-block FLOPs), mask compaction + forward + backward",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic" if args.inputs == "random" else "synthetic, all-zero inputs (power-limit probe, not a benchmark figure)",
        "config": {"workload": w["desc"], "nnz_block_pairs": nnz, "fwd_TFLOP": fl_fwd * 1e-12, "bwd_TFLOP": fl_bwd * 1e-12},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "detail": detail,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
