#!/usr/bin/env python3
"""Benchmark of the gfx950 sparse-attention hot path on one MI355X.

One "step" is one pass of gathered block-sparse attention over the headline workload
(B=2, H=32, N=16384, d=128, 64x64 blocks, 26 of 256 key blocks per q-block row = 10 %
density, seeded synthetic bf16 inputs already resident in HBM).  The JSON line reports
kept-block TFLOP/s (4*64*64*128 flops per kept block), ms per step, the bf16-MFMA
roofline fraction of the attention kernel, the HBM roofline fraction of the mask
compaction stream (``mask_pass``), and a CPU baseline measured on this host's cores.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from fgattn_tk_cuda_amd import capi, workloads as wl  # noqa: E402

# MI355X published peaks
PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBPS = 8000.0

# HBM-side bytes per launch from `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs of this
# file (--only sparse / --only compact), scaled by what the same counters read for the plain
# 1 GiB copy of --only copy (FETCH_SIZE x2.0, WRITE_SIZE x1.0).  Text summaries of those runs
# sit in profiles/counters_*.txt; they are measured offline, not in this process.
TRAFFIC_SPARSE_BYTES = 4.746e9 + 0.2726e9   # rocprofv3 FETCH_SIZE x2.0 + WRITE_SIZE x1.0, see profiles/
TRAFFIC_COMPACT_BYTES = 805.4e6 + 64.5e6    # fetch + write of compact_kernel


# The part raises its clocks over the first tens of milliseconds of sustained load: the same
# kernel measures 1.25 ms over launches 4-13 after idle and 1.07 ms from launch ~100 on.
# Every timed leg therefore first keeps the GPU busy with its own kernel for RAMP_MS (untimed,
# reported as "clock_ramp_ms"), then does the W warm-up launches, then times exactly K launches.
RAMP_MS = 300.0


def clock_ramp(fn, ramp_ms: float = RAMP_MS):
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ramp_ms:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()


def time_steps(fn, steps: int, warmup: int):
    """Average milliseconds of fn() over `steps` launches, HIP events on the launch stream."""
    stream = torch.cuda.current_stream()
    clock_ramp(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record(stream)
    for _ in range(steps):
        fn()
    stop.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall_ms


def bench_sparse(dev, steps, warmup, seed=0):
    c = wl.CONFIGS["cfg3_sparse_16k"]
    B, H, S, D, qblk, kvblk = c["B"], c["H"], c["S"], c["D"], c["qblk"], c["kvblk"]
    nk = wl.ceil_div(S, kvblk)
    count = int(round(c["density"] * nk))
    q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=seed))
    bi, bc = (t.to(dev) for t in wl.uniform_block_lists(B, H, S, qblk, kvblk, count, seed=seed + 1))
    o = torch.empty_like(q)
    lse = torch.empty((B, H, S), dtype=torch.float32, device=dev)

    def step():
        capi.sp_attn_blocks(o, q, k, v, bi, bc, lse=lse, qblk=qblk)

    ms, wall_ms = time_steps(step, steps, warmup)
    kept = int(bc.sum().item())
    flops = wl.kept_block_flops(kept, qblk, kvblk, D)
    if os.environ.get("SPATTN_BENCH_NOCHECK") is None:
        assert torch.isfinite(o.float()).all().item(), "non-finite attention output"
    return dict(ms=ms, wall_ms=wall_ms, flops=flops, kept_blocks=kept, B=B, H=H, S=S, D=D, qblk=qblk, kvblk=kvblk,
                count=count, tensors=(q, k, v, bi, bc, o))


def bench_tokens(dev, steps, warmup, seed=0, res=None):
    """The headline workload handed over the way the reference operator takes it: the same
    kept keys as token-id lists kv_indices [B,H,S/64,S] int32 + counts (sp_attn)."""
    res = res or bench_sparse(dev, 2, 1, seed=seed)
    q, k, v, bi, bc, o = res["tensors"]
    S, qblk = res["S"], res["qblk"]
    tok, num = (t.to(dev) for t in wl.blocks_to_tokens(bi.cpu(), bc.cpu(), S))
    ms, _ = time_steps(lambda: capi.sp_attn(o, q, k, v, tok, num, qblk=qblk), steps, warmup)
    return dict(ms=ms, flops=res["flops"], list_bytes=4.0 * tok.numel())


def bench_zipf(dev, steps, warmup, seed=0):
    """cfg5: B=1 H=8 N=65536 d=128, 128-row q-blocks, per-row block counts ~ Zipf(1.2) clipped to
    [1,1024]: the default schedule against the longest-list-first work order (same results)."""
    c = wl.CONFIGS["cfg5_zipf_64k"]
    B, H, S, D, qblk = c["B"], c["H"], c["S"], c["D"], c["qblk"]
    q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=seed))
    cnt = wl.zipf_counts(B, H, S // qblk, s=c["zipf_s"], lo=1, hi=c["max_blocks"], seed=seed + 3)
    bi, bc = (t.to(dev) for t in wl.ragged_block_lists(B, H, S, qblk, 64, cnt, seed=seed + 4))
    o = torch.empty_like(q)
    order = torch.empty((bc.numel(),), dtype=torch.int32, device=dev)
    flops = 4.0 * float(cnt.sum()) * qblk * 64 * D
    ms0, _ = time_steps(lambda: capi.sp_attn_blocks(o, q, k, v, bi, bc, qblk=qblk), steps, warmup)
    ms_o, _ = time_steps(lambda: capi.qblock_order(order, bc), steps, warmup)

    def ordered():
        capi.qblock_order(order, bc)
        capi.sp_attn_blocks(o, q, k, v, bi, bc, qblk=qblk, order=order)

    ms1, _ = time_steps(ordered, steps, warmup)
    return dict(ms_default=ms0, ms_ordered=ms1, ms_order_kernel=ms_o, flops=flops, kept_blocks=int(cnt.sum()))


def bench_compaction(dev, steps, warmup, seed=0):
    """booleanmask_to_indexmask at the padded threshold workload: B=1, H=24, N=32760 -> mask
    [1,24,256,32768] int32 with ~8 % of the entries set."""
    c = wl.CONFIGS["cfg4_threshold_padded"]
    B, H, S = c["B"], c["H"], c["S"]
    ms_ = 128 * wl.ceil_div(S, 128)
    SB = ms_ // 128
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    mask = (torch.rand((B, H, SB, ms_), device=dev, generator=g) < c["keep"]).to(torch.int32)
    kvi = torch.full((B, H, SB, ms_), ms_, dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)

    def step():
        capi.booleanmask_to_indexmask(kvi, kvn, mask, S)

    ms, _ = time_steps(step, steps, warmup)
    kept = int(kvn.sum().item())
    nbytes = 4.0 * B * H * SB * ms_ + 4.0 * kept + 4.0 * B * H * SB
    return dict(ms=ms, bytes=nbytes, kept=kept, shape=[B, H, SB, ms_])


def bench_packed(dev, steps, warmup, seed=0):
    """The bit-packed mask cache at the same mask: pack_mask (int32 votes -> bits) and
    packedmask_to_indexmask (bits -> index lists, the fused unpack + compaction)."""
    c = wl.CONFIGS["cfg4_threshold_padded"]
    B, H, S = c["B"], c["H"], c["S"]
    ms_ = 128 * wl.ceil_div(S, 128)
    SB = ms_ // 128
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    mask = (torch.rand((B, H, SB, ms_), device=dev, generator=g) < c["keep"]).to(torch.int32)
    packed = torch.empty((B, H, SB, ms_ // 8), dtype=torch.uint8, device=dev)
    kvi = torch.full((B, H, SB, ms_), ms_, dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    ms_pack, _ = time_steps(lambda: capi.pack_mask(packed, mask), steps, warmup)
    ms_idx, _ = time_steps(lambda: capi.packedmask_to_indexmask(kvi, kvn, packed, S), steps, warmup)
    kept = int(kvn.sum().item())
    rows = B * H * SB
    return dict(ms_pack=ms_pack, bytes_pack=4.0 * rows * ms_ + rows * ms_ / 8.0,
                ms_index=ms_idx, bytes_index=rows * ms_ / 8.0 + 4.0 * kept + 4.0 * rows, kept=kept)


def bench_topk(dev, steps, warmup, seed=0, score_pad=0):
    """The top-k mask generator at the threshold workload's shape (B=1, H=24, N=32760, d=64,
    128-row q-blocks), keeping 8 % of the keys per q-block: q-block means, one product per
    head, a radix select per row.  Bytes: q and k once, the bf16 score matrix written and read
    once, the lists written."""
    c = wl.CONFIGS["cfg4_threshold_padded"]
    B, H, S, D = c["B"], c["H"], c["S"], c["D"]
    q, k, _ = (t.to(dev) for t in wl.clustered_qkv(B, H, S, D, seed=seed))
    SB = wl.ceil_div(S, 128)
    Sp = 128 * SB
    select_k = int(round(c["keep"] * S))
    stride = 128 * wl.ceil_div(select_k, 128)
    kvi = torch.full((B, H, SB, stride), stride, dtype=torch.int32, device=dev)
    kvn = torch.zeros((B, H, SB), dtype=torch.int32, device=dev)
    score = torch.empty((B, H, SB, Sp + score_pad), dtype=torch.bfloat16, device=dev)
    qmean = torch.empty((B, H, SB, D), dtype=torch.bfloat16, device=dev)
    ms, _ = time_steps(lambda: capi.qk_topkmask_indices(kvi, kvn, score, qmean, q, k, select_k, blocksz=128), steps, warmup)
    rows = B * H * SB
    nbytes = 2.0 * (q.numel() + k.numel()) + 2.0 * qmean.numel() + 2 * 2.0 * rows * S + 4.0 * rows * select_k + 4.0 * rows
    return dict(ms=ms, bytes=nbytes, select_k=select_k, rows=rows)


def bench_copy(dev, steps, warmup, seed=0):
    """A plain 1 GiB device-to-device copy: the known-size kernel that the FETCH_SIZE /
    WRITE_SIZE counters of the other kernels are scaled by."""
    n = 1 << 28
    a = torch.ones((n,), dtype=torch.float32, device=dev)
    b = torch.empty_like(a)
    ms, _ = time_steps(lambda: b.copy_(a), steps, warmup)
    return dict(ms=ms, read_bytes=4.0 * n, write_bytes=4.0 * n)


def bench_dense(dev, steps, warmup, seed=0):
    c = wl.CONFIGS["cfg2_dense"]
    B, H, S, D = c["B"], c["H"], c["S"], c["D"]
    q, k, v = (t.to(dev) for t in wl.randn_qkv(B, H, S, D, seed=seed))
    o = torch.empty_like(q)
    ms, _ = time_steps(lambda: capi.full_attn(o, q, k, v), steps, warmup)
    return dict(ms=ms, flops=4.0 * B * H * S * S * D)


def bench_sweeps(dev, steps, warmup, seed=0, heads=None):
    """The two QK^T sweeps of the pre-pass (maxq_denom, booleanmask_128) at B=1,H=24,N=32760,d=64."""
    c = wl.CONFIGS["cfg4_threshold_padded"]
    B, H, S, D = c["B"], heads or c["H"], c["S"], c["D"]
    q, k, _ = (t.to(dev) for t in wl.clustered_qkv(B, H, S, D, seed=seed))
    Sp = 128 * wl.ceil_div(S, 128)
    mx = torch.empty((B, H, 1, Sp), device=dev)
    dn = torch.empty((B, H, 1, Sp), device=dev)
    mask = torch.zeros((B, H, Sp // 128, Sp), dtype=torch.int32, device=dev)
    ms1, _ = time_steps(lambda: capi.maxq_denom(mx, dn, q, k), steps, warmup)
    ms2, _ = time_steps(lambda: capi.booleanmask_128(mask, mx, dn, q, k, 1e-3), steps, warmup)
    flops = 2.0 * B * H * float(Sp) * Sp * D
    return dict(ms_maxq_denom=ms1, ms_booleanmask=ms2, flops=flops, mask_bytes=4.0 * mask.numel())


def cpu_baseline(res, budget_s=15.0):
    """Dense-masked PyTorch attention on the host cores over a bounded sample of the
    headline workload: 2048-row slabs of successive heads until the time budget is used."""
    from oracle import cpu_masked_attention as cma

    q, k, v, bi, bc, _ = res["tensors"]
    B, H, S, D, qblk, kvblk = res["B"], res["H"], res["S"], res["D"], res["qblk"], res["kvblk"]
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    chunk = 2048
    rows, kept, t_used, heads = 0, 0, 0.0, 0
    for bh in range(B * H):
        if t_used >= budget_s:
            break
        b, h = divmod(bh, H)
        qh, kh, vh = (t[b, h].float().cpu() for t in (q, k, v))
        bih, bch = bi[b, h].cpu(), bc[b, h].cpu()
        heads += 1
        for r0 in range(0, S, chunk):
            r1 = min(S, r0 + chunk)
            t0 = time.perf_counter()
            cma.masked_attention_rows(qh, kh, vh, bih, bch, r0, r1, qblk, kvblk)
            t_used += time.perf_counter() - t0
            kept += int(bch[r0 // qblk: wl.ceil_div(r1, qblk)].sum())
            rows += r1 - r0
            if t_used >= budget_s:
                break
    flops = wl.kept_block_flops(kept, qblk, kvblk, D)
    return {
        "value": flops / t_used / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": "dense-masked fp32 torch attention (QK^T, -inf outside kept blocks, softmax, PV) on %d query rows "
                  "(%d heads touched) of the %d in the workload, %.1f s; kept-block flops of those rows / time"
                  % (rows, heads, B * H * S, t_used),
        "seconds": t_used,
        "ms_per_step_extrapolated": t_used * (B * H * S / max(rows, 1)) * 1e3,
    }


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-extras", action="store_true", help="only the headline kernel")
    ap.add_argument("--only", default="", help="run one leg only: sparse|tokens|compact|dense|sweeps|copy|packed|topk|zipf (no JSON contract)")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print("bench.py: this library is single-GPU; run with --gpus 1 (got %d)" % args.gpus, file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    capi.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.only:
        fn = {"sparse": bench_sparse, "compact": bench_compaction, "dense": bench_dense, "sweeps": bench_sweeps,
              "copy": bench_copy, "packed": bench_packed, "tokens": bench_tokens, "topk": bench_topk, "zipf": bench_zipf}[args.only]
        r = fn(dev, args.steps, args.warmup)
        r.pop("tensors", None)
        print(json.dumps(r))
        return 0

    res = bench_sparse(dev, args.steps, args.warmup)
    tflops = res["flops"] / (res["ms"] * 1e-3) / 1e12
    out = {
        "metric": "kept-block TFLOP/s, gathered block-sparse attention N=16K d=128 10% density",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms"], "clock_ramp_ms": RAMP_MS, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cfg3: sp_attn over KV-block lists, B=2 H=32 N=16384 d=128, q-block 64, kv-block 64, "
                               "26 of 256 key blocks per row incl. diagonal, bf16 O + fp32 lse",
                   "kept_blocks": res["kept_blocks"], "flops_per_step": res["flops"]},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_SPARSE_BYTES, "traffic_unit": "bytes",
                     "kernel": "attn_fwd_kernel<128,64,KV_BLOCKS>"},
    }
    if not args.no_extras:
        tk = bench_tokens(dev, args.steps, args.warmup, res=res)
        out["token_lists"] = {"workload": "cfg3 with the kept keys as token-id lists (the reference operator's form)",
                              "kernel": "attn_fwd_kernel<128,64,KV_TOKENS>", "ms": tk["ms"],
                              "tflops": tk["flops"] / (tk["ms"] * 1e-3) / 1e12,
                              "mfma_frac": tk["flops"] / (tk["ms"] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
        zp = bench_zipf(dev, max(2, args.steps // 4), 2)
        out["zipf_lists"] = {"workload": "cfg5: B=1 H=8 N=65536 d=128, q-block 128, Zipf(1.2) block counts in [1,1024]",
                             "ms_default_order": zp["ms_default"], "ms_longest_first": zp["ms_ordered"],
                             "order_kernel_ms": zp["ms_order_kernel"],
                             "tflops_longest_first": zp["flops"] / zp["ms_ordered"] / 1e9,
                             "mfma_frac_longest_first": zp["flops"] / zp["ms_ordered"] / 1e9 / PEAK_BF16_TFLOPS}
        cp = bench_compaction(dev, args.steps, args.warmup)
        gbps = cp["bytes"] / (cp["ms"] * 1e-3) / 1e9
        out["mask_pass"] = {"kernel": "compact_kernel (booleanmask_to_indexmask)", "workload": "cfg4 mask %s int32, %.1f%% kept"
                            % (cp["shape"], 100.0 * cp["kept"] / np.prod(cp["shape"])), "ms": cp["ms"],
                            "roofline": {"bound": "hbm", "achieved": gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                                         "frac": gbps / PEAK_HBM_GBPS, "traffic": TRAFFIC_COMPACT_BYTES,
                                         "traffic_unit": "bytes", "algorithmic_bytes": cp["bytes"]}}
        pk = bench_packed(dev, args.steps, args.warmup)
        out["mask_cache"] = {
            "workload": "same mask, bit-packed (1 bit per key)",
            "pack_mask_ms": pk["ms_pack"], "pack_mask_gbps": pk["bytes_pack"] / pk["ms_pack"] / 1e6,
            "pack_mask_hbm_frac": pk["bytes_pack"] / pk["ms_pack"] / 1e6 / PEAK_HBM_GBPS,
            "packedmask_to_indexmask_ms": pk["ms_index"], "packedmask_to_indexmask_gbps": pk["bytes_index"] / pk["ms_index"] / 1e6,
            "packedmask_to_indexmask_hbm_frac": pk["bytes_index"] / pk["ms_index"] / 1e6 / PEAK_HBM_GBPS,
            "algorithmic_bytes": [pk["bytes_pack"], pk["bytes_index"]]}
        tp = bench_topk(dev, max(2, args.steps // 4), 2)
        out["topk_mask"] = {"workload": "cfg4 shape, q-block-mean top-k, %d keys per q-block" % tp["select_k"],
                            "ms": tp["ms"], "gbps": tp["bytes"] / tp["ms"] / 1e6,
                            "hbm_frac": tp["bytes"] / tp["ms"] / 1e6 / PEAK_HBM_GBPS, "algorithmic_bytes": tp["bytes"]}
        dn = bench_dense(dev, args.steps, args.warmup)
        out["dense_full_attn"] = {"workload": "cfg2: B=4 H=16 N=4096 d=64", "ms": dn["ms"],
                                  "tflops": dn["flops"] / (dn["ms"] * 1e-3) / 1e12,
                                  "mfma_frac": dn["flops"] / (dn["ms"] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
        sw = bench_sweeps(dev, max(2, args.steps // 10), 1)
        out["prepass_sweeps"] = {
            "workload": "cfg4: B=1 H=24 N=32760 d=64",
            "maxq_denom_ms": sw["ms_maxq_denom"], "maxq_denom_tflops": sw["flops"] / sw["ms_maxq_denom"] / 1e9,
            "booleanmask_128_ms": sw["ms_booleanmask"], "booleanmask_128_tflops": sw["flops"] / sw["ms_booleanmask"] / 1e9,
            "booleanmask_128_write_gbps": sw["mask_bytes"] / sw["ms_booleanmask"] / 1e6}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(res)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
