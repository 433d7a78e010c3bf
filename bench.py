"""Headline benchmark: paged FlagRot decode attention on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload int4|int2|kivi|mq]

A step is one decode layer-step: one launch of the paged decode attention (through the C ABI of
libflagrot_kernels.so) over the whole batch, on a synthetic cache that is already resident in HBM.  Successive steps
cycle through several distinct copies of the cache so that no page is served from the last-level cache.

Workloads (BASELINE.json configs):
  int4  configs[1]: INT4 FlagRot (key-only 2x2 codebook, kind konlya), Llama-3.1-8B GQA shape 32q/8kv, d=128,
        batch 32, context 8192, page 16, randomly permuted page table.                       [default, headline]
  int2  configs[2]: INT2 FlagRot (kind konlya2) with static key centring, 4 sink + 128 window BF16 tokens,
        batch 64, context 16384.
  kivi  configs[3]: KIVI-style FlagRot INT2 (keys per channel over 32-token groups, values per token), 128-token
        BF16 residual, Qwen-32B shape 64q/8kv, d=128, batch 16, context 32768 (libflagrot_kivi.so).
  mq    configs[4]: prefix-cached multi-query prefill over INT4 pages (libflagrot_mq.so, the MFMA path): 4 requests x
        512 new tokens over a 16384-token cached prefix, Qwen-32B shape 64q/8kv, d=128; --mq-fmt konlya | int4a.
        value = TFLOP/s of the attention (4 x 128 flops per visible (row, key) pair), roofline bound "mfma".
Prints ONE JSON line: value = achieved GB/s of page bytes (the reference's convention: B * L * Hkv * bytes per token),
with `roofline` (HBM, measured with events on the launch stream) and `cpu_baseline` (the numpy oracle's
dequantise-then-attend path, timed on the host on configs[0]'s shape).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

LOG2E = 1.4426950408889634
PEAK_HBM_GBPS = 8000.0
P, HKV, G, DH = 16, 8, 4, 128


def synth_kv(T, g, dev, torch, outliers=4, gain=8.0, mu=None):
    """K ~ N(0,1) with `outliers` channels per head x gain and per-token norms ~ lognormal(0, 0.5); V ~ N(0,1)."""
    kv = torch.randn(T, 2 * HKV, DH, generator=g, device=dev)
    for h in range(HKV):
        ch = torch.randint(0, DH, (outliers,), generator=g, device=dev)
        kv[:, h, ch] *= gain
    kv[:, :HKV] *= torch.exp(0.5 * torch.randn(T, 1, 1, generator=g, device=dev))
    if mu is not None:
        kv[:, :HKV] += mu[None]
    return kv.bfloat16()


def settle(torch, launch, busy_ms=40.0, batch=16):
    """untimed launches until the GPU has been busy for busy_ms (clock ramp out of idle), then a synchronisation"""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    done, i = 0.0, 0
    while done < busy_ms and i < 100000:
        e0.record()
        for _ in range(batch):
            launch(i)
            i += 1
        e1.record()
        torch.cuda.synchronize()
        done += e0.elapsed_time(e1)


def build_cache(torch, K, dev, kind, B, L, seed, kmu=None, chunk_tokens=8192):
    """fills one pool with B sequences of L tokens through the selecting writer; returns pool, block table, calib."""
    g = torch.Generator(device=dev).manual_seed(seed)
    npages = B * ((L + P - 1) // P)
    pool = torch.zeros(npages + 16, HKV, K.cb_chunk_bytes(kind, P), dtype=torch.uint8, device=dev)
    perm = torch.randperm(npages + 16, generator=g, device=dev)[:npages].int()
    bt = perm.view(B, -1).contiguous()
    w = 0.5 + 1.5 * torch.rand(HKV, DH, generator=g, device=dev)
    CT = torch.diag_embed(w).contiguous()                      # C_q = diag(w) (symmetric: C^T = C)
    co = w.contiguous()
    t0 = time.perf_counter()
    for b in range(B):
        for s in range(0, L, chunk_tokens):
            n = min(chunk_tokens, L - s)
            kv = synth_kv(n, g, dev, torch, mu=kmu)
            pos = torch.arange(s, s + n, device=dev)
            slots = bt[b].long()[pos // P] * P + pos % P
            K.cb_write3(kv, slots, CT, co, None, None, kind, pool, P, split=False, kmu=kmu)    # = cb_write bytes
    torch.cuda.synchronize()
    return pool, bt, CT, co, time.perf_counter() - t0


def cpu_baseline(torch, K, dev):
    """the oracle's decode path (page parse + dequantise + inverse transforms + fp64 softmax attention) on
    configs[0]'s shape: batch 1, context 2048, 32q/8kv; the cache bytes come from the HIP writer."""
    import numpy as np
    from oracle import attend as A
    kind, L = "konly", 2048
    pool, bt, CT, co, _ = build_cache(torch, K, dev, kind, 1, L, seed=0)
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, G * HKV, DH, generator=g).bfloat16()
    qb = q.view(torch.int16).numpy().view(np.uint16)
    hp, hbt = pool.cpu().numpy(), bt.cpu().numpy()
    ts = []
    for _ in range(4):
        t0 = time.perf_counter()
        A.decode_reference(qb, hp, kind, P, hbt, [L], 1 / math.sqrt(DH))
        ts.append(time.perf_counter() - t0)
    t = sorted(ts[1:])[len(ts[1:]) // 2]
    nbytes = L * HKV * 144
    try:
        from threadpoolctl import threadpool_info
        cores = max([i.get("num_threads", 1) for i in threadpool_info()] + [1])
    except Exception:
        cores = 1
    return {"value": round(nbytes / t / 1e9, 6), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"numpy oracle decode_reference, B=1 L={L} 32q/8kv INT4 (konly) pages = {nbytes} page bytes, "
                      f"median of 3 after 1 warm-up: {t * 1e6:.0f} us per layer-step; host has {os.cpu_count()} cpus"}


def main_kivi(args, torch, dev):
    """configs[3] through libflagrot_kivi.so: fill by the value writer + key group encoder, time kv_attn."""
    from flagrot_releaser_amd import kivi as KV
    KV.lib()
    B, L, Gq, W, NQ, outl, gain = 16, 32768, 8, 128, 64, 8, 12.0
    name = ("configs[3]: KIVI-style FlagRot INT2 paged decode (per-channel keys over 32-token groups, per-token values), "
            "128-token BF16 residual, Qwen-32B GQA 64q/8kv d=128, B=16 L=32768 page=16")
    CB = KV.chunk_bytes(DH)
    g = torch.Generator(device=dev).manual_seed(3)
    Lp = L - W
    npages = B * (Lp // P)
    pool = torch.zeros(npages + 16, HKV, CB, dtype=torch.uint8, device=dev)
    bt = torch.randperm(npages + 16, generator=g, device=dev)[:npages].int().view(B, -1).contiguous()
    co = (0.5 + 1.5 * torch.rand(HKV, DH, generator=g, device=dev)).contiguous()
    qs = torch.randn(HKV, NQ, DH, generator=g, device=dev).contiguous()
    lz = torch.full((HKV, NQ), 6.0, device=dev)
    t0 = time.perf_counter()
    for b in range(B):
        for s0 in range(0, Lp, 8192):
            n = min(8192, Lp - s0)
            kv = synth_kv(n, g, dev, torch, outliers=outl, gain=gain)
            pos = torch.arange(s0, s0 + n, device=dev)
            slots = bt[b].long()[pos // P] * P + pos % P
            KV.v_write(kv, slots, co, None, pool, HKV, DH)
            KV.k_encode(kv, torch.arange(n, device=dev).view(-1, 32), slots.view(-1, 32).contiguous(), qs, lz,
                        1 / math.sqrt(DH), pool, HKV, DH)
    torch.cuda.synchronize()
    fill_s = time.perf_counter() - t0
    ncopy = max(1, min(8, int(6e9 // pool.numel())))
    pools = [pool] + [pool.clone() for _ in range(ncopy - 1)]
    q = torch.randn(B, Gq * HKV, DH, generator=g, device=dev).bfloat16()
    out = torch.zeros(B, Gq * HKV * DH, dtype=torch.bfloat16, device=dev)
    ring = torch.randn((B + 1) * W, 2 * HKV, DH, generator=g, device=dev).bfloat16()
    tail_len = torch.full((B,), W, dtype=torch.int32, device=dev)
    tail_idx = torch.arange(B, dtype=torch.int32, device=dev)
    cached = torch.full((B,), Lp, dtype=torch.int32, device=dev)
    ns, ch = KV.plan(B, Lp, HKV)
    if args.nsplit:
        ns = args.nsplit
        ch = -(-Lp // ns // 32) * 32
        ns = -(-Lp // ch)
    ws = KV.Workspace(B * HKV * (ns + 1), Gq, DH, dev)
    scale = LOG2E / math.sqrt(DH)

    def step(i):
        KV.attn(q, pools[i % ncopy], bt, cached, out, ns, ch, ws, scale, 0, Gq, ring=ring, tail_len=tail_len,
                tail_idx=tail_idx, T=W)

    for i in range(args.warmup):
        step(i)
    settle(torch, step)              # clocks out of idle
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    ev[0].record()
    for i in range(args.steps):
        step(i)
        ev[i + 1].record()
    torch.cuda.synchronize()
    per = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(args.steps))
    ms_per_step = ev[0].elapsed_time(ev[-1]) / args.steps
    alg_bytes = B * Lp * HKV * (CB // P) + B * W * 2 * HKV * DH * 2
    gbps = alg_bytes / (ms_per_step * 1e-3) / 1e9
    traffic = None
    try:
        with open(os.path.join(ROOT, "profiles", "decode_traffic.json")) as f:
            traffic = json.load(f).get("kivi", {}).get("traffic_bytes")
    except OSError:
        pass
    res = {
        "metric": "paged decode attention: achieved HBM GB/s of page bytes per layer-step (us per layer-step alongside)",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "us_per_layer_step": round(ms_per_step * 1e3, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8 codes, f32 products and accumulate",
        "data": "synthetic", "config": {"workload": name, "nsplit": ns, "chunk": ch, "cache_copies_cycled": ncopy,
                                         "sink": 0, "window": W},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                     "frac": round(gbps / PEAK_HBM_GBPS, 4), "traffic": traffic,
                     "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_us": round(ms_per_step * 1e3, 2),
                     "median_launch_us": round(per[len(per) // 2] * 1e3, 2), "min_launch_us": round(per[0] * 1e3, 2),
                     "note": "one step = kv_attn = the split kernel + the merge kernel"},
        "writer": {"prefill_fill_s": round(fill_s, 3), "prefill_tokens": B * Lp,
                   "note": "value writer + key group encoder (64 calibration queries), includes synthetic input generation"},
    }
    print(json.dumps(res))


def main_mq(args, torch, dev):
    """configs[4] through libflagrot_mq.so: one step = frmq_prep_q + frmq_attn + frmq_merge of one layer."""
    from flagrot_releaser_amd import kernels as K
    from flagrot_releaser_amd import prefill_mq as MQ
    MQ.lib()
    R, NQ, PRE, Gq = 4, 512, 16384, 8
    L = PRE + NQ
    fmt = args.mq_fmt
    k2 = fmt == "konlya"
    name = (f"configs[4]: multi-query prefill over INT4 FlagRot pages ({fmt}), Qwen-32B GQA 64q/8kv d=128, {R} requests x "
            f"{NQ} new tokens over a {PRE}-token cached prefix (L={L}), page=16, causal inside the chunk")
    g = torch.Generator(device=dev).manual_seed(4)
    npg = (L + P - 1) // P
    pool = torch.zeros(R * npg + 16, HKV, 144 * P, dtype=torch.uint8, device=dev)
    bt = torch.randperm(R * npg + 16, generator=g, device=dev)[:R * npg].int().view(R, npg).contiguous()
    w = 0.5 + 1.5 * torch.rand(HKV, DH, generator=g, device=dev)
    CT, co = torch.diag_embed(w).contiguous(), w.contiguous()
    kmask = (torch.rand(HKV, 4, generator=g, device=dev) < 0.5).to(torch.uint8)
    mask = torch.cat([kmask, torch.zeros_like(kmask)]).contiguous()
    for r in range(R):
        for s0 in range(0, L, 8192):
            n = min(8192, L - s0)
            kv = synth_kv(n, g, dev, torch)
            pos = torch.arange(s0, s0 + n, device=dev)
            slots = bt[r].long()[pos // P] * P + pos % P
            if k2:
                K.cb_write(kv, slots, CT, co, fmt, pool, P)
            else:
                K.w3_static_write(kv, slots, mask, None, pool, P, fmt=fmt)
    torch.cuda.synchronize()
    reqs = [(r, r * NQ, (r + 1) * NQ, L, PRE) for r in range(R)]
    plan = MQ.build_plan(reqs, Gq, HKV, 0, dev)
    q = (2.0 * torch.randn(R * NQ, Gq * HKV, DH, generator=g, device=dev)).bfloat16()
    out = torch.zeros(R * NQ, Gq * HKV * DH, dtype=torch.bfloat16, device=dev)
    scale = LOG2E / math.sqrt(DH)

    def step(i):
        q16 = MQ.prep_q(q, scale, Gq, plan.idx, None, None if k2 else kmask)
        opart, ml = MQ.attn(q16, pool, bt, plan, Gq, 0, k2, False)
        MQ.merge(plan, opart, ml, Gq, out=out)

    for i in range(args.warmup):
        step(i)
    settle(torch, step)              # clocks out of idle
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    ev[0].record()
    for i in range(args.steps):
        step(i)
        ev[i + 1].record()
    torch.cuda.synchronize()
    per = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(args.steps))
    ms_per_step = ev[0].elapsed_time(ev[-1]) / args.steps
    pairs = R * Gq * HKV * sum(PRE + t + 1 for t in range(NQ))
    flops = 4.0 * DH * pairs
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    res = {
        "metric": "multi-query prefill attention over INT4 pages: achieved TFLOP/s per layer (ms per layer alongside)",
        "value": round(tflops, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 operands, f32 accumulate", "data": "synthetic",
        "config": {"workload": name, "tiles": plan.ntiles, "items": plan.nitems, "rows_per_tile": plan.rows},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": 2500.0, "unit": "TFLOP/s",
                     "frac": round(tflops / 2500.0, 4), "traffic": None, "algorithmic_flops_per_launch": flops,
                     "avg_launch_us": round(ms_per_step * 1e3, 1), "median_launch_us": round(per[len(per) // 2] * 1e3, 1),
                     "note": "one step = frmq_prep_q + frmq_attn + frmq_merge; the attention kernel dominates"},
    }
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="int4", choices=["int4", "int2", "kivi", "mq"])
    ap.add_argument("--mq-fmt", default="konlya", choices=["konlya", "int4a"])
    ap.add_argument("--nsplit", type=int, default=0, help="override the planner's split count")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU (every (sequence, KV head) is independent: tensor-parallel "
              "ranks own KV heads and exchange nothing here); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from flagrot_releaser_amd import kernels as K
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    if args.workload == "kivi":
        return main_kivi(args, torch, dev)
    if args.workload == "mq":
        return main_mq(args, torch, dev)
    K.lib()
    if args.workload == "int4":
        kind, B, L, S, W, cell = "konlya", 32, 8192, 0, 0, 144
        name = "configs[1]: INT4 FlagRot konlya paged decode, Llama-3.1-8B GQA 32q/8kv d=128, B=32 L=8192 page=16"
    else:
        kind, B, L, S, W, cell = "konlya2", 64, 16384, 4, 128, 80
        name = ("configs[2]: INT2 FlagRot konlya2 paged decode + static key centring + 4 sink / 128 window BF16, "
                "Qwen3-8B GQA 32q/8kv d=128, B=64 L=16384 page=16")
    g = torch.Generator(device=dev).manual_seed(1)
    kmu = None
    if args.workload == "int2":
        kmu = (2.0 * torch.randn(HKV, DH, generator=g, device=dev)).contiguous()
    pool, bt, CT, co, fill_s = build_cache(torch, K, dev, kind, B, L, seed=1, kmu=kmu)
    pool_bytes = pool.numel()
    ncopy = max(1, min(8, int(6e9 // pool_bytes)))
    pools = [pool] + [pool.clone() for _ in range(ncopy - 1)]
    q = torch.randn(B, G * HKV, DH, generator=g, device=dev).bfloat16()
    out = torch.zeros(B, G * HKV * DH, dtype=torch.bfloat16, device=dev)
    T = S + W
    tkw = {}
    Lpages = L - W if T else L                      # the newest W tokens live in the BF16 ring, not in pages
    seq = torch.full((B,), Lpages, dtype=torch.int32, device=dev)
    if T:
        ring = torch.randn(B + 1, T, 2 * HKV, DH, generator=g, device=dev).bfloat16()
        tkw = dict(tail=ring, tail_len=torch.full((B,), T, dtype=torch.int32, device=dev),
                   tail_idx=torch.arange(B, dtype=torch.int32, device=dev), tail_bs=ring.stride(0),
                   tail_ts=ring.stride(1), kv_start=S)
    ns, ch = K.plan_cb(B, Lpages, HKV, P, kind, nsplit=args.nsplit or None)
    ws = K.Workspace(B, HKV, B * HKV * (ns + 1), dev)
    scale = LOG2E / math.sqrt(DH)

    def step(i):
        K.cb_attn(q, pools[i % ncopy], bt, seq, out, ns, ch, ws, scale, kind, **tkw)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    # Launches with pre-bound arguments (checks and pointer marshalling done once, as under graph capture).  The
    # untimed warm-up continues until the GPU has been busy for 40 ms: out of idle the clocks take about that long to
    # settle (the first 200 launches after an idle period measured 86 us per step, every later 200 launches 74-76).
    bound = [K.cb_attn(q, pools[j], bt, seq, out, ns, ch, ws, scale, kind, bound=True, **tkw) for j in range(ncopy)]
    settle(torch, lambda i: bound[i % ncopy]())
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(args.steps):
        bound[i % ncopy]()
        ev[i + 1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(args.steps))
    total_ms = ev[0].elapsed_time(ev[-1])
    ms_per_step = total_ms / args.steps
    page_bytes = B * (Lpages - S) * HKV * cell
    tail_bytes = B * T * 2 * HKV * DH * 2
    alg_bytes = page_bytes + tail_bytes
    gbps = alg_bytes / (ms_per_step * 1e-3) / 1e9

    # decode-step writer (T = B new tokens) and the prefill-time writer rate, for the record
    kv_new = synth_kv(B, g, dev, torch, mu=kmu)
    slots_new = (bt[:, -1].long() * P + (P - 1)).contiguous()
    for _ in range(3):
        K.cb_write(kv_new, slots_new, CT, co, kind, pools[0], P, kmu=kmu)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        K.cb_write(kv_new, slots_new, CT, co, kind, pools[0], P, kmu=kmu)
    e1.record()
    torch.cuda.synchronize()
    writer_us = e0.elapsed_time(e1) / 20 * 1e3

    traffic = None
    try:   # measured with rocprofv3 --pmc (see profiles/k_decode_*_flagrot.txt); not measurable from inside this process
        with open(os.path.join(ROOT, "profiles", "decode_traffic.json")) as f:
            traffic = json.load(f).get(args.workload, {}).get("traffic_bytes")
    except OSError:
        pass
    res = {
        "metric": "paged decode attention: achieved HBM GB/s of page bytes per layer-step (us per layer-step alongside)",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "us_per_layer_step": round(ms_per_step * 1e3, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8 codes, fp16 products, f32 accumulate",
        "data": "synthetic", "config": {"workload": name, "nsplit": ns, "chunk": ch, "cache_copies_cycled": ncopy,
                                         "launch": "eager, arguments bound once",
                                         "sink": S, "window": W},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                     "frac": round(gbps / PEAK_HBM_GBPS, 4), "traffic": traffic,
                     "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_us": round(ms_per_step * 1e3, 2),
                     "median_launch_us": round(per[len(per) // 2] * 1e3, 2), "min_launch_us": round(per[0] * 1e3, 2)},
        "writer": {"decode_step_us": round(writer_us, 2), "decode_step_tokens": B,
                   "prefill_fill_s": round(fill_s, 3), "prefill_tokens": B * L,
                   "note": "prefill_fill_s includes synthetic input generation"},
        "host_wall_s": round(wall, 4),
    }
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline(torch, K, dev)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
