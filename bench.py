"""Headline benchmark: paged FlagRot decode attention on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload int4|int2|kivi|mq] [--only]

A step is one decode layer-step: one launch of the paged decode attention (through the C ABI of
libflagrot_kernels.so) over the whole batch, on a synthetic cache that is already resident in HBM.  Successive steps
cycle through several distinct copies of the cache so that no page is served from the last-level cache.

Timing: after W warm-up steps and a clock-settling run, the K steps are timed between two events on the launch stream in
two submissions, 7 times each: (a) captured into ONE HIP graph and replayed (the reference's method,
scripts/bench_attn_int2.py:42-64 of the reference), (b) launched eagerly with arguments bound once.  Each carries an
overhead of its own on top of the steps' device time -- a graph replay has a fixed begin / end cost on the device (5-9 us
per replay, measured with a copy kernel), which a short graph (K = 20) does not amortise; eager launches leave gaps when
the host falls behind -- so the figures come from the smaller of the two MEDIANS; both are in the record (`graph_us`,
`eager_us`, `timing_used`).

Workloads (BASELINE.json configs):
  int4  configs[1]: INT4 FlagRot (key-only 2x2 codebook, kind konlya), Llama-3.1-8B GQA shape 32q/8kv, d=128,
        batch 32, context 8192, page 16, randomly permuted page table.                       [default, headline]
  int2  configs[2]: INT2 FlagRot (kind konlya2) with static key centring, 4 sink + 128 window BF16 tokens,
        batch 64, context 16384.
  int2_b32  INT2 FlagRot (kind konlya2) at the headline shape: batch 32, context 8192, no BF16 rows.
  kivi  configs[3]: KIVI-style FlagRot INT2 (keys per channel over 32-token groups, values per token), 128-token
        BF16 residual, Qwen-32B shape 64q/8kv, d=128, batch 16, context 32768 (libflagrot_kivi.so).
  mq    configs[4]: prefix-cached multi-query prefill over INT4 pages (libflagrot_mq.so, the MFMA path): 4 requests x
        512 new tokens over a 16384-token cached prefix, Qwen-32B shape 64q/8kv, d=128; --mq-fmt konlya | int4a.
        value = TFLOP/s of the attention (4 x 128 flops per visible (row, key) pair), roofline bound "mfma".
Prints ONE JSON line for the chosen workload: value = achieved GB/s of page bytes (the reference's convention:
B * L * Hkv * bytes per token), `roofline`, `cpu_baseline` (the numpy oracle's writer and dequantise-then-attend legs
timed on the host on configs[0]'s shape, one thread) and `checked` (sampled sequences of the timed launch's output
compared with the oracle, outside the timed region).  Without --workload (the default run) the other three workloads
are run as short legs as well and reported under `workloads`, and configs[1] is also run with the split plan the
reference's own host planner makes from this library's occupancy answer (`reference_planner`).
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
PEAK_F16_TFLOPS = 2500.0
P, HKV, G, DH = 16, 8, 4, 128
ATOL, RTOL = 2e-3, 1e-2          # the bar of the attention outputs: |out - ref| <= ATOL + RTOL |ref|
REPLAYS = 7
TRAFFIC_FILE = "profiles/decode_traffic.json"


def synth_kv(T, g, dev, torch, outliers=4, gain=8.0, mu=None, hkv=HKV, dh=DH):
    """K ~ N(0,1) with `outliers` channels per head x gain and per-token norms ~ lognormal(0, 0.5); V ~ N(0,1)."""
    kv = torch.randn(T, 2 * hkv, dh, generator=g, device=dev)
    for h in range(hkv):
        ch = torch.randint(0, dh, (outliers,), generator=g, device=dev)
        kv[:, h, ch] *= gain
    kv[:, :hkv] *= torch.exp(0.5 * torch.randn(T, 1, 1, generator=g, device=dev))
    if mu is not None:
        kv[:, :hkv] += mu[None]
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


def timed(torch, launch, steps, warmup, eager=None):
    """launch(i): step i on torch's current stream.  W warm-up steps, clock settling, then (a) the K steps eagerly
    (through `eager(i)` when given: the same step with pre-bound arguments) and (b) the K steps as one HIP graph
    replayed REPLAYS times.  Returns per-step microseconds: graph median / min replay, eager average."""
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    run = eager or launch
    settle(torch, run)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    eager = []
    for _ in range(REPLAYS):
        e0.record()
        for i in range(steps):
            run(i)
        e1.record()
        torch.cuda.synchronize()
        eager.append(e0.elapsed_time(e1) / steps * 1e3)
    eager.sort()
    eager_us = eager[len(eager) // 2]
    cur = torch.cuda.current_stream()
    side = torch.cuda.Stream()
    side.wait_stream(cur)
    with torch.cuda.stream(side):
        launch(0)                               # the capture stream's first use of every library, outside the capture
    cur.wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(steps):
            launch(i)
    graph.replay()
    torch.cuda.synchronize()
    settle(torch, run)
    reps = []
    for _ in range(REPLAYS):
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        reps.append(e0.elapsed_time(e1) / steps * 1e3)
    reps.sort()
    del graph
    graph_us = reps[len(reps) // 2]
    # Both spans hold exactly the same K steps between two events on the launch stream; each carries its own overhead on
    # top of the steps' device time (a graph replay has a fixed begin / end cost on the device -- 5 to 9 us per replay,
    # measured with a copy kernel, which K = 20 steps do not amortise; eager launches can leave gaps when the host falls
    # behind), so the smaller median is the tighter measurement of the steps themselves.  Both are reported.
    best = min(graph_us, eager_us)
    return {"us": best, "timing_used": "graph replay" if best == graph_us else "eager launches (bound arguments)",
            "graph_us": graph_us, "graph_min_us": reps[0], "graph_max_us": reps[-1], "eager_us": eager_us,
            "eager_min_us": eager[0]}


def within(got, ref):
    """worst |got - ref| / (ATOL + RTOL |ref|) over all elements (<= 1: inside the bar)"""
    import numpy as np
    return float((np.abs(got - ref) / (ATOL + RTOL * np.abs(ref))).max())


def error_stats(got, ref):
    """the three yardsticks in use for attention outputs: `elementwise` = within() (the bar of the FlagRot decode),
    `max_over_max` = max |err| / max |ref| (the reference's bar for its KIVI kernels, tests/test_kivi.py:243: 1e-2),
    `rel_l2` = |err|_2 / |ref|_2 (what the reference reports for its multi-query prefill next to BF16 FlashAttention's
    ~3e-3, scripts/bench_mq_prefill.py:42,221-235)"""
    import numpy as np
    err = np.abs(got - ref)
    return {"elementwise": within(got, ref), "max_over_max": float(err.max() / max(np.abs(ref).max(), 1e-30)),
            "rel_l2": float(np.linalg.norm(err) / max(np.linalg.norm(ref), 1e-30))}


def describe(st):
    return (f"worst |err| / (2e-3 + 1e-2 |ref|) = {st['elementwise']:.3f}, max |err| / max |ref| = {st['max_over_max']:.2e}, "
            f"relative L2 = {st['rel_l2']:.2e}")


def build_cache(torch, K, dev, kind, B, L, seed, kmu=None, chunk_tokens=8192, hkv=HKV, dh=DH):
    """fills one pool with B sequences of L tokens through the selecting writer; returns pool, block table, calib."""
    g = torch.Generator(device=dev).manual_seed(seed)
    npages = B * ((L + P - 1) // P)
    pool = torch.zeros(npages + 16, hkv, K.cb_chunk_bytes(kind, P) * (dh // 128), dtype=torch.uint8, device=dev)
    perm = torch.randperm(npages + 16, generator=g, device=dev)[:npages].int()
    bt = perm.view(B, -1).contiguous()
    w = 0.5 + 1.5 * torch.rand(hkv, dh, generator=g, device=dev)
    CT = torch.diag_embed(w).contiguous()                      # C_q = diag(w) (symmetric: C^T = C)
    co = w.contiguous()
    t0 = time.perf_counter()
    for b in range(B):
        for s in range(0, L, chunk_tokens):
            n = min(chunk_tokens, L - s)
            kv = synth_kv(n, g, dev, torch, mu=kmu, hkv=hkv, dh=dh)
            pos = torch.arange(s, s + n, device=dev)
            slots = bt[b].long()[pos // P] * P + pos % P
            if dh == 128:
                K.cb_write3(kv, slots, CT, co, None, None, kind, pool, P, split=False, kmu=kmu)    # = cb_write bytes
            else:
                K.cb_write(kv, slots, CT, co, kind, pool, P, kmu=kmu)
    torch.cuda.synchronize()
    return pool, bt, CT, co, time.perf_counter() - t0


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or "unknown"


def blas_threads(limit=None):
    """context that pins numpy's thread pools to `limit` threads (None: as the host gives them), and the count in use"""
    import contextlib
    try:
        from threadpoolctl import threadpool_info, threadpool_limits
    except Exception:      # no threadpoolctl: numpy runs with whatever its BLAS was built with
        return contextlib.nullcontext(), None
    if limit is None:
        n = max([i.get("num_threads", 1) for i in threadpool_info()] or [1])
        return contextlib.nullcontext(), n
    return threadpool_limits(limits=limit), limit


def median_time(fn, runs=5):
    fn()                                   # one warm-up
    ts = []
    for _ in range(runs):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[len(ts) // 2]


def configs0(torch, K, dev, runs=5, timed_legs=True):
    """configs[0] (batch 1, context 2048, 32q/8kv, head dim 128, page 16, INT4 key-only pages of kind konly with groups
    of 32, uniform calibration weights C_q = I and c_o = 1, identity page order) through BOTH paths on the same seeded
    inputs: the oracle's writer + page packer + dequantise-then-attend on the host, and the HIP writer + decode through
    the C ABI.  Returns the comparison (pool bytes equal, attention inside the bar) and, when asked, the host timings:
    median of `runs` after one warm-up, with one thread and with the host's own thread count."""
    import numpy as np
    from oracle import attend as A
    from oracle import pages as PG
    from oracle import quant as Q
    kind, L = "konly", 2048
    g = torch.Generator(device=dev).manual_seed(0)
    kv = synth_kv(L, g, dev, torch)
    gq = torch.Generator().manual_seed(0)
    q = torch.randn(1, G * HKV, DH, generator=gq).bfloat16()
    kvb = kv.cpu().view(torch.int16).numpy().view(np.uint16)
    qb = q.view(torch.int16).numpy().view(np.uint16)
    C = np.stack([np.eye(DH, dtype=np.float32)] * HKV)
    npages = L // P
    slots = np.arange(L, dtype=np.int64)
    hbt = np.arange(npages, dtype=np.int32)[None]
    cb = PG.chunk_bytes(kind, P)

    def write_host():
        pool = np.zeros((npages, HKV, cb), dtype=np.uint8)
        codes, words, _ = Q.k2_encode(kvb, C, kind)
        PG.pack_tokens(pool, slots, codes, words, kind, P)
        return pool

    want = write_host()
    ref = A.decode_reference(qb, want, kind, P, hbt, [L], 1 / math.sqrt(DH))
    # the same inputs through the HIP libraries
    dpool = torch.zeros(npages, HKV, cb, dtype=torch.uint8, device=dev)
    CT = torch.eye(DH, device=dev).repeat(HKV, 1, 1).contiguous()
    co = torch.ones(HKV, DH, device=dev)
    K.cb_write(kv, torch.from_numpy(slots).to(dev), CT, co, kind, dpool, P)
    torch.cuda.synchronize()
    same = bool(np.array_equal(dpool.cpu().numpy(), want))
    out = torch.zeros(1, G * HKV * DH, dtype=torch.bfloat16, device=dev)
    ns, ch = K.plan_cb(1, L, HKV, P, kind)
    ws = K.Workspace(1, HKV, HKV * (ns + 1), dev)
    K.cb_attn(q.to(dev), dpool, torch.from_numpy(hbt).to(dev), torch.tensor([L], dtype=torch.int32, device=dev), out, ns, ch,
              ws, LOG2E / math.sqrt(DH), kind)
    torch.cuda.synchronize()
    got = out.view(1, G * HKV, DH).float().cpu().numpy().astype(np.float64)
    st = error_stats(got, ref)
    res = {"pool_bytes_equal": same, "errors": st, "nsplit": ns, "chunk": ch,
           "checked": bool(same and st["elementwise"] <= 1.0),
           "check": f"configs[0] through the HIP path: writer pool {'byte-equal to' if same else 'DIFFERS from'} the "
                    f"oracle's packed pool ({want.size} bytes); decode vs the oracle's dequantise-then-attend: " + describe(st)}
    if not timed_legs:
        return res
    legs = {}
    for label, limit in (("one_thread", 1), ("host_threads", None)):
        ctx, n = blas_threads(limit)
        with ctx:
            tw = median_time(write_host, runs)
            td = median_time(lambda: A.decode_reference(qb, want, kind, P, hbt, [L], 1 / math.sqrt(DH)), runs)
        legs[label] = {"threads": n, "writer_s": tw, "decode_s": td}
    res["legs"] = legs
    return res


def cpu_baseline(torch, K, dev):
    """the oracle's two legs on configs[0], timed on this host: (i) the selecting writer for the 2048 tokens x 8 KV heads
    (K with selection, V plain) + page packing, (ii) one decode step = page parse + dequantise + inverse transforms +
    fp64 softmax attention for the 32 q heads.  The same inputs go through the HIP path and the two are compared."""
    L = 2048
    r = configs0(torch, K, dev)
    one, full = r["legs"]["one_thread"], r["legs"]["host_threads"]
    nbytes = L * HKV * 144
    t = one["decode_s"]
    return {"value": round(nbytes / t / 1e9, 6), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"numpy oracle on configs[0] (B=1 L={L} 32q/8kv INT4 konly, C_q = I, c_o = 1, page 16), median of 5 runs "
                      f"after one warm-up, one thread: decode step (decode_reference, {nbytes} page bytes) = {t * 1e6:.0f} us "
                      f"per layer-step; writer (k2_encode + pack_tokens, {L} tokens x {HKV} KV heads, K and V) = "
                      f"{one['writer_s']:.2f} s = {one['writer_s'] / L * 1e6:.0f} us per token",
            "decode_us_per_layer_step": round(t * 1e6, 0), "writer_us_per_token": round(one["writer_s"] / L * 1e6, 1),
            "host_threads": {"threads": full["threads"], "decode_us_per_layer_step": round(full["decode_s"] * 1e6, 0),
                             "GBps": round(nbytes / full["decode_s"] / 1e9, 6),
                             "writer_us_per_token": round(full["writer_s"] / L * 1e6, 1)},
            "cpu": cpu_model(), "os_cpu_count": os.cpu_count(), "torch_num_threads": torch.get_num_threads(),
            "checked": r["checked"], "pool_bytes_equal": r["pool_bytes_equal"], "errors": r["errors"], "check": r["check"]}


def reference_plan(B, Lmax, Hkv, slots):
    """the split plan a caller written against the reference makes for a key-only kind: smallest modelled cost
    ceil(B Hkv ns / slots) (chunk + 1024) + 4 ns [ns > 1] over chunks of whole 64-token blocks of at most 8192 tokens,
    slots = (what fr_cb_occupancy returns) x (multi_processor_count); integrations/vllm_flagrot/vllm_flagrot/
    kernels.py:247-265 of the reference."""
    best = None
    for ns in range(max(1, math.ceil(Lmax / 8192)), min(512, math.ceil(Lmax / 64)) + 1):
        chunk = math.ceil(Lmax / ns / 64) * 64
        if chunk > 8192:
            continue
        nse = math.ceil(Lmax / chunk)
        if best is not None and nse == best[1]:
            continue
        cost = math.ceil(B * Hkv * nse / slots) * (chunk + 1024) + (4 * nse if nse > 1 else 0)
        if best is None or cost < best[0] - 1e-9:
            best = (cost, nse, chunk)
    return best[1], best[2]


# ------------------------------------------------------------------------------------------------ FlagRot decode
def run_flagrot(args, torch, dev, workload, steps, warmup, plans=("own",)):
    """configs[1] / configs[2] through libflagrot_kernels.so.  Returns {plan: result dict}."""
    import numpy as np
    from flagrot_releaser_amd import kernels as K
    from oracle import attend as A
    K.lib()
    if workload == "int4":
        kind, B, L, S, W, cell = "konlya", 32, 8192, 0, 0, 144
        name = "configs[1]: INT4 FlagRot konlya paged decode, Llama-3.1-8B GQA 32q/8kv d=128, B=32 L=8192 page=16"
    elif workload == "int2_b32":
        kind, B, L, S, W, cell = "konlya2", 32, 8192, 0, 0, 80
        name = ("INT2 FlagRot konlya2 paged decode at the headline shape (the metric names INT4 and INT2): Llama-3.1-8B "
                "GQA 32q/8kv d=128, B=32 L=8192 page=16, no BF16 rows")
    else:
        kind, B, L, S, W, cell = "konlya2", 64, 16384, 4, 128, 80
        name = ("configs[2]: INT2 FlagRot konlya2 paged decode + static key centring + 4 sink / 128 window BF16, "
                "Qwen3-8B GQA 32q/8kv d=128, B=64 L=16384 page=16")
    HKV, DH, G = globals()["HKV"], globals()["DH"], globals()["G"]
    if getattr(args, "batch", 0) or getattr(args, "context", 0) or getattr(args, "window", -1) >= 0:
        # shape overrides for experiments: not a baseline configuration
        B, L = getattr(args, "batch", 0) or B, getattr(args, "context", 0) or L
        if getattr(args, "window", -1) >= 0:
            W = args.window
            S = S if W else 0
        name += f" [shape override: B={B} L={L} sink={S} window={W}: not a baseline configuration]"
    if getattr(args, "gqa", 4) != 4:              # not a configuration of the baseline: GQA groups of 8 (Qwen-32B's 64q/8kv) on the same pages
        G = int(args.gqa)
        name = name.replace("32q/8kv", f"{G * HKV}q/{HKV}kv") + f" [GQA {G}: not a baseline configuration]"
    if getattr(args, "head_dim", 128) == 256:     # not a configuration of the baseline: the head dim 256 kernels, same page bytes
        HKV, DH, G = 4, 256, 6
        name = (f"{'INT4' if workload == 'int4' else 'INT2'} FlagRot {kind} paged decode at head dim 256, GQA 24q/4kv, B={B} "
                f"L={L} page=16" + (f", {S} sink / {W} window BF16" if S + W else "") + " (no baseline configuration)")
        cell *= 2
    g = torch.Generator(device=dev).manual_seed(1)
    kmu = None
    if workload == "int2":
        kmu = (2.0 * torch.randn(HKV, DH, generator=g, device=dev)).contiguous()
    pool, bt, CT, co, fill_s = build_cache(torch, K, dev, kind, B, L, seed=1, kmu=kmu, hkv=HKV, dh=DH)
    ncopy = max(1, min(8, int(6e9 // pool.numel())))
    pools = [pool] + [pool.clone() for _ in range(ncopy - 1)]
    q = torch.randn(B, G * HKV, DH, generator=g, device=dev).bfloat16()
    out = torch.zeros(B, G * HKV * DH, dtype=torch.bfloat16, device=dev)
    T = S + W
    tkw = {}
    Lpages = L - W if T else L                      # the newest W tokens live in the BF16 ring, not in pages
    seq = torch.full((B,), Lpages, dtype=torch.int32, device=dev)
    ring = None
    if T:
        ring = torch.randn(B + 1, T, 2 * HKV, DH, generator=g, device=dev).bfloat16()
        tkw = dict(tail=ring, tail_len=torch.full((B,), T, dtype=torch.int32, device=dev),
                   tail_idx=torch.arange(B, dtype=torch.int32, device=dev), tail_bs=ring.stride(0),
                   tail_ts=ring.stride(1), kv_start=S)
    scale = LOG2E / math.sqrt(DH)
    page_bytes = B * (Lpages - S) * HKV * cell
    tail_bytes = B * T * 2 * HKV * DH * 2
    alg_bytes = page_bytes + tail_bytes
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    results = {}
    for plan in plans:
        if plan == "own":
            ns, ch = K.plan_cb(B, Lpages, HKV, P, kind, nsplit=args.nsplit or None, G=G, Dh=DH)
            if getattr(args, "chunk", 0):
                ns, ch = math.ceil(Lpages / args.chunk), args.chunk
        else:      # "reference": the reference front end's cost model fed with this library's occupancy answer
            occ = K.lib().fr_cb_occupancy(K.CB_KINDS[kind], 0, K.STAGES, P)
            ns, ch = reference_plan(B, Lpages, HKV, max(1, occ) * cus)
        if DH == 128 and G == 4:
            ws = K.Workspace(B, HKV, B * HKV * (ns + 1), dev)
        else:
            hv = K.vheads(HKV, G, DH, kind)
            ws = K.Workspace(B, hv, B * hv * (ns + 1), dev, K.tile_of(K.v2_variant(kind, G, DH)), DH)

        def step(i):
            K.cb_attn(q, pools[i % ncopy], bt, seq, out, ns, ch, ws, scale, kind, **tkw)

        # eager leg: arguments bound once (checks and pointer marshalling done once, as under graph capture)
        bound = [K.cb_attn(q, pools[j], bt, seq, out, ns, ch, ws, scale, kind, bound=True, **tkw) for j in range(ncopy)]
        t = timed(torch, step, steps, warmup, eager=lambda i: bound[i % ncopy]())
        us = t["us"]
        gbps = alg_bytes / (us * 1e-6) / 1e9
        # outside the timed region: sampled sequences of the output of one more launch against the oracle
        out.zero_()
        step(0)
        torch.cuda.synchronize()
        rows = sorted({0, min(B // 2 + 1, B - 1), B - 1})   # every index < B, also for a batch override of 1 or 2
        idx = bt[rows].long().reshape(-1)
        mp = pools[0].index_select(0, idx).cpu().numpy()
        mbt = np.arange(idx.numel(), dtype=np.int32).reshape(len(rows), -1)
        qb = q[rows].cpu().view(torch.int16).numpy().view(np.uint16)
        tb = None if ring is None else ring[rows].cpu().view(torch.int16).numpy().view(np.uint16)
        ref = A.decode_reference(qb, mp, kind, P, mbt, [Lpages] * len(rows), 1 / math.sqrt(DH), tail=tb,
                                 tail_len=None if tb is None else [T] * len(rows), kv_start=S)
        got = out[rows].view(len(rows), G * HKV, DH).float().cpu().numpy().astype(np.float64)
        st = error_stats(got, ref)
        results[plan] = {
            "workload": name, "us_per_layer_step": round(us, 2), "GBps": round(gbps, 1),
            "frac": round(gbps / PEAK_HBM_GBPS, 4), "nsplit": ns, "chunk": ch,
            "timing_used": t["timing_used"], "graph_us": round(t["graph_us"], 2), "graph_min_us": round(t["graph_min_us"], 2),
            "graph_max_us": round(t["graph_max_us"], 2), "eager_us": round(t["eager_us"], 2), "algorithmic_bytes_per_launch": alg_bytes,
            "cache_copies_cycled": ncopy, "steps": steps, "sink": S, "window": W,
            "checked": bool(st["elementwise"] <= 1.0), "bar": "elementwise <= 1", "errors": st,
            "check": f"sequences {rows} x all {G * HKV} heads vs the fp64 oracle: " + describe(st),
        }
    # the yardstick: a kernel that only READS the same pages through the same block table, with the decode kernel's
    # workgroup layout (flagrot_releaser_amd/csrc/probe_read.hip), timed the same way on the same caches
    if DH == 128:
        from flagrot_releaser_amd import probe as PR
        PR.lib()
        sink_word = torch.zeros(4, dtype=torch.int32, device=dev)
        tr = timed(torch, lambda i: PR.read_pages(pools[i % ncopy], bt, seq, sink_word, P), steps, warmup)
        rus = tr["us"]
        first = results[plans[0]]
        first["read_probe"] = {"us": round(rus, 2), "GBps": round(page_bytes / (rus * 1e-6) / 1e9, 1),
                               "frac_of_peak": round(page_bytes / (rus * 1e-6) / 1e9 / PEAK_HBM_GBPS, 4),
                               "decode_over_read": round(first["us_per_layer_step"] / rus, 3),
                               "note": "a kernel that only reads the launch's page chunks through the same block table "
                                       "(16-wavefront workgroup per (sequence, KV head), 4 pages in flight per wavefront, non-temporal loads "
                                       "as in the decode kernels)"}
    # decode-step writer (T = B new tokens) and the prefill-time writer rate, for the record
    kv_new = synth_kv(B, g, dev, torch, mu=kmu, hkv=HKV, dh=DH)
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
    first = results[plans[0]]
    first["writer"] = {"decode_step_us": round(e0.elapsed_time(e1) / 20 * 1e3, 2), "decode_step_tokens": B,
                       "prefill_fill_s": round(fill_s, 3), "prefill_tokens": B * L,
                       "note": "prefill_fill_s includes synthetic input generation"}
    # one prefill-sized call (a sequence's first n_pre tokens, consecutive slots of its pages) on resident inputs: the
    # exact selecting writer and, at head dim 128, the screened one (same bytes); into the last cache copy, after
    # everything that reads the caches
    n_pre = min(L, 8192)
    kv_pre = synth_kv(n_pre, g, dev, torch, mu=kmu, hkv=HKV, dh=DH)
    pos = torch.arange(n_pre, device=dev)
    slots_pre = (bt[0].long()[pos // P] * P + pos % P).contiguous()

    def writer_us(call, reps=10):
        for _ in range(2):
            call()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            call()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps * 1e3

    token_bytes = 2 * HKV * DH * 2 + HKV * cell                # bf16 K and V rows in, one page cell per KV head out
    legs = {"exact": lambda: K.cb_write(kv_pre, slots_pre, CT, co, kind, pools[-1], P, kmu=kmu)}
    if DH == 128:
        legs["screened"] = lambda: K.cb_write3(kv_pre, slots_pre, CT, co, None, None, kind, pools[-1], P, split=False, kmu=kmu)
    pre = {"tokens": n_pre, "kv_heads": HKV, "bytes_per_token_in_plus_out": token_bytes}
    for leg, call in legs.items():
        us_w = writer_us(call)
        pre[leg] = {"us": round(us_w, 1), "Mtokens_per_s": round(n_pre / us_w, 2),
                    "GBps_in_plus_out": round(n_pre * token_bytes / (us_w * 1e-6) / 1e9, 1)}
    first["writer"]["prefill_call"] = pre
    return results


# ------------------------------------------------------------------------------------------------ KIVI decode
def run_kivi(args, torch, dev, steps, warmup):
    """configs[3] through libflagrot_kivi.so: fill by the value writer + key group encoder, time kv_attn."""
    import numpy as np
    from flagrot_releaser_amd import kivi as KV
    from oracle import kivi as OK
    from oracle import quant as Q
    KV.lib()
    f8 = bool(args.f8)
    B, L, Gq, W, NQ, outl, gain = 16, 32768, 8, 128, 64, 8, 12.0
    HKV, DH = globals()["HKV"], globals()["DH"]
    name = ("configs[3]: KIVI-style FlagRot INT2 paged decode (per-channel keys over 32-token groups, per-token values"
            + (", FP8 meta" if f8 else "") + "), 128-token BF16 residual, Qwen-32B GQA 64q/8kv d=128, B=16 L=32768 page=16")
    if getattr(args, "head_dim", 128) == 256:       # not a configuration of the baseline: the head dim 256 kernels on the reference's test shape class
        B, L, Gq, HKV, DH = 16, 8192 + W, 6, 4, 256
        name = ("KIVI-style FlagRot INT2 paged decode at head dim 256" + (", FP8 meta" if f8 else "") +
                f", 128-token BF16 residual, GQA 24q/4kv d=256, B={B} L={L} page=16 (no baseline configuration)")
    elif getattr(args, "batch", 0) or getattr(args, "context", 0) or getattr(args, "gqa", 4) != 4:
        # shape overrides for experiments (the reference micro-benchmark sweeps B and L at 32q/8kv): not a baseline configuration
        B, L = getattr(args, "batch", 0) or B, (getattr(args, "context", 0) or L - W) + W
        Gq = int(args.gqa) if (getattr(args, "batch", 0) or getattr(args, "context", 0)) else Gq
        name = ("KIVI-style FlagRot INT2 paged decode" + (", FP8 meta" if f8 else "") + f", 128-token BF16 residual, GQA "
                f"{Gq * HKV}q/{HKV}kv d=128, B={B} L={L} page=16 [shape override: not a baseline configuration]")
    CB = KV.chunk_bytes(DH, f8)
    g = torch.Generator(device=dev).manual_seed(3)
    Lp = L - W
    npages = B * (Lp // P)
    pool = torch.zeros(npages + 16, HKV, CB, dtype=torch.uint8, device=dev)
    bt = torch.randperm(npages + 16, generator=g, device=dev)[:npages].int().view(B, -1).contiguous()
    co = torch.rand(HKV, DH, generator=g, device=dev).contiguous()
    qs = (0.3 * torch.randn(HKV, NQ, DH, generator=g, device=dev)).contiguous()
    lz = torch.full((HKV, NQ), 5.0, device=dev)
    t0 = time.perf_counter()
    for b in range(B):
        for s0 in range(0, Lp, 8192):
            n = min(8192, Lp - s0)
            kv = synth_kv(n, g, dev, torch, outliers=outl, gain=gain, hkv=HKV, dh=DH)
            pos = torch.arange(s0, s0 + n, device=dev)
            slots = bt[b].long()[pos // P] * P + pos % P
            KV.v_write(kv, slots, co, None, pool, HKV, DH, f8=f8)
            KV.k_encode(kv, torch.arange(n, device=dev).view(-1, 32), slots.view(-1, 32).contiguous(), qs, lz,
                        1 / math.sqrt(DH), pool, HKV, DH, f8=f8)
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
    ns, ch = KV.plan(B, Lp, HKV, D=DH)
    if args.nsplit:
        ns = args.nsplit
        ch = -(-Lp // ns // 32) * 32
        ns = -(-Lp // ch)
    ws = KV.Workspace(B * HKV * (ns + 1), Gq, DH, dev)
    scale = LOG2E / math.sqrt(DH)

    def step(i):
        KV.attn(q, pools[i % ncopy], bt, cached, out, ns, ch, ws, scale, 0, Gq, ring=ring, tail_len=tail_len,
                tail_idx=tail_idx, T=W, f8=f8)

    t = timed(torch, step, steps, warmup)
    us = t["us"]
    alg_bytes = B * Lp * HKV * (CB // P) + B * W * 2 * HKV * DH * 2
    gbps = alg_bytes / (us * 1e-6) / 1e9
    # check: one sequence, all heads, against fp64 attention over the oracle's dequantised pages + ring rows
    out.zero_()
    step(0)
    torch.cuda.synchronize()
    b = B - 1
    ch_np = pools[0].index_select(0, bt[b].long()).cpu().numpy()
    Kd, Vd = OK.dequant_groups(ch_np, DH, f8=f8)
    rg = Q.bf16_to_f32(ring.view(B + 1, W, 2 * HKV, DH)[b].cpu().view(torch.int16).numpy().view(np.uint16)).astype(np.float64)
    qf = Q.bf16_to_f32(q[b].cpu().view(torch.int16).numpy().view(np.uint16)).astype(np.float64)
    ref = OK.attention_reference(qf, Kd, Vd, 0, Lp, rg[:, :HKV], rg[:, HKV:], Gq, 1 / math.sqrt(DH))
    got = out[b].view(Gq * HKV, DH).float().cpu().numpy().astype(np.float64)
    st = error_stats(got, ref)
    # the prefill support path: one sequence's whole paged prefix back to bf16 K and V (kv_dequant), eager launches
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    dk = torch.empty(Lp, HKV, DH, dtype=torch.bfloat16, device=dev)
    dv = torch.empty_like(dk)
    for i in range(13):
        if i == 3:
            e0.record()
        KV.NATIVE.run("kv_dequant", pools[i % ncopy], bt[i % B], 0, Lp // 32, Lp, HKV, DH, False, dk, dv, int(f8),
                      KV.current_stream())
    e1.record()
    torch.cuda.synchronize()
    dq_us = e0.elapsed_time(e1) / 10 * 1e3
    dq_bytes = Lp * HKV * (CB // P) + 2 * Lp * HKV * DH * 2
    return {"workload": name, "us_per_layer_step": round(us, 2), "GBps": round(gbps, 1),
            "frac": round(gbps / PEAK_HBM_GBPS, 4), "nsplit": ns, "chunk": ch,
            "timing_used": t["timing_used"], "graph_us": round(t["graph_us"], 2), "graph_min_us": round(t["graph_min_us"], 2),
            "graph_max_us": round(t["graph_max_us"], 2), "eager_us": round(t["eager_us"], 2), "algorithmic_bytes_per_launch": alg_bytes,
            "cache_copies_cycled": ncopy, "steps": steps, "sink": 0, "window": W,
            "checked": bool(st["elementwise"] <= 1.0), "bar": "elementwise <= 1",
            "errors": st, "check": f"sequence {b} x all {Gq * HKV} heads vs fp64 attention over the oracle's dequantised "
                                   "pages: " + describe(st),
            "note": "one step = kv_attn = the split kernel + the merge kernel",
            "dequant": {"tokens": Lp, "us": round(dq_us, 1), "GBps": round(dq_bytes / (dq_us * 1e-6) / 1e9, 1),
                        "note": "kv_dequant of one sequence's paged prefix to bf16 K and V (page bytes read + rows "
                                "written), eager launches into preallocated outputs"},
            "writer": {"prefill_fill_s": round(fill_s, 3), "prefill_tokens": B * Lp,
                       "note": f"value writer + key group encoder ({NQ} calibration queries), includes synthetic input generation"}}


# ------------------------------------------------------------------------------------------------ MQ prefill
def run_mq(args, torch, dev, steps, warmup, fmt):
    """configs[4] through libflagrot_mq.so: one step = frmq_prep_q + frmq_attn + frmq_merge of one layer."""
    import numpy as np
    from flagrot_releaser_amd import kernels as K
    from flagrot_releaser_amd import prefill_mq as MQ
    from oracle import attend as A
    from oracle import mq as OM
    MQ.lib()
    R, NQ, PRE, Gq = 4, 512, 16384, 8
    HKV, DH = globals()["HKV"], globals()["DH"]
    k2 = fmt == "konlya"
    if getattr(args, "head_dim", 128) == 256:       # not a configuration of the baseline: the head dim 256 kernel on the reference's test shape class
        assert k2, "head dim 256: key-only pages (--mq-fmt konlya)"
        R, NQ, PRE, Gq, HKV, DH = 2, 512, 8192, 6, 4, 256
    L = PRE + NQ
    name = (f"configs[4]: multi-query prefill over INT4 FlagRot pages ({fmt}), Qwen-32B GQA 64q/8kv d=128, {R} requests x "
            f"{NQ} new tokens over a {PRE}-token cached prefix (L={L}), page=16, causal inside the chunk")
    if DH == 256:
        name = (f"multi-query prefill over INT4 FlagRot pages ({fmt}) at head dim 256, GQA {Gq * HKV}q/{HKV}kv, {R} requests x "
                f"{NQ} new tokens over a {PRE}-token cached prefix (L={L}), page=16 (no baseline configuration)")
    g = torch.Generator(device=dev).manual_seed(4)
    npg = (L + P - 1) // P
    pool = torch.zeros(R * npg + 16, HKV, 144 * P * (DH // 128), dtype=torch.uint8, device=dev)
    bt = torch.randperm(R * npg + 16, generator=g, device=dev)[:R * npg].int().view(R, npg).contiguous()
    w = 0.5 + 1.5 * torch.rand(HKV, DH, generator=g, device=dev)
    CT, co = torch.diag_embed(w).contiguous(), w.contiguous()
    kmask = (torch.rand(HKV, 4, generator=g, device=dev) < 0.5).to(torch.uint8)
    mask = torch.cat([kmask, torch.zeros_like(kmask)]).contiguous()
    for r in range(R):
        for s0 in range(0, L, 8192):
            n = min(8192, L - s0)
            kv = synth_kv(n, g, dev, torch, hkv=HKV, dh=DH)
            pos = torch.arange(s0, s0 + n, device=dev)
            slots = bt[r].long()[pos // P] * P + pos % P
            if k2:
                K.cb_write(kv, slots, CT, co, fmt, pool, P)
            else:
                K.w3_static_write(kv, slots, mask, None, pool, P, fmt=fmt)
    torch.cuda.synchronize()
    reqs = [(r, r * NQ, (r + 1) * NQ, L, PRE) for r in range(R)]
    plan = MQ.build_plan(reqs, Gq, HKV, 0, dev, D=DH)
    q = (2.0 * torch.randn(R * NQ, Gq * HKV, DH, generator=g, device=dev)).bfloat16()
    out = torch.zeros(R * NQ, Gq * HKV * DH, dtype=torch.bfloat16, device=dev)
    scale = LOG2E / math.sqrt(DH)
    keep = {}

    def step(i):
        q16 = MQ.prep_q(q, scale, Gq, plan.idx, None, None if k2 else kmask)
        opart, ml = MQ.attn(q16, pool, bt, plan, Gq, 0, k2, False)
        MQ.merge(plan, opart, ml, Gq, out=out)
        keep["q16"] = q16

    t = timed(torch, step, steps, warmup)
    us = t["us"]
    pairs = R * Gq * HKV * sum(PRE + t_ + 1 for t_ in range(NQ))
    flops = 4.0 * DH * pairs
    tflops = flops / (us * 1e-6) / 1e12
    # check: the first and the last 4 rows of request R - 1, two KV heads (16 q heads), against fp64 attention over
    # the oracle's dequantised pages (static format: keys in the stored basis, q16 was rotated to match)
    out.zero_()
    step(0)
    torch.cuda.synchronize()
    r, nh = R - 1, 2
    mp = pool.index_select(0, bt[r].long())[:, :nh].contiguous().cpu().numpy()
    Kp, Vp = A.dequant_pages(mp, fmt, P, Dh=DH)
    Kd, Vd = Kp.reshape(-1, nh, DH)[:L], Vp.reshape(-1, nh, DH)[:L]
    q16 = keep["q16"].view(R * NQ, Gq * HKV, DH)
    gots, refs = [], []
    for t0_ in (0, NQ - 4):
        rows = slice(r * NQ + t0_, r * NQ + t0_ + 4)
        qb = q16[rows, :nh * Gq].cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
        ref, _ = OM.attention(qb, {0: Kd}, {0: Vd}, [(0, 0, 4, L, PRE + t0_)], Gq, 0)
        got = out[rows].view(4, Gq * HKV, DH)[:, :nh * Gq].float().cpu().numpy().astype(np.float64)
        gots.append(got)
        refs.append(ref)
    st = error_stats(np.stack(gots), np.stack(refs))
    # where the element-wise yardstick |err| <= 2e-3 + 1e-2 |ref| is exceeded (the bar of this kernel is the relative L2)
    ga, ra = np.stack(gots), np.stack(refs)
    ratio = np.abs(ga - ra) / (ATOL + RTOL * np.abs(ra))
    over = ratio > 1.0
    worst = np.unravel_index(np.argmax(ratio), ratio.shape)
    st["over_elementwise_bar"] = {
        "fraction": float(over.mean()), "count": int(over.sum()), "of": int(over.size),
        "median_abs_ref_of_those": float(np.median(np.abs(ra[over]))) if over.any() else None,
        "median_abs_err_of_those": float(np.median(np.abs(ga - ra)[over])) if over.any() else None,
        "rms_ref_all": float(np.sqrt((ra ** 2).mean())), "rms_err_all": float(np.sqrt(((ga - ra) ** 2).mean())),
        "worst": {"ref": float(ra[worst]), "got": float(ga[worst]), "row_max_abs_ref": float(np.abs(ra[worst[:3]]).max())}}
    probe = mfma_probe(torch, dev)
    return {"workload": name, "ms_per_layer": round(us * 1e-3, 4), "TFLOPs": round(tflops, 1),
            "mfma_probe": {**probe, "kernel_over_lds_probe": round(tflops / max(probe["lds_operand_TFLOPs"], 1e-9), 4)},
            "frac": round(tflops / PEAK_F16_TFLOPS, 4), "bound": "mfma", "peak_TFLOPs": PEAK_F16_TFLOPS,
            "timing_used": t["timing_used"], "graph_us": round(t["graph_us"], 1), "graph_min_us": round(t["graph_min_us"], 1),
            "graph_max_us": round(t["graph_max_us"], 1), "eager_us": round(t["eager_us"], 1), "algorithmic_flops_per_launch": flops, "steps": steps,
            "tiles": plan.ntiles, "items": plan.nitems, "rows_per_tile": plan.rows,
            "checked": bool(st["rel_l2"] <= 3e-3), "bar": "rel_l2 <= 3e-3 (BF16 FlashAttention's error, the reference's yardstick)",
            "errors": st, "check": f"request {r}, rows 0-3 and {NQ - 4}-{NQ - 1}, {nh * Gq} q heads vs fp64 attention over "
                                   "the oracle's dequantised pages: " + describe(st),
            "note": "one step = frmq_prep_q + frmq_attn + frmq_merge; the attention kernel dominates"}


def mfma_probe(torch, dev, iters=4000):
    """the matrix pipe's reachable dense-fp16 rate on this box: a kernel of nothing but v_mfma_f32_32x32x16_f16 (one
    workgroup of 8 wavefronts per CU), operands in registers / one operand of every instruction read from LDS"""
    from flagrot_releaser_amd import probe as PR
    PR.lib()
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    out = {}
    for mode, key in ((0, "registers_TFLOPs"), (1, "lds_operand_TFLOPs")):
        PR.mfma_burst(mode, iters // 8, cus, sink)
        torch.cuda.synchronize()
        best = 0.0
        for _ in range(3):
            e0.record()
            flops = PR.mfma_burst(mode, iters, cus, sink)
            e1.record()
            torch.cuda.synchronize()
            best = max(best, flops / (e0.elapsed_time(e1) * 1e-3) / 1e12)
        out[key] = round(best, 1)
    out["nominal_TFLOPs"] = PEAK_F16_TFLOPS
    out["note"] = (f"{cus} workgroups x 8 wavefronts x {iters} x 4 v_mfma_f32_32x32x16_f16, best of 3 launches "
                   "(flagrot_releaser_amd/csrc/probe_mfma.hip)")
    return out


def plain_shape(args):
    """the committed traffic figures belong to the workloads at their own shapes (and to GQA 8 on the int4 pages)"""
    return (getattr(args, "head_dim", 128) == 128 and getattr(args, "gqa", 4) in (4, 8) and not getattr(args, "batch", 0)
            and not getattr(args, "context", 0) and getattr(args, "window", -1) < 0 and not getattr(args, "f8", False))


def traffic_of(workload):
    try:   # measured with rocprofv3 --pmc in separate runs (FETCH_SIZE / WRITE_SIZE); a process cannot count its own
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            return json.load(f).get(workload, {}).get("traffic_bytes")
    except OSError:
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=None, choices=["int4", "int2", "int2_b32", "kivi", "mq"])
    ap.add_argument("--mq-fmt", default="konlya", choices=["konlya", "int4a"])
    ap.add_argument("--f8", action="store_true", help="kivi: FP8-meta pages")
    ap.add_argument("--head-dim", type=int, default=128, choices=[128, 256], help="256 = the head dim 256 kernels (GQA 24q/4kv, the reference's test shape class); not a baseline configuration")
    ap.add_argument("--batch", type=int, default=0, help="int4 / int2 / kivi workloads: another batch size (not a baseline configuration)")
    ap.add_argument("--context", type=int, default=0, help="int4 / int2 / kivi workloads: another context length (kivi: cached tokens besides the 128 BF16 rows; not a baseline configuration)")
    ap.add_argument("--window", type=int, default=-1, help="int4 / int2 workloads: BF16 window tokens (0: no BF16 rows and no sinks; not a baseline configuration)")
    ap.add_argument("--gqa", type=int, default=4, help="int4 / int2 workloads: query heads per KV head (8 = tiles of 8 heads; not a baseline configuration)")
    ap.add_argument("--nsplit", type=int, default=0, help="override the planner's split count")
    ap.add_argument("--chunk", type=int, default=0, help="int4 / int2 workloads: tokens per split, overriding the planner (experiments)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", action="store_true", help="the chosen workload only (no extra legs)")
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
    workload = args.workload or "int4"
    extras = args.workload is None and not args.only
    metric = "paged decode attention: achieved HBM GB/s of page bytes per layer-step (us per layer-step alongside)"
    common = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
              "vs_baseline": None, "data": "synthetic"}
    timing = (f"the {args.steps} steps between two events on the launch stream, submitted (a) as one HIP graph and (b) as eager "
              f"launches with bound arguments, {REPLAYS} times each: the smaller of the two medians (timing_used says which)")
    if workload == "mq":
        r = run_mq(args, torch, dev, args.steps, args.warmup, args.mq_fmt)
        res = {"metric": "multi-query prefill attention over INT4 pages: achieved TFLOP/s per layer (ms per layer alongside)",
               "value": r["TFLOPs"], "unit": "TFLOP/s", **common, "ms_per_step": r["ms_per_layer"],
               "dtype": "f16 operands, f32 accumulate",
               "config": {"workload": r["workload"], "tiles": r["tiles"], "items": r["items"],
                          "rows_per_tile": r["rows_per_tile"], "timing": timing},
               "roofline": {"bound": "mfma", "achieved": r["TFLOPs"], "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                            "frac": r["frac"], "traffic": None,
                            "algorithmic_flops_per_launch": r["algorithmic_flops_per_launch"],
                            "avg_launch_us": r["ms_per_layer"] * 1e3, "timing_used": r["timing_used"], "graph_us": r["graph_us"],
                            "eager_us": r["eager_us"]},
               "mfma_probe": r["mfma_probe"],
               "checked": r["checked"], "bar": r["bar"], "errors": r["errors"], "check": r["check"]}
    else:
        if workload == "kivi":
            r = run_kivi(args, torch, dev, args.steps, args.warmup)
            dtype = "u8 codes, f16 products, f32 accumulate"
        else:
            plans = ("own", "reference") if (extras and workload == "int4") else ("own",)
            rr = run_flagrot(args, torch, dev, workload, args.steps, args.warmup, plans)
            r = rr["own"]
            dtype = "u8 codes, f16 products, f32 accumulate"
        res = {"metric": metric, "value": r["GBps"], "unit": "GB/s", **common,
               "ms_per_step": round(r["us_per_layer_step"] * 1e-3, 6), "us_per_layer_step": r["us_per_layer_step"],
               "dtype": dtype,
               "config": {"workload": r["workload"], "nsplit": r["nsplit"], "chunk": r["chunk"],
                          "cache_copies_cycled": r["cache_copies_cycled"], "timing": timing, "sink": r["sink"],
                          "window": r["window"]},
               "roofline": {"bound": "hbm", "achieved": r["GBps"], "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": r["frac"],
                            "traffic": traffic_of(workload + ("_gqa8" if getattr(args, "gqa", 4) == 8 else "")) if plain_shape(args) else None,
                            "traffic_source": TRAFFIC_FILE + " (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of this launch in "
                                              "separate runs, scaled by a device copy; not measured in this run)",
                            "algorithmic_bytes_per_launch": r["algorithmic_bytes_per_launch"],
                            "avg_launch_us": r["us_per_layer_step"], "timing_used": r["timing_used"], "graph_us": r["graph_us"],
                            "graph_min_us": r["graph_min_us"], "graph_max_us": r["graph_max_us"], "eager_us": r["eager_us"]},
               "checked": r["checked"], "bar": r["bar"], "errors": r["errors"], "check": r["check"]}
        for extra in ("writer", "dequant", "read_probe"):
            if extra in r:
                res[extra] = r[extra]
        if workload == "int4" and extras:
            ref = rr["reference"]
            res["reference_planner"] = {k: ref[k] for k in ("nsplit", "chunk", "us_per_layer_step", "frac", "graph_us", "eager_us", "checked")}
            res["reference_planner"]["note"] = ("the split plan the reference front end's own cost model makes from "
                                                "fr_cb_occupancy x multi_processor_count, run through the same library")
    if extras:
        short = max(10, args.steps // 5)
        wl = {}
        torch.cuda.empty_cache()
        wl["int2"] = run_flagrot(args, torch, dev, "int2", short, 5)["own"]
        torch.cuda.empty_cache()
        wl["int2_b32_l8192"] = run_flagrot(args, torch, dev, "int2_b32", short, 5)["own"]
        torch.cuda.empty_cache()
        wl["kivi"] = run_kivi(args, torch, dev, short, 5)
        torch.cuda.empty_cache()
        wl["mq_" + args.mq_fmt] = run_mq(args, torch, dev, max(5, args.steps // 20), 3, args.mq_fmt)
        torch.cuda.empty_cache()
        res["workloads"] = wl
        res["checked_all"] = bool(res["checked"] and all(v["checked"] for v in wl.values()))
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline(torch, K, dev)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
