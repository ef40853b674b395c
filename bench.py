#!/usr/bin/env python3
"""Benchmark of the MI355X attention hot path (one GPU).

Primary line (the metric BASELINE.json names): split-KV decode attention, Llama-3.1-8B head
shape (32 query heads, 8 KV heads, head_dim 128), F16 KV cache, KV length 32768, batch 16
independent sequences -- 2 GiB of KV per step, far beyond the 256 MB Infinity Cache, so the
rate is an HBM rate.  A "step" is one attention call over the whole batch with Q/K/V already
resident in HBM.  `value` is algorithmic bytes / wall time of the timed region.

`roofline` is computed from the dominant kernel's own duration (HIP events recorded by the
library on the launch stream around the split-KV kernel of every timed step).
`cpu_baseline` times the restated reference CPU backend (AVX2+FMA+F16C, one task per Q head) on
a bounded sample (one of the 16 sequences) on the host cores of the same box.
`extras` reports the other benchmark configurations with the same accounting.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "argus-engine_amd"), os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0       # MI355X published HBM3E bandwidth
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense f16 MFMA


def decode_bytes(hq, hkv, d, L, batch, kv_elem_bytes=2, scores=False):
    """Algorithmic bytes of one decode call: K+V over the valid length, Q in, out (+ scores)."""
    per_seq = 2 * hkv * L * d * kv_elem_bytes + hq * d * 4 * 2
    if scores:
        per_seq += hq * L * 4
    return per_seq * batch


SPIN_UP_SECONDS = 0.3


def spin_up(fn):
    """Untimed: repeat the step until the GPU has left its idle clocks.  A fresh process starts at a
    low engine clock and takes ~0.1 s of load to ramp; a handful of sub-millisecond warm-up launches
    does not get there (measured: the same prefill kernel 718 us after 5 launches, 615 us after 300)."""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < SPIN_UP_SECONDS:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()


def time_region(fn, steps, warmup):
    import torch
    spin_up(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


_EVENT_GAP_MS = None


def event_gap_ms():
    """What an empty interval between two event records reads on this box (about 4.5 us): the library's
    per-kernel brackets include it."""
    global _EVENT_GAP_MS
    if _EVENT_GAP_MS is None:
        import torch
        gaps = []
        for _ in range(20):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            e1.record()
            torch.cuda.synchronize()
            gaps.append(e0.elapsed_time(e1))
        gaps.sort()
        _EVENT_GAP_MS = gaps[len(gaps) // 2]
    return _EVENT_GAP_MS


def measure(ctx, step, steps, warmup):
    """(wall seconds per step, dominant-kernel ms, tail ms).  The wall clock is taken over a pass that
    records no events; the kernel durations come from a second pass in which the library brackets the
    dominant kernel and the rest of the call (the combine pass) with HIP events on the launch stream.
    Such a bracket also measures the events themselves, which matters below ~50 us: there the device
    time of a call is taken from one event pair around all `steps` calls issued back to back, and the
    brackets (less the reading of an empty one) only say how that time divides between the dominant
    kernel and the tail (never more than that device time in total)."""
    import torch
    spin_up(step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    ctx.kernel_timing_begin(steps)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    kms, tail = ctx.kernel_timing_end2(steps)
    n = max(len(kms), 1)
    k_ms, t_ms = sum(kms) / n, sum(tail) / n
    if k_ms < 0.05:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        dev_ms = min(e0.elapsed_time(e1) / steps, wall * 1e3)
        gap = event_gap_ms()
        k, t = max(k_ms - gap, 1e-6), max(t_ms - gap, 0.0)
        if t < 0.0005:  # nothing was launched behind the dominant kernel
            t = 0.0
        scale = min(1.0, dev_ms / (k + t))  # (calls issued slower than they run leave the device idle in between)
        k_ms, t_ms = k * scale, t * scale
    elif k_ms + t_ms > wall * 1e3:  # the brackets' own cost, on a call the device never idles in
        scale = wall * 1e3 / (k_ms + t_ms)
        k_ms, t_ms = k_ms * scale, t_ms * scale
    return wall, k_ms, t_ms


def result(wall, kernel_ms, tail_ms, nbytes, **more):
    r = dict(ms_per_step=wall * 1e3, kernel_ms=kernel_ms, combine_ms=tail_ms, bytes=nbytes, gbps_wall=nbytes / wall / 1e9,
             gbps_kernel=nbytes / (kernel_ms * 1e-3) / 1e9 if kernel_ms else None,
             gbps_kernels=nbytes / ((kernel_ms + tail_ms) * 1e-3) / 1e9 if kernel_ms else None)
    r.update(more)
    return r


def bench_decode(ctx, hq, hkv, d, L, batch, steps, warmup, capacity=None, scores=False, softcap=0.0,
                 rotate=1, seed=137, stats=False):
    """Returns dict(ms_per_step, kernel_ms, bytes).  `rotate` distinct KV buffers are cycled so a
    cache smaller than the rotation set cannot serve repeated reads.  stats: scores in the logits +
    (max, sum) form that the device-side reduce consumes (no rewrite of the rows as probabilities)."""
    import torch
    cap = capacity or L
    g = torch.Generator(device="cuda").manual_seed(seed)
    ks, vs = [], []
    for _ in range(rotate):
        ks.append(torch.randn((batch, hkv, cap, d), generator=g, device="cuda", dtype=torch.float32).half())
        vs.append(torch.randn((batch, hkv, cap, d), generator=g, device="cuda", dtype=torch.float32).half())
    q = torch.randn((batch, hq, d), generator=g, device="cuda", dtype=torch.float32)
    out = torch.empty((batch, hq, d), device="cuda", dtype=torch.float32)
    scs = [torch.empty((batch, hq, cap), device="cuda", dtype=torch.float32) for _ in range(rotate)] if scores else None
    st = torch.empty((batch, hq, 2), device="cuda", dtype=torch.float32) if (scores and stats) else None
    state = {"i": 0}

    def step():
        i = state["i"] % rotate
        state["i"] += 1
        ctx.attention_gen(q, ks[i], vs[i], out, hkv, L, cap, scores=scs[i] if scores else None,
                          score_stride=cap if scores else 0, batch=batch, kv_batch_stride=hkv * cap * d, softcap=softcap,
                          score_stats=st)

    wall, kernel_ms, tail_ms = measure(ctx, step, steps, warmup)
    r = result(wall, kernel_ms, tail_ms, decode_bytes(hq, hkv, d, L, batch, 2, scores))
    r["plan"] = ctx.last_decode_plan()
    return r


def bench_decode_blocks(ctx, fmt, hq, hkv, d, L, batch, steps, warmup, rotate=1, scores=False, stats=False):
    """Decode attention over a block-quantised cache (q4_0 / q4_1 / q8_0 / q2_0 rows of 18- / 20- / 34- / 12-byte blocks):
    synthetic blocks (random codes, f16 scales sized for N(0,1)-like values); algorithmic bytes are
    the attended block rows of K and V plus Q and out."""
    import torch
    import argus_hip as A
    bb = {"q4_0": 18, "q4_1": 20, "q8_0": 34, "q2_0": 12}[fmt]
    kv_dtype = {"q4_0": A.Q4_0, "q4_1": A.Q4_1, "q8_0": A.Q8_0, "q2_0": A.Q2_0}[fmt]
    row_bytes = d // 32 * bb
    g = torch.Generator(device="cuda").manual_seed(11)

    def blocks():
        raw = torch.randint(0, 256, (batch * hkv * L * d // 32, bb), generator=g, device="cuda", dtype=torch.uint8)
        lo, hi = {"q4_0": (0.1, 0.3), "q4_1": (0.1, 0.3), "q8_0": (0.005, 0.02), "q2_0": (0.8, 1.6)}[fmt]
        scale = (torch.rand(raw.shape[0], generator=g, device="cuda") * (hi - lo) + lo).half()
        raw[:, 0:2] = scale.view(torch.uint8).reshape(-1, 2)
        if fmt in ("q2_0", "q4_1"):  # [f16 d][f16 m]: minimum at half the code range below zero
            raw[:, 2:4] = (scale.float() * (-1.5 if fmt == "q2_0" else -7.5)).half().view(torch.uint8).reshape(-1, 2)
        return raw.reshape(-1)

    ks = [blocks() for _ in range(rotate)]
    vs = [blocks() for _ in range(rotate)]
    q = torch.randn((batch, hq, d), generator=g, device="cuda", dtype=torch.float32)
    out = torch.empty((batch, hq, d), device="cuda", dtype=torch.float32)
    sc = torch.empty((batch, hq, L), device="cuda", dtype=torch.float32) if scores else None
    st = torch.empty((batch, hq, 2), device="cuda", dtype=torch.float32) if (scores and stats) else None
    state = {"i": 0}

    def step():
        i = state["i"] % rotate
        state["i"] += 1
        ctx.attention_gen(q, ks[i], vs[i], out, hkv, L, L, batch=batch, kv_batch_stride=hkv * L * d, kv_dtype=kv_dtype,
                          scores=sc, score_stride=L if scores else 0, score_stats=st)

    wall, kernel_ms, tail_ms = measure(ctx, step, steps, warmup)
    nbytes = batch * (2 * hkv * L * row_bytes + 2 * hq * d * 4 + (hq * L * 4 if scores else 0))
    return result(wall, kernel_ms, tail_ms, nbytes,
                  f16_equivalent_gbps_kernel=decode_bytes(hq, hkv, d, L, batch, 2, False) / (kernel_ms * 1e-3) / 1e9)


def bench_kivi(ctx, bits, steps, warmup, hq=32, hkv=8, d=128, n_tokens=8192, res_cap=128, res_f16=False,
               rotate=8, batch=1):
    """Benchmark configuration 4: q_tokens = 8064 quantised + 128 residual tokens.  Blocks are synthetic
    (random codes, f16 scale/min headers); `rotate` block sets are cycled.  batch > 1 runs that many
    caches (e.g. the layers of a model) in one launch so the rate is not launch-latency bound."""
    import torch
    q_tokens = (n_tokens - 1) // res_cap * res_cap
    res_tokens = n_tokens - q_tokens
    bb = 4 + 32 * bits // 8
    nblk1 = q_tokens * hkv * d // 32
    nblk = nblk1 * batch
    g = torch.Generator(device="cuda").manual_seed(4)

    def blocks():
        raw = torch.randint(0, 256, (nblk, bb), generator=g, device="cuda", dtype=torch.uint8)
        hdr = torch.empty((nblk, 2), device="cuda", dtype=torch.float16)
        hdr[:, 0] = 6.0 / (2 ** bits - 1)
        hdr[:, 1] = -3.0
        raw[:, :4] = hdr.view(torch.uint8)
        return raw.reshape(-1)

    sets = [(blocks(), blocks()) for _ in range(rotate)]
    rdt = torch.float16 if res_f16 else torch.float32
    res_k = torch.randn((batch, hkv, res_cap, d), generator=g, device="cuda").to(rdt)
    res_v = torch.randn((batch, hkv, res_cap, d), generator=g, device="cuda").to(rdt)
    q = torch.randn((batch, hq, d), generator=g, device="cuda")
    out = torch.empty((batch, hq, d), device="cuda")
    state = {"i": 0}

    def step():
        qk, qv = sets[state["i"] % rotate]
        state["i"] += 1
        ctx.attention_gen_quant(q, qk, qv, res_k, res_v, out, hkv, q_tokens, res_tokens, res_cap,
                                1.0 / d ** 0.5, bits, batch=batch, block_batch_stride_bytes=nblk1 * bb,
                                res_batch_stride=hkv * res_cap * d)

    wall, kernel_ms, tail_ms = measure(ctx, step, steps, warmup)
    nbytes = 2 * nblk * bb + batch * (2 * hkv * res_tokens * d * (2 if res_f16 else 4) + hq * d * 4 * 2)
    return result(wall, kernel_ms, tail_ms, nbytes)


def bench_prefill(ctx, steps, warmup, hq=32, hkv=8, d=64, s=2048, batch=1, f16_io=True):
    """Benchmark configuration 2: causal GQA prefill; FLOPs use the causal count 4*Hq*d*S(S+1)/2."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(42)
    io = torch.float16 if f16_io else torch.float32
    q = torch.randn((batch, s, hq, d), generator=g, device="cuda").to(io)
    k = torch.randn((batch, hkv, s, d), generator=g, device="cuda").half()
    v = torch.randn((batch, hkv, s, d), generator=g, device="cuda").half()
    out = torch.empty((batch, s, hq, d), device="cuda", dtype=io)

    def step():
        rc = ctx.flash_attention_prefill(q, k, v, out, hq, hkv, s, s, d, s, batch_size=batch)
        assert rc == 1

    wall, kernel_ms, _ = measure(ctx, step, steps, warmup)
    flops = 4 * hq * d * s * (s + 1) // 2 * batch
    return dict(us_per_call=round(wall * 1e6, 2), kernel_us=round(kernel_ms * 1e3, 2), causal_flops=flops,
                tflops_kernel=round(flops / (kernel_ms * 1e-3) / 1e12, 1),
                mfma_frac_kernel=round(flops / (kernel_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                tflops_wall=round(flops / wall / 1e12, 1))


def bench_aux(ctx, steps, warmup):
    """The data-movement kernels either side of the attention calls, each at a size of the benchmark
    configurations: microseconds per call (torch events on the current stream, `steps` calls back to
    back) and the rate on the bytes the call has to move."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(3)
    res = {}

    def timed(name, fn, nbytes, note):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / steps
        res[name] = {"us_per_call": round(us, 2), "bytes": nbytes, "gbps": round(nbytes / us / 1e3, 1),
                     "hbm_frac": round(nbytes / us / 1e3 / 8000.0, 4), "note": note}

    # (a-4) H2O score reduce: 32 layers x 32 heads of probabilities over 32768 positions
    nl, hq, hkv, L = 32, 32, 8, 32768
    # three score buffers of 137 MB are cycled: 411 MB, beyond the 256 MB Infinity Cache, so the rate is an HBM rate
    bufs = [torch.rand((nl, hq, L), generator=g, device="cuda") for _ in range(3)]
    imp = torch.zeros(L, device="cuda")
    himp = torch.zeros(hkv * L, device="cuda")
    lf = torch.zeros(nl * L, device="cuda")
    turn = {"i": 0}

    def next_scores():
        turn["i"] += 1
        return bufs[turn["i"] % len(bufs)]

    spin_up(lambda: ctx.score_reduce(next_scores(), imp, himp, 0.9, nl, hq, hkv, L, L, L))
    timed("score_reduce_L32768_32x32", lambda: ctx.score_reduce(next_scores(), imp, himp, 0.9, nl, hq, hkv, L, L, L),
          bufs[0].numel() * 4 + 2 * (imp.numel() + himp.numel()) * 4,
          "fused importance + per-KV-head importance; 3 score buffers cycled (411 MB)")
    timed("score_reduce_per_layer_L32768_32x32", lambda: ctx.score_reduce_per_layer(next_scores(), lf, 0.9, nl, hq, hkv, L, L, L),
          bufs[0].numel() * 4 + 2 * lf.numel() * 4, "per-layer importance; 3 score buffers cycled (411 MB)")
    stats = torch.rand((nl, hq, 2), generator=g, device="cuda") + 1.0
    timed("score_reduce_L32768_32x32_from_logits", lambda: ctx.score_reduce(next_scores(), imp, himp, 0.9, nl, hq, hkv, L, L, L, stats=stats),
          bufs[0].numel() * 4 + 2 * (imp.numel() + himp.numel()) * 4,
          "the same reduce over logits + (max, sum): exp(s - max) / sum applied while reading")
    del bufs

    # (f-1) KV scatter of a 2048-token prefill chunk, F32 rows -> F16 HeadMajor cache
    hkv, d, cap, sl = 8, 128, 32768, 2048
    ks = torch.randn((sl, hkv, d), generator=g, device="cuda")
    vs = torch.randn((sl, hkv, d), generator=g, device="cuda")
    kd = torch.zeros((hkv, cap, d), device="cuda", dtype=torch.float16)
    vd = torch.zeros_like(kd)
    timed("kv_scatter_f32_to_f16_2048_tokens", lambda: ctx.kv_scatter(ks, vs, kd, vd, hkv, d, cap, 100, seq_len=sl),
          2 * sl * hkv * d * (4 + 2), "K and V rows of one layer")
    k1, v1 = ks[:1].contiguous(), vs[:1].contiguous()
    timed("kv_scatter_f32_to_f16_1_token", lambda: ctx.kv_scatter(k1, v1, kd, vd, hkv, d, cap, 100),
          2 * hkv * d * 6, "decode step: launch latency")

    # (f-4) descriptor codec over one layer's cache of 32768 tokens (8 KV heads x 128)
    import argus_hip as O  # the named descriptors
    n = 32768 * hkv * d
    x = torch.randn(n, generator=g, device="cuda")
    for name, desc, bb in (("q4_0", O.DESC_Q4_0, 18), ("q2_0", O.DESC_Q2_0, 12)):
        blocks = torch.zeros(n // 32 * bb, dtype=torch.uint8, device="cuda")
        f16 = torch.zeros(n, dtype=torch.float16, device="cuda")
        timed("kv_encode_descriptor_%s_32768_tokens" % name, lambda: ctx.kv_encode_descriptor(desc, x, blocks, n),
              n * 4 + blocks.numel(), "F32 rows -> blocks")
        timed("kv_decode_descriptor_%s_to_f16_32768_tokens" % name, lambda: ctx.kv_decode_descriptor(desc, blocks, f16, n),
              blocks.numel() + n * 2, "blocks -> F16 rows (the floor's decode pass)")

    # (f-2) KIVI flush of a full 128-token residual, and the F16 view of one flush (config-4 shape)
    R, hkv, d = 128, 8, 128
    for bits in (2, 4, 8):
        bb = 4 + 32 * bits // 8
        res_k = torch.randn((hkv, R, d), generator=g, device="cuda")
        res_v = torch.randn((hkv, R, d), generator=g, device="cuda")
        nblk = hkv * R * d // 32
        qk = torch.zeros(nblk * bb, dtype=torch.uint8, device="cuda")
        qv = torch.zeros(nblk * bb, dtype=torch.uint8, device="cuda")
        timed("kivi_flush_q%d_128_tokens" % bits, lambda: ctx.quant_flush(res_k, res_v, qk, qv, hkv, R, d, R, 0, 0, bits),
              2 * hkv * R * d * 4 + 2 * nblk * bb, "quantise K and V residuals (launch latency: 1 MB)")
        view = torch.zeros((R + 2, hkv, d), device="cuda", dtype=torch.float16)
        timed("kivi_dequant_flush_q%d_key_128_tokens" % bits,
              lambda: ctx.quant_dequant_flush(qk, view, hkv, d, R // 32, 0, 0, bits, True),
              nblk * bb + hkv * R * d * 2, "blocks -> F16 view rows")
    # (a-6) PFA side channel: probabilities of the trailing 32 query rows of a 2048-token prefill chunk
    # over a 8192-token prefix, 32 heads, F16 HeadMajor K
    nq, nkv, d, sl, prefix, qwin = 32, 8, 128, 2048, 8192, 32
    q = torch.randn((sl, nq, d), generator=g, device="cuda")
    k = torch.randn((nkv, prefix, d), generator=g, device="cuda").half()
    sum_out = torch.zeros((nq, prefix), device="cuda")
    per_row = torch.zeros((qwin, prefix), device="cuda")
    timed("pfa_scores_window32_prefix8192", lambda: ctx.prefill_attention_scores(
        q, k, nq, nkv, d, sl, prefix, d, prefix * d, prefix - sl, qwin, sum_out=sum_out, per_row=per_row),
        nkv * prefix * d * 2 + (nq * prefix + qwin * prefix) * 4 * 2,
        "K read once + the two score buffers updated; %d MMAC" % (nq * qwin * prefix * d // 1000000))
    return res


def cpu_baseline_decode(hq, hkv, d, L, budget_s=12.0):
    """Restated CpuBackendAVX2::attention_gen on one sequence of the primary workload."""
    import numpy as np
    import oracle
    rng = np.random.default_rng(137)
    q = rng.standard_normal((hq, d), dtype=np.float32)
    k = rng.standard_normal((hkv, L, d), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((hkv, L, d), dtype=np.float32).astype(np.float16)
    cores = min(hq, int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1), 16)
    oracle.attention_gen(q, k, v, hkv, L, L, impl="avx2", n_threads=cores)  # warm-up
    times = []
    t_start = time.perf_counter()
    while len(times) < 20 or (time.perf_counter() - t_start < budget_s and len(times) < 8000):
        t0 = time.perf_counter()
        oracle.attention_gen(q, k, v, hkv, L, L, impl="avx2", n_threads=cores)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_start > 2.5 * budget_s:
            break
    times.sort()
    med = times[len(times) // 2]
    nbytes = decode_bytes(hq, hkv, d, L, 1)
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("model name"):
                    model = ln.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "cpu_model": model, "nproc": os.cpu_count(),
            "sample": "1 of the 16 sequences (Hq32 Hkv8 d128 L32768 F16 KV), median of %d calls, %.1f us/call; "
                      "restated CpuBackendAVX2::attention_gen, one task per Q head" % (len(times), med * 1e6)}


# HBM bytes per launch of the primary workload's kernel, from rocprofv3 FETCH_SIZE + WRITE_SIZE runs
# scaled by what the same counters read for a plain 1 GiB copy (x2.000 and x1.000).  Counters cannot
# be read from inside this process, so the figure is the one of the profile run named beside it in
# the output (`traffic_source`), not a measurement of this run.
DECODE_TRAFFIC_BYTES = 2_161_394_139
DECODE_TRAFFIC_SOURCE = "profiles/decode_mfma_cfg3_L32768_b16_hbm_traffic.md"


def bench_layer_loop(ctx, steps, warmup, hq=32, hkv=8, d=128, L=4096, layers=32):
    """What a decode step of a model issues: one attention call per layer, back to back on one
    stream, each layer with its own KV cache (32 x 16.8 MB = 537 MB, beyond the Infinity Cache).
    Eager: the calls are issued from this process (its per-call cost is part of the figure).
    Graph: the same 32 calls of the entry point that allocates nothing, captured once into a HIP
    graph and replayed -- kernels only on the stream.  Returns microseconds per token (32 layers)."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(9)
    ks = [torch.randn((hkv, L, d), generator=g, device="cuda").half() for _ in range(layers)]
    vs = [torch.randn((hkv, L, d), generator=g, device="cuda").half() for _ in range(layers)]
    q = torch.randn((layers, hq, d), generator=g, device="cuda")
    out = torch.empty((layers, hq, d), device="cuda")

    def token(noalloc=False):
        for i in range(layers):
            ctx.attention_gen(q[i], ks[i], vs[i], out[i], hkv, L, L, noalloc=noalloc)

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps

    spin_up(token)
    res = {"layers": layers, "kv_len": L, "eager_us_per_token": round(timed(token), 2)}
    eager = out.clone()
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            token(noalloc=True)  # kernels loaded, launch facts cached before the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        out.zero_()
        with torch.cuda.graph(graph, stream=side):
            token(noalloc=True)
        ok = True
        for _ in range(3):  # every replay is checked against the eager result, with eager work in between
            out.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            ok = ok and bool(torch.equal(out, eager))
        res["graph_replays_match_eager"] = ok
        res["graph_us_per_token"] = round(timed(graph.replay), 2)
    except Exception as e:  # capture is optional: report why it is missing
        res["graph_error"] = str(e)[:200]
    nbytes = layers * decode_bytes(hq, hkv, d, L, 1)
    res["bytes_per_token"] = nbytes
    for k in ("eager", "graph"):
        if k + "_us_per_token" in res:
            res[k + "_gbps"] = round(nbytes / res[k + "_us_per_token"] / 1e3, 1)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extras", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--workload", default="primary",
                    choices=["primary", "decode_b1", "prefill", "prefill_d128", "kivi_q4", "kivi_q8", "cfg5", "q4_0", "q4_0_b1", "primary_scores_stats",
                             "q8_0", "q4_0_d64", "copy_calib", "aux", "layers", "primary_scores", "cfg5_b64", "prefill_d64_16k"],
                    help="run one secondary workload alone (for profiling) instead of the primary line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (every box has one GPU; the path shards by "
              "sequence / KV head without exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import argus_hip
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    ctx = argus_hip.Context(0)
    info = ctx.device_info()

    if args.workload != "primary":
        w = args.workload
        if w == "copy_calib":
            # plain 1 GiB device copy: the known-size reference the HBM traffic counters are scaled by
            src = torch.ones(1 << 28, device="cuda")
            dst = torch.empty_like(src)
            for _ in range(args.warmup + args.steps):
                dst.copy_(src)
            torch.cuda.synchronize()
            res = {"bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4}
        elif w == "aux":
            res = bench_aux(ctx, args.steps, args.warmup)
        elif w == "layers":
            res = bench_layer_loop(ctx, args.steps, args.warmup)
        elif w == "primary_scores":
            res = bench_decode(ctx, 32, 8, 128, 32768, 16, args.steps, args.warmup, scores=True)
        elif w == "primary_scores_stats":
            res = bench_decode(ctx, 32, 8, 128, 32768, 16, args.steps, args.warmup, scores=True, stats=True)
        elif w == "cfg5_b64":
            res = bench_decode(ctx, 8, 4, 256, 2048, 64, args.steps, args.warmup, capacity=4096, scores=True, softcap=50.0)
        elif w == "decode_b1":
            res = bench_decode(ctx, 32, 8, 128, 32768, 1, args.steps, args.warmup, rotate=4)
        elif w == "prefill":
            res = bench_prefill(ctx, args.steps, args.warmup)
        elif w == "prefill_d128":
            res = bench_prefill(ctx, args.steps, args.warmup, hq=32, hkv=8, d=128, s=8192)
        elif w == "prefill_d64_16k":
            res = bench_prefill(ctx, args.steps, args.warmup, hq=32, hkv=8, d=64, s=16384)
        elif w in ("q4_0", "q8_0"):
            res = bench_decode_blocks(ctx, w, 32, 8, 128, 32768, 16, args.steps, args.warmup)
        elif w == "q4_0_d64":
            res = bench_decode_blocks(ctx, "q4_0", 14, 2, 64, 32768, 64, args.steps, args.warmup)
        elif w == "q4_0_b1":
            res = bench_decode_blocks(ctx, "q4_0", 32, 8, 128, 32768, 1, args.steps, args.warmup, rotate=8)
        elif w == "cfg5":
            res = bench_decode(ctx, 8, 4, 256, 2048, 8, args.steps, args.warmup, capacity=4096, scores=True,
                               softcap=50.0, rotate=8, stats=True)
        else:
            res = bench_kivi(ctx, 4 if w == "kivi_q4" else 8, args.steps, args.warmup, batch=32, rotate=2)
        print(json.dumps({"workload": w, "steps": args.steps, "warmup": args.warmup, "result": res}))
        return

    hq, hkv, d, L, batch = 32, 8, 128, 32768, 16
    r = bench_decode(ctx, hq, hkv, d, L, batch, args.steps, args.warmup)
    line = {
        "metric": "decode_attn_hbm_gbps_32k_kv",
        "value": round(r["gbps_wall"], 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(r["ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 3: split-KV decode attention, Llama-3.1-8B shape "
                               "(Hq32 Hkv8 d128), F16 KV, KV length 32768, batch 16, seeded N(0,1)",
                   "kv_dtype": "f16", "accumulate": "f32",
                   "mfma_operands": "f16 (K and V as stored; Q as f16 hi + lo pair, probabilities rounded to f16); "
                                    "logits, softmax, sums and outputs f32",
                   "batch": batch, "kv_len": L,
                   "us_per_call": round(r["ms_per_step"] * 1e3, 2),
                   "tokens_per_s": round(batch / (r["ms_per_step"] * 1e-3), 1)},
        "roofline": {"bound": "hbm", "achieved": round(r["gbps_kernel"], 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(r["gbps_kernel"] / HBM_PEAK_GBPS, 4), "traffic": DECODE_TRAFFIC_BYTES,
                     "traffic_source": DECODE_TRAFFIC_SOURCE,
                     "kernel": "decode_mfma_kernel<128,2>", "kernel_ms": round(r["kernel_ms"], 5),
                     "combine_ms": round(r["combine_ms"], 5),
                     "frac_with_combine": round(r["gbps_kernels"] / HBM_PEAK_GBPS, 4),
                     "algorithmic_bytes": r["bytes"], "plan": r["plan"]},
        "device": {"name": info.name.decode(), "arch": info.gcn_arch.decode(), "cus": info.compute_units,
                   "clock_mhz": info.clock_mhz},
    }

    if not args.no_extras:
        ex = {}
        es, ew = max(20, args.steps), max(3, args.warmup)

        def add(name, res, note=""):
            ex[name] = {"us_per_call": round(res["ms_per_step"] * 1e3, 2),
                        "kernel_us": round(res["kernel_ms"] * 1e3, 2),
                        "combine_us": round(res["combine_ms"] * 1e3, 2),
                        "gbps_kernel": round(res["gbps_kernel"], 1),
                        "hbm_frac_kernel": round(res["gbps_kernel"] / HBM_PEAK_GBPS, 4),
                        "hbm_frac_with_combine": round(res["gbps_kernels"] / HBM_PEAK_GBPS, 4),
                        "bytes": res["bytes"], "note": note}

        add("cfg3_L32768_b1", bench_decode(ctx, 32, 8, 128, 32768, 1, es, ew, rotate=4),
            "4 KV buffer sets rotated (512 MiB > Infinity Cache)")
        add("cfg3_L4096_b16", bench_decode(ctx, 32, 8, 128, 4096, 16, es, ew, rotate=2), "2 sets rotated")
        add("cfg3_L4096_b1", bench_decode(ctx, 32, 8, 128, 4096, 1, es, ew, rotate=16), "16 sets rotated")
        add("cfg3_L32768_b16_scores", bench_decode(ctx, 32, 8, 128, 32768, 16, es, ew, scores=True, stats=True),
            "scores emitted as logits + (max, sum) per row, the form the device-side H2O reduce reads (67 MB per call)")
        add("cfg3_L32768_b16_scores_as_probabilities", bench_decode(ctx, 32, 8, 128, 32768, 16, es, ew, scores=True),
            "the trait's form: combine_us is the pass that rewrites the 67 MB of logits as probabilities")
        add("cfg3_L256_b1", bench_decode(ctx, 32, 8, 128, 256, 1, es, ew, rotate=16),
            "short context: one workgroup per KV head, one launch (no combine pass)")
        add("cfg3_L256_b16", bench_decode(ctx, 32, 8, 128, 256, 16, es, ew, rotate=8), "short context, 16 sequences: one launch")
        add("cfg1_qwen_L1024_b1", bench_decode(ctx, 14, 2, 64, 1024, 1, es, ew), "latency-bound (0.5 MiB)")
        add("cfg5_gemma2_L2048_cap4096_b8_scores_softcap50",
            bench_decode(ctx, 8, 4, 256, 2048, 8, es, ew, capacity=4096, scores=True, softcap=50.0, rotate=8, stats=True),
            "scores emitted as logits + (max, sum); 8 KV and score buffer sets rotated (537 MB of attended rows)")
        add("cfg5_gemma2_L2048_cap4096_b8_scores_as_probabilities",
            bench_decode(ctx, 8, 4, 256, 2048, 8, es, ew, capacity=4096, scores=True, softcap=50.0, rotate=8),
            "the trait's form (rows rewritten as probabilities by the combine pass)")
        add("cfg5_gemma2_L2048_cap4096_b64_scores_softcap50",
            bench_decode(ctx, 8, 4, 256, 2048, 64, es, ew, capacity=4096, scores=True, softcap=50.0, stats=True),
            "the same shape with 64 sequences per call (542 MB): the kernel's rate once the call is not latency-bound")
        add("cfg4_kivi_q4_L8192_res128_f32", bench_kivi(ctx, 4, es, ew), "8 block sets rotated; single launch, 11.4 MB")
        add("cfg4_kivi_q8_L8192_res128_f32", bench_kivi(ctx, 8, es, ew), "8 block sets rotated; single launch, 19.7 MB")
        add("cfg4_kivi_q4_L8192_res128_f16", bench_kivi(ctx, 4, es, ew, res_f16=True), "F16 residual window")
        add("cfg4_kivi_q4_x32_caches", bench_kivi(ctx, 4, es, ew, batch=32, rotate=2),
            "32 caches (sequences) per launch, 365 MB: amortised rate")
        add("cfg4_kivi_q8_x32_caches", bench_kivi(ctx, 8, es, ew, batch=32, rotate=2),
            "32 caches (sequences) per launch, 629 MB: amortised rate")
        add("kivi_q4_d64_Hq32_Hkv8_x32_caches", bench_kivi(ctx, 4, es, ew, hq=32, hkv=8, d=64, batch=32, rotate=2),
            "head_dim 64 (Llama-3.2-1B head shape), 32 caches per launch, 183 MB")
        add("cfg3_q4_0_blocks_L32768_b16", bench_decode_blocks(ctx, "q4_0", 32, 8, 128, 32768, 16, es, ew),
            "--kv-format q4_0 rows attended in-kernel, 604 MB of blocks")
        add("cfg3_q4_0_blocks_L32768_b16_scores", bench_decode_blocks(ctx, "q4_0", 32, 8, 128, 32768, 16, es, ew, scores=True, stats=True),
            "q4_0 rows with scores emitted as logits + (max, sum) per row (67 MB per call)")
        add("cfg3_q4_0_blocks_L32768_b16_scores_as_probabilities", bench_decode_blocks(ctx, "q4_0", 32, 8, 128, 32768, 16, es, ew, scores=True),
            "the trait's form: combine_us is the pass that rewrites the 67 MB of logits as probabilities")
        add("cfg3_q8_0_blocks_L32768_b16", bench_decode_blocks(ctx, "q8_0", 32, 8, 128, 32768, 16, es, ew),
            "--kv-format q8_0 rows attended in-kernel, 1141 MB of blocks")
        add("cfg3_q2_0_blocks_L32768_b16", bench_decode_blocks(ctx, "q2_0", 32, 8, 128, 32768, 16, es, ew),
            "--kv-format q2_0 rows attended in-kernel, 403 MB of blocks")
        add("qwen_d64_q4_0_blocks_L32768_b64", bench_decode_blocks(ctx, "q4_0", 14, 2, 64, 32768, 64, es, ew),
            "head_dim 64 (Hq14 Hkv2), 302 MB of q4_0 blocks")
        add("gemma_d256_q4_0_blocks_L32768_b8", bench_decode_blocks(ctx, "q4_0", 16, 8, 256, 32768, 8, es, ew),
            "head_dim 256 (Hq16 Hkv8), 604 MB of q4_0 blocks")
        ex["cfg2_prefill_llama1b_S2048_f16"] = bench_prefill(ctx, es, ew)
        ex["cfg2_prefill_llama1b_S2048_f16_batch4"] = bench_prefill(ctx, es, ew, batch=4)
        ex["cfg2_prefill_llama1b_S2048_f16_batch8"] = bench_prefill(ctx, es, ew, batch=8)
        ex["cfg2_prefill_llama1b_S2048_f32io"] = bench_prefill(ctx, es, ew, f16_io=False)
        ex["prefill_llama8b_d128_S8192_f16"] = bench_prefill(ctx, max(5, es // 4), 2, hq=32, hkv=8, d=128, s=8192)
        ex["prefill_d64_by_seq_len"] = {str(sl): bench_prefill(ctx, max(5, es // 4), 2, s=sl)["mfma_frac_kernel"]
                                        for sl in (1024, 2048, 4096, 8192, 16384)}
        ex["decode_32_layers_cfg3_L4096_b1"] = bench_layer_loop(ctx, max(5, es // 4), 2)
        ex["aux_kernels"] = bench_aux(ctx, es, ew)
        line["extras"] = ex

    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_decode(hq, hkv, d, L)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
