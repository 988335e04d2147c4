#!/usr/bin/env python3
"""Benchmark of the KV-cache decode hot path on one MI355X.

Workload (the configuration the metric is quoted on): a Llama-3-8B-shaped GQA decode
layer in f16 — 32 query heads, 8 KV heads, head_dim 128 — with the KV cache prefilled to
8192 tokens, then single-token steps.  One step = append one K token and one V token to
the in-place caches + decode attention of one query token per sequence over the whole
cache (causal).  Batch 8 is the headline line; batches 1 and 32 are reported beside it.
The steps visit LAYERS such layers' caches round-robin (4 x 268 MB at batch 8), as the layers of
a decoder do: a launch then never finds its cache in the 256 MB Infinity Cache left there by the
previous launch, and the figures are HBM figures.  (`cache_resident_*` repeats the kernel
timing on a single layer's cache, which the Infinity Cache partly serves: 5-9 points higher.)

Prints ONE JSON line.  `value` = algorithmic HBM bytes of a step / wall time of a step
(inputs resident in HBM), `roofline` = the decode-attention kernel alone, timed with HIP
events on the stream it runs on, `cpu_baseline` = the CPU restatement of tract's default
runtime (concat cache + flash SDPA) on this box's host cores, on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HQ, HKV, D, CTX = 32, 8, 128, 8192
LAYERS = 4
PREWARM_LAUNCHES = 1000   # untimed attention launches before the warm-up steps (clock ramp), see run_batch
HBM_PEAK_GBS = 8000.0
# HBM traffic of one decode-attention launch at the default arguments (batch 8, context 8226 in the
# kernel loop), from two `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE), each
# counter scaled by what it reads for the 128 MiB prefill copy of known size: FETCH_SIZE
# 134135.5 x 1.9991 KiB + WRITE_SIZE 650 x 0.9993 KiB.
PMC_TRAFFIC_BYTES_B8_CTX8226 = int((134135.5 * 1.9991 + 650.0 * 0.9993) * 1024)
PMC_ALGORITHMIC_BYTES_B8_CTX8226 = 2 * 8 * 8 * 8226 * 128 * 2 + 2 * 8 * 32 * 128 * 2


def cfg_seed(cfg, what):
    return 20260000 + 100 * cfg + {"q": 0, "k": 1, "v": 2}[what]


def algorithmic_bytes(B, T, e_kv=2, e_q=2):
    """K and V read once per KV head + Q read and O write + the appended K/V token."""
    return 2 * B * HKV * T * D * e_kv + 2 * B * HQ * D * e_q + 2 * B * HKV * D * e_kv


def seeded_f16(seed, shape):
    g = np.random.Generator(np.random.PCG64(seed))
    return g.standard_normal(shape, dtype=np.float32).astype(np.float16)


def run_batch(ta, B, steps, warmup, kernel_iters, layers=LAYERS, windows=5):
    """Returns a dict of measurements for batch size B."""
    sts = [ta.InPlaceKvSdpa(axis=2, causal=True, scale=None).state() for _ in range(layers)]
    # prefill: one append of 8192 seeded tokens per sequence (the same values in every layer)
    kp = np.empty((B, HKV, CTX, D), dtype=np.float16)
    vp = np.empty((B, HKV, CTX, D), dtype=np.float16)
    for b in range(B):
        kp[b] = seeded_f16(cfg_seed(2, "k") + 1000 * b, (HKV, CTX, D))
        vp[b] = seeded_f16(cfg_seed(2, "v") + 1000 * b, (HKV, CTX, D))
    for st in sts:
        st.k.push(kp)
        st.v.push(vp)
    del kp, vp
    n = warmup + windows * steps
    scale_q = np.float32(1.0 / np.sqrt(D))
    q_all = (seeded_f16(cfg_seed(2, "q"), (n, B, HQ, 1, D)).astype(np.float32) * scale_q).astype(np.float16)
    k_all = seeded_f16(cfg_seed(2, "k") + 7, (n, B, HKV, 1, D))
    v_all = seeded_f16(cfg_seed(2, "v") + 7, (n, B, HKV, 1, D))
    dq = [ta.DeviceTensor.from_numpy(q_all[i]) for i in range(n)]
    dk = [ta.DeviceTensor.from_numpy(k_all[i]) for i in range(n)]
    dv = [ta.DeviceTensor.from_numpy(v_all[i]) for i in range(n)]
    out = ta.DeviceTensor((B, HQ, 1, D), np.float16)

    def step(i):
        sts[i % layers].eval_into(dq[i], dk[i], dv[i], out)

    # Bring the device to its steady clocks first: the first ~100 launches after the idle set-up phase run
    # about 5 % slower than the same launches later.  These launches read the caches and change no state.
    for j in range(PREWARM_LAUNCHES):
        sts[j % layers].attend(dq[0], out=out)
    # A layer's first step doubles its capacity 8192 -> 16384 (one reallocation: the valid region of K and V moves to
    # new planes).  Those `layers` steps are the first of the warm-up and are timed on their own, so that the line can
    # say what the doubling costs a 128-step generation; the timed windows below hold no growth.
    g0, g1 = ta.Event(), ta.Event()
    n_growth = min(layers, warmup)
    ta.synchronize()
    g0.record()
    for i in range(n_growth):
        step(i)
    g1.record()
    for i in range(n_growth, warmup):
        step(i)
    growth_step_us = ta.Event.elapsed_ms(g0, g1) / max(1, n_growth) * 1e3
    # The timed region is `steps` steps between two device synchronisations, taken `windows` times on
    # fresh inputs (every step appends, so the caches keep growing).  Each window is timed twice over:
    # by the host's clock around the synchronisations, and by two HIP events recorded on the stream just
    # before the first and just after the last step.  The event time is the device's time for the steps;
    # the host's clock adds one launch latency and one synchronisation latency (together 40-80 us), which
    # a short window (20 steps are 1 ms at batch 8) does not amortise and a decoder that keeps its stream
    # fed never pays.  The median window by event time gives `value`; the host's clock is reported beside it.
    wins = []
    e0, e1 = ta.Event(), ta.Event()
    for w in range(windows):
        first = warmup + w * steps
        ta.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for i in range(first, first + steps):
            step(i)
        e1.record()
        ta.synchronize()
        wall = time.perf_counter() - t0
        ev = ta.Event.elapsed_ms(e0, e1) * 1e-3
        # context length seen by timed step i: the layer's prefill plus its earlier visits plus this token
        ctx_sum = sum(CTX + i // layers + 1 for i in range(first, first + steps))
        wins.append({"event_s": ev, "wall_s": wall, "bytes": algorithmic_bytes(B, ctx_sum / steps)})
    wins.sort(key=lambda x: x["event_s"])
    med = wins[len(wins) // 2]
    dt = med["event_s"]
    wall_med = sorted(x["wall_s"] for x in wins)[len(wins) // 2]
    res = {
        "batch": B,
        "ms_per_step": dt / steps * 1e3,
        "us_per_token": dt / steps * 1e6,
        "step_gbs": med["bytes"] / (dt / steps) / 1e9,
        "wall_ms_per_step": wall_med / steps * 1e3,
        "wall_step_gbs": med["bytes"] / (wall_med / steps) / 1e9,
        "windows": windows,
        "window_ms_per_step_min_max": [round(wins[0]["event_s"] / steps * 1e3, 5), round(wins[-1]["event_s"] / steps * 1e3, 5)],
        "reallocs": sts[0].k.reallocs(),
        "context_end": sts[0].k.len(),
        "prewarm_launches": PREWARM_LAUNCHES,
    }

    # The attention launch without the fused append (`attend`), for reference: HIP events around windows of launches on
    # the stream.  A step IS one launch of the same kernel (the append rides along), so the step windows above are
    # what the roofline figure rests on; this loop only shows that the append costs nothing measurable.
    def kernel_time(states, n_windows=5):
        e0, e1 = ta.Event(), ta.Event()
        for j in range(max(3, len(states))):
            states[j % len(states)].attend(dq[0], out=out)
        ta.synchronize()
        per = max(20, kernel_iters // n_windows)
        secs = []
        for _ in range(n_windows):
            e0.record()
            for j in range(per):
                states[j % len(states)].attend(dq[0], out=out)
            e1.record()
            secs.append(ta.Event.elapsed_ms(e0, e1) / per * 1e-3)
        secs.sort()
        return secs[len(secs) // 2], secs[0], secs[-1]

    T_now = sum(st.k.len() for st in sts) / layers
    kbytes = 2 * B * HKV * T_now * D * 2 + 2 * B * HQ * D * 2  # K+V once per KV head, Q read, O write
    sec, sec_min, sec_max = kernel_time(sts)
    res["kernel_us"] = sec * 1e6
    res["kernel_us_min_max"] = [round(sec_min * 1e6, 3), round(sec_max * 1e6, 3)]
    res["kernel_bytes"] = int(kbytes)
    res["kernel_gbs"] = kbytes / sec / 1e9
    sec1, _, _ = kernel_time(sts[:1])
    res["cache_resident_kernel_us"] = sec1 * 1e6
    res["cache_resident_kernel_gbs"] = (2 * B * HKV * sts[0].k.len() * D * 2 + 2 * B * HQ * D * 2) / sec1 / 1e9
    res["step_bytes"] = int(med["bytes"])
    res["growth_step_us"] = growth_step_us
    # one doubling per layer and generation, spread over cfg2's 128 steps
    res["growth_us_per_token_over_128_steps"] = max(0.0, growth_step_us - dt / steps * 1e6) / 128.0
    # the last launch was layer 0's cache with query 0: kept for the parity spot check
    res["last_out"] = out.to_numpy()
    res["last_q"] = q_all[0]
    res["state"] = sts[0]
    return res


def cpu_baseline(B, budget_s=20.0):
    """The reference's default CPU path (concat cache growth + FlashSdpaOp::eval with its
    whole-tensor casts), restated in C (oracle/), threaded over (batch, q head) like rayon's
    global pool, on this host's cores; bounded sample of the same workload."""
    from oracle import oracle as orc
    orc.build()
    threads = min(orc.max_threads(), os.cpu_count() or 1)
    k = np.empty((B, HKV, CTX, D), dtype=np.float16)
    v = np.empty((B, HKV, CTX, D), dtype=np.float16)
    for b in range(B):
        k[b] = seeded_f16(cfg_seed(2, "k") + 1000 * b, (HKV, CTX, D))
        v[b] = seeded_f16(cfg_seed(2, "v") + 1000 * b, (HKV, CTX, D))
    q = (seeded_f16(cfg_seed(2, "q"), (B, HQ, 1, D)).astype(np.float32) / np.sqrt(D)).astype(np.float16)
    kn = seeded_f16(cfg_seed(2, "k") + 7, (B, HKV, 1, D))
    vn = seeded_f16(cfg_seed(2, "v") + 7, (B, HKV, 1, D))
    times = []
    t_start = time.perf_counter()
    steps = 0
    while steps < 2 or (time.perf_counter() - t_start < budget_s and steps < 16):
        t0 = time.perf_counter()
        _, k, v = orc.decode_step_f16(q, k, v, kn, vn, threads=threads)
        times.append(time.perf_counter() - t0)
        steps += 1
    med = float(np.median(times[1:])) if len(times) > 1 else times[0]
    T = CTX + steps / 2.0
    return {
        "value": algorithmic_bytes(B, T) / med / 1e9,
        "unit": "GB/s",
        "us_per_token": med * 1e6,
        "cores": threads,
        "kind": "port",
        "sample": f"{steps} decode steps (1 warm-up + median of the rest) at batch {B}, context {CTX}+, "
                  "C restatement of tract's CPU path (concat cache reallocation + flash SDPA with whole-tensor "
                  "f32 casts), not the tract binary",
    }


def time_calls(ta, fn, iters):
    """Average microseconds of fn() over `iters` back-to-back calls (HIP events on the stream), after
    at least 3 calls and about 10 ms of untimed calls (the device's clocks settle)."""
    t0 = time.perf_counter()
    calls = 0
    while calls < 3 or (time.perf_counter() - t0 < 0.010 and calls < 2000):
        fn()
        calls += 1
        if calls % 16 == 0:
            ta.synchronize()
    ta.synchronize()
    e0, e1 = ta.Event(), ta.Event()
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    return ta.Event.elapsed_ms(e0, e1) / iters * 1e3


def parity_sample(out, q, k, v, heads, seqs=None, k_dequant=None):
    """Max-abs difference between the GPU's `out` and the oracle's flash SDPA on a sample: query heads `heads` of
    batch entries `seqs` (default: the first).  Runs after the timed region; the oracle is the checker only."""
    from oracle import oracle as orc
    g = q.shape[1] // k.shape[1]
    worst = 0.0
    for b in (seqs if seqs is not None else [0]):
        for h in heads:
            kh = h // g
            want = orc.flash_sdpa(q[b:b + 1, h:h + 1], np.ascontiguousarray(k[b:b + 1, kh:kh + 1]),
                                  np.ascontiguousarray(v[b:b + 1, kh:kh + 1]), causal=True, threads=8)
            worst = max(worst, float(np.abs(want.astype(np.float32) - out[b:b + 1, h:h + 1].astype(np.float32)).max()))
    return worst


def base_line(args, workload, value, unit, ms_per_step, dtype, roofline, extra):
    line = {
        "metric": "decode-attn over KV cache: achieved HBM GB/s (% of peak) + us/token at 8k ctx",
        "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic", "config": {"workload": workload}, "roofline": roofline,
    }
    line.update(extra)
    return line


def run_cfg1(ta, args):
    """cfg1, the reference's own CPU-runnable case: batch 1, 32 = 32 heads, d = 64, f32, the cache grows
    from empty to 256 tokens one decode step at a time (capacities 1, 2, 4 ... 256: 8 reallocations)."""
    from oracle import oracle as orc
    H, Dh, n = 32, 64, 256
    g = np.random.Generator(np.random.PCG64(cfg_seed(1, "q")))
    q_all = g.standard_normal((n, 1, H, 1, Dh), dtype=np.float32)
    k_all = np.random.Generator(np.random.PCG64(cfg_seed(1, "k"))).standard_normal((n, 1, H, 1, Dh), dtype=np.float32)
    v_all = np.random.Generator(np.random.PCG64(cfg_seed(1, "v"))).standard_normal((n, 1, H, 1, Dh), dtype=np.float32)
    dq = [ta.DeviceTensor.from_numpy(q_all[i]) for i in range(n)]
    dk = [ta.DeviceTensor.from_numpy(k_all[i]) for i in range(n)]
    dv = [ta.DeviceTensor.from_numpy(v_all[i]) for i in range(n)]
    out = ta.DeviceTensor((1, H, 1, Dh), np.float32)
    best, st = None, None
    for rep in range(3):   # the whole 256-step generation, three times; the fastest is reported
        st = ta.InPlaceKvSdpa(axis=2, causal=True).state()
        ta.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            st.eval_into(dq[i], dk[i], dv[i], out)
        ta.synchronize()
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    got = out.to_numpy()
    want = orc.flash_sdpa(q_all[-1], np.concatenate(list(k_all), axis=2), np.concatenate(list(v_all), axis=2), causal=True)
    err = float(np.abs(got - want).max())
    assert err <= 1e-3, err
    assert st.k.valid_contiguous().tobytes() == np.concatenate(list(k_all), axis=2).tobytes()
    by = sum(2 * H * (t + 1) * Dh * 4 + 2 * H * Dh * 4 + 2 * H * Dh * 4 for t in range(n))
    us = best / n * 1e6
    t0 = time.perf_counter()
    kc = vc = None
    for i in range(n):   # the reference's CPU path on the same steps: concat cache + flash SDPA
        kc, vc = orc.concat_append(kc, k_all[i], 2), orc.concat_append(vc, v_all[i], 2)
        orc.flash_sdpa(q_all[i], kc, vc, causal=True)
    cpu_us = (time.perf_counter() - t0) / n * 1e6
    gbs = by / best / 1e9
    roof = {"bound": "hbm", "kernel": "sdpa_decode_kernel<f32,64,1>", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 5), "traffic": None}
    line = base_line(args, "cfg1: batch 1, 32 heads, d=64, f32, 256 decode steps from an empty cache (a correctness "
                     "configuration: at most 4 MB per step, the step is launch latency)", round(gbs, 2), "GB/s",
                     round(us / 1e3, 5), "f32", roof,
                     {"us_per_token": round(us, 2), "reallocs": st.k.reallocs(), "capacity_end": st.k.capacity(),
                      "parity_max_abs_vs_oracle": err, "cache_bit_exact": True})
    line["steps"], line["warmup"] = n, 0
    line["cpu_baseline"] = {"value": round(by / n / cpu_us / 1e3, 3), "unit": "GB/s", "us_per_token": round(cpu_us, 1), "cores": 1,
                            "kind": "port", "sample": "the same 256 steps with the C restatement (concat cache growth + flash SDPA), one thread"}
    return line


def run_cfg3(ta, args):
    """Chunked prefill: 8 chunks of 512 tokens appended to an empty cache, each followed by causal
    attention of the chunk over the cache so far.  MFMA-bound; value = causal-effective TFLOP/s."""
    S, C = 512, 8
    st = ta.InPlaceKvSdpa(axis=2, causal=True).state()
    per_chunk, tot_us, tot_fl = [], 0.0, 0.0
    ks, vs, err = [], [], 0.0
    for c in range(1, C + 1):
        k = seeded_f16(cfg_seed(3, "k") + c, (1, HKV, S, D))
        v = seeded_f16(cfg_seed(3, "v") + c, (1, HKV, S, D))
        st.k.push(k), st.v.push(v)
        ks.append(k), vs.append(v)
        qh = (seeded_f16(cfg_seed(3, "q") + c, (1, HQ, S, D)).astype(np.float32) / np.sqrt(D)).astype(np.float16)
        q = ta.DeviceTensor.from_numpy(qh)
        out = ta.DeviceTensor((1, HQ, S, D), np.float16)
        us = time_calls(ta, lambda: st.attend(q, out=out), 20)
        if c in (1, 4, C):   # after the timing: the chunk's output against the oracle on three query heads (checker only)
            err = max(err, parity_sample(out.to_numpy(), qh, np.concatenate(ks, axis=2), np.concatenate(vs, axis=2), [0, 13, 31]))
        pairs = S * (S * c) - S * (S - 1) // 2
        fl = 4.0 * HQ * D * pairs
        per_chunk.append({"kv_len": S * c, "us": round(us, 2), "tflops": round(fl / us / 1e6, 1)})
        tot_us += us
        tot_fl += fl
    tf = tot_fl / tot_us / 1e6
    roof = {"bound": "mfma", "kernel": "sdpa_prefill_pp_kernel<128,4,false,F16> (key splits merged in the kernel)", "achieved": round(tf, 1), "peak": 2500.0,
            "unit": "TFLOP/s", "frac": round(tf / 2500.0, 4), "traffic": None}
    return base_line(args, "cfg3: chunked prefill, 8 x 512 tokens into an empty cache, causal SDPA of each chunk over "
                     "the cache so far (32q/8kv d=128 f16, batch 1); attention launches only", round(tf, 1), "TFLOP/s",
                     round(tot_us / C / 1e3, 5), "f16", roof,
                     {"chunks": per_chunk, "total_us": round(tot_us, 1), "parity_max_abs_vs_oracle": err,
                      "parity_sample": "chunks 1, 4 and 8, query heads 0, 13 and 31, all 512 queries, against the oracle"})


def run_cfg4(ta, args):
    """Block-quantised KV cache, batch 8, contexts 4096 and 16384, decode with fused dequant."""
    res = {}
    # (the last two: 64 query heads over the 8 kv heads, the group size of the larger decoders)
    for name, fmt, ek, T, hq in [(n, f, e, T, HQ) for n, f, e in (("q8_0", ta.Q8_0, 34 / 32), ("q4_0", ta.Q4_0, 18 / 32), ("f16", None, 2.0))
                                 for T in (4096, 16384)] + [("q8_0", ta.Q8_0, 34 / 32, 16384, 64), ("q4_0", ta.Q4_0, 18 / 32, 16384, 64)]:
        if True:
            B = 8
            layers = 4 if T <= 4096 or fmt is not None else 2   # > 256 MB in total: no Infinity Cache reuse between launches
            sts = [ta.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state() for _ in range(layers)]
            rng = np.random.default_rng(cfg_seed(4, "k"))
            chan = rng.choice(HKV * D, size=10, replace=False)
            k = seeded_f16(cfg_seed(4, "k") + T, (B, HKV, T, D)).astype(np.float32)
            kf = k.transpose(0, 2, 1, 3).reshape(B, T, HKV * D)
            kf[:, :, chan] *= 20.0
            k = kf.reshape(B, T, HKV, D).transpose(0, 2, 1, 3).astype(np.float16)
            v = seeded_f16(cfg_seed(4, "v") + T, (B, HKV, T, D))   # (not K again: swapped planes or scales would show)
            for st in sts:
                for c, x in ((st.k, k), (st.v, v)):
                    c.reserve(T + 1024, like=(x.shape, x.dtype))
                    c.push(x)
            qh = (seeded_f16(cfg_seed(4, "q"), (B, hq, 1, D)).astype(np.float32) / np.sqrt(D)).astype(np.float16)
            q = ta.DeviceTensor.from_numpy(qh)
            out = ta.DeviceTensor((B, hq, 1, D), np.float16)
            turn = [0]

            def one():
                sts[turn[0] % layers].attend(q, out=out)
                turn[0] += 1

            us = time_calls(ta, one, 100)
            # after the timing: sequences 0 and 7, four query heads, against the oracle over the dequantised blocks
            from oracle import oracle as orc
            sts[0].attend(q, out=out)
            kd, vd = k[[0, 7]], v[[0, 7]]
            if fmt is not None:
                ofmt = getattr(orc, "FMT_" + name.upper())
                kd = orc.dequant(ofmt, orc.quant(ofmt, kd), np.float16)
                vd = orc.dequant(ofmt, orc.quant(ofmt, vd), np.float16)
            o = out.to_numpy()[[0, 7]]
            err = parity_sample(o, qh[[0, 7]], kd, vd, [0, 9, 18, 31], seqs=[0, 1])
            # the whole decode step of a layer (the new token's K and V quantised into the cache, then attention); the
            # caches have room for these appends, so none of them grows
            tk = ta.DeviceTensor.from_numpy(seeded_f16(cfg_seed(4, "k") + 7, (B, HKV, 1, D)))
            tv = ta.DeviceTensor.from_numpy(seeded_f16(cfg_seed(4, "v") + 7, (B, HKV, 1, D)))

            def step():
                sts[turn[0] % layers].eval_into(q, tk, tv, out=out)
                turn[0] += 1

            step_us = time_calls(ta, step, 64)
            del sts
            by = 2 * B * HKV * T * D * ek + 2 * B * hq * D * 2
            res[f"{name}_ctx{T}" + ("" if hq == HQ else f"_{hq}q")] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": int(by), "parity_max_abs_vs_oracle": err,
                                     "step_us": round(step_us, 2)}
    head = res["q8_0_ctx16384"]
    roof = {"bound": "hbm", "kernel": "sdpa_decode_mfma_kernel<128,8,Q8_0,false,true,412>", "achieved": head["gbs"], "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(head["gbs"] / HBM_PEAK_GBS, 4), "traffic": None}
    return base_line(args, "cfg4: decode over a Q8_0 / Q4_0 quantised KV cache (fused dequant), batch 8, contexts 4096 "
                     "and 16384, 1% outlier channels x20; attention launches only, rotating over 2-4 layers' caches; "
                     "headline = Q8_0 at 16384; the _64q cases have 64 query heads over the 8 kv heads",
                     head["gbs"], "GB/s", round(head["us"] / 1e3, 5), "q8_0/f16", roof,
                     {"cases": res, "parity_max_abs_vs_oracle": max(c["parity_max_abs_vs_oracle"] for c in res.values()),
                      "parity_sample": "every case: sequences 0 and 7, query heads 0, 9, 18, 31, against the oracle's attention over the dequantised blocks"})


def run_cfg5(ta, args):
    """Ragged multi-sequence decode: 64 sequences with their own capacity-doubling caches carved
    from one pool, lengths uniform in [512, 32768]; a step appends one token to every sequence
    and attends within each sequence's own length (one fused call)."""
    n_seq = 64
    rng = np.random.default_rng(cfg_seed(5, "q") + 3)
    lens = rng.integers(512, 32768, size=n_seq, endpoint=True)
    pool = ta.KvPool(int(lens.sum()) * HKV * D * 2 * 2 * 3 + (64 << 20))
    kcs, vcs = [], []
    for i, n in enumerate(lens):
        k = seeded_f16(cfg_seed(5, "k") + i, (1, HKV, int(n), D))
        kc, vc = ta.InPlaceKvCache(2, pool=pool), ta.InPlaceKvCache(2, pool=pool)
        kc.push(k), vc.push(k)
        kcs.append(kc), vcs.append(vc)
    ws = ta.Workspace(n_seq, HQ, 1, D)
    n = args.steps + args.warmup
    steps = min(args.steps, 64)
    n = steps + args.warmup
    qs = [ta.DeviceTensor.from_numpy((seeded_f16(cfg_seed(5, "q") + i, (n_seq, HQ, 1, D)).astype(np.float32) / np.sqrt(D)).astype(np.float16)) for i in range(n)]
    kn = [ta.DeviceTensor.from_numpy(seeded_f16(cfg_seed(5, "k") + 1000 + i, (n_seq, HKV, 1, D))) for i in range(n)]
    out = ta.DeviceTensor((n_seq, HQ, 1, D), np.float16)
    for i in range(args.warmup):
        ta.inplace_kv_sdpa_eval_ragged(qs[i], kn[i], kn[i], kcs, vcs, workspace=ws, out=out)
    ta.synchronize()
    t0 = time.perf_counter()
    for i in range(args.warmup, n):
        ta.inplace_kv_sdpa_eval_ragged(qs[i], kn[i], kn[i], kcs, vcs, workspace=ws, out=out)
    ta.synchronize()
    dt = (time.perf_counter() - t0) / steps
    tot = int(sum(c.len() for c in kcs))
    by = 2 * HKV * D * 2 * tot + 2 * n_seq * HQ * D * 2 + 2 * n_seq * HKV * D * 2
    us_k = time_calls(ta, lambda: ta.sdpa_decode_ragged(qs[0], kcs, vcs, workspace=ws, out=out), 20)
    # after the timing: the last launch's output for the shortest, the longest and two other sequences against the
    # oracle over those sequences' caches as they now are (read back from the device)
    o, q0 = out.to_numpy(), qs[0].to_numpy()
    sample = sorted({int(np.argmin(lens)), int(np.argmax(lens)), 7, 40})
    err = max(parity_sample(o[i:i + 1], q0[i:i + 1], kcs[i].valid_contiguous(), vcs[i].valid_contiguous(), [0, 13, 31]) for i in sample)
    roof = {"bound": "hbm", "kernel": "sdpa_decode_mfma_ragged_kernel<128,8,F16,true>", "achieved": round(by / us_k / 1e3, 1),
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(by / us_k / 1e3 / HBM_PEAK_GBS, 4), "traffic": None,
            "kernel_us": round(us_k, 2), "algorithmic_bytes_per_launch": int(by)}
    st = pool.stats()
    return base_line(args, f"cfg5: ragged decode, 64 sequences (lengths 512..32768, sum {tot}), per-sequence "
                     "capacity-doubling caches in one pool, one fused append+attention call per step",
                     round(by / dt / 1e9, 1), "GB/s", round(dt * 1e3, 5), "f16", roof,
                     {"steps": steps, "us_per_step": round(dt * 1e6, 1), "pool_bytes": st["bytes_total"],
                      "pool_in_use": st["bytes_in_use"], "pct_of_hbm_peak": round(100 * by / dt / 1e9 / HBM_PEAK_GBS, 2),
                      "parity_max_abs_vs_oracle": err,
                      "parity_sample": f"sequences {sample} (shortest, longest, two others), query heads 0, 13, 31, after the timed steps"})


def run_append(ta, args):
    """Kernels (1) and (2) on their own: the bulk append of a prefill (8 sequences x 8 kv heads x 16384 tokens x 128,
    f16 source) into a reserved cache, as plain f16 rows and quantised to Q8_0 / Q4_0 on the way, and the append of one
    decode token per sequence.  Two sources and two caches in turn (each pair moves more than the 256 MB Infinity Cache).
    Algorithmic bytes per element: 2 read + 2, 34/32 or 18/32 written."""
    from oracle import oracle as orc
    B, T = 8, 16384
    n_el = B * HKV * T * D
    srcs = [ta.DeviceTensor.from_numpy(seeded_f16(cfg_seed(4, "k") + i, (B, HKV, T, D))) for i in range(2)]
    tok = ta.DeviceTensor.from_numpy(seeded_f16(cfg_seed(4, "k") + 9, (B, HKV, 1, D)))
    res, turn = {}, [0]
    for name, fmt, wb in (("f16", None, 2.0), ("q8_0", ta.Q8_0, 34 / 32), ("q4_0", ta.Q4_0, 18 / 32)):
        caches = [ta.InPlaceKvCache(2, storage_format=fmt) for _ in range(2)]
        for c in caches:
            c.reserve(T + 64, like=((B, HKV, T, D), np.float16))
            c.push(srcs[0])

        def bulk():
            c = caches[turn[0] % 2]
            c.truncate(0)
            c.push(srcs[turn[0] % 2])
            turn[0] += 1

        us = time_calls(ta, bulk, 20)
        by = n_el * (2 + wb)
        res[f"bulk_append_{name}_8x8x16384x128"] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": int(by)}

        def one_token():
            c = caches[turn[0] % 2]
            c.truncate(T)
            c.push(tok)
            turn[0] += 1

        us1 = time_calls(ta, one_token, 200)
        res[f"token_append_{name}_8x8x1x128"] = {"us": round(us1, 2)}
        if fmt is not None:   # after the timing: the stored blocks of two heads against the oracle's, bit for bit
            c = caches[(turn[0] + 1) % 2]
            c.truncate(0)
            c.push(srcs[1])
            got = c.valid_contiguous()[3, 5]
            want = orc.quant(getattr(orc, "FMT_" + name.upper()), srcs[1].to_numpy()[3, 5])
            res[f"bulk_append_{name}_8x8x16384x128"]["blocks_bit_exact_vs_oracle"] = bool(got.tobytes() == want.tobytes())
        del caches
    head = res["bulk_append_q8_0_8x8x16384x128"]
    roof = {"bound": "hbm", "kernel": "quant_append_kernel<f16> (Q8_0)", "achieved": head["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(head["gbs"] / HBM_PEAK_GBS, 4), "traffic": None}
    return base_line(args, "append: bulk append of a 16384-token prefill (batch 8, 8 kv heads, d=128, f16 source) into a reserved "
                     "cache as f16 rows, Q8_0 and Q4_0 blocks, and the append of one token per sequence; headline = Q8_0 bulk append",
                     head["gbs"], "GB/s", round(head["us"] / 1e3, 5), "f16->q8_0", roof, {"cases": res})


def run_kivi(ta, args):
    """The KIVI-style quantised caches on their own: the ingest of a 16384-token prefill (8 x 8 kv heads x 128, f16 source)
    into per-token Value stores and block x channel Key stores at 8 and 4 bits, the dequantising read of the whole cache
    (the QuantizedDynKeyValueCache op's output) and one QuantizedKvSdpa decode step over 8192 tokens.  Algorithmic bytes
    per element: ingest reads 2 and writes bits / 8 (+ parameters); the read moves bits / 8 in and 2 out."""
    from oracle import oracle as orc
    from tract_amd import kivi
    B, T = 8, 16384
    n_el = B * HKV * T * D
    srcs = [ta.DeviceTensor.from_numpy(seeded_f16(cfg_seed(4, "k") + i, (B, HKV, T, D))) for i in range(2)]
    tok = ta.DeviceTensor.from_numpy(seeded_f16(cfg_seed(4, "k") + 9, (B, HKV, 1, D)))
    res, turn = {}, [0]
    for name, layout in (("value_per_token", kivi.KIVI_PER_TOKEN), ("key_block_channel", kivi.KIVI_BLOCK_CHANNEL)):
        for bits in (8, 4):
            caches = [kivi.KiviCache(layout, bits, kivi.SINK_TOKENS, B, HKV, D) for _ in range(2)]
            for c in caches:
                c.append(srcs[0])

            def bulk():
                c = caches[turn[0] % 2]
                c.reset()
                c.append(srcs[turn[0] % 2])
                turn[0] += 1

            us = time_calls(ta, bulk, 20)
            params = (B * HKV * T * 8) if layout == kivi.KIVI_PER_TOKEN else (B * HKV * (T // 32) * D * 8)
            by = n_el * (2 + bits / 8) + params
            res[f"ingest_{name}_{bits}bit_8x8x16384x128"] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": int(by)}
            outs = [ta.DeviceTensor((B, HKV, caches[0].len(), D), np.float16) for _ in range(2)]

            def read():
                caches[turn[0] % 2].dequantize(out=outs[turn[0] % 2])
                turn[0] += 1

            us = time_calls(ta, read, 20)
            by = n_el * (bits / 8 + 2) + params
            res[f"dequantize_{name}_{bits}bit_8x8x16384x128"] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": int(by)}
            us1 = time_calls(ta, lambda: caches[0].append(tok), 64)
            res[f"token_ingest_{name}_{bits}bit"] = {"us": round(us1, 2)}
            # after the timing: one head's state against the oracle's, bit for bit
            c = caches[1]
            c.reset()
            c.append(srcs[1])
            ref = orc.KiviStore(orc.KIVI_PER_TOKEN if layout == kivi.KIVI_PER_TOKEN else orc.KIVI_BLOCK_CHANNEL, D, bits)
            for row in srcs[1].to_numpy()[3, 5].astype(np.float32):
                ref.push_token(row)
            got, want = c.state(), ref.state()
            at = 3 * HKV + 5
            res[f"ingest_{name}_{bits}bit_8x8x16384x128"]["state_bit_exact_vs_oracle"] = bool(
                got["packed"][at].tobytes() == want["packed"].tobytes() and np.array_equal(got["lo"][at], want["lo"])
                and np.array_equal(got["scale"][at], want["scale"]) and got["sink"][at].tobytes() == want["sink"].tobytes())
            del caches, outs
    # QuantizedKvSdpa: one decode step over an 8192-token cache (one launch pushes the token, one attends over the codes)
    Tc = 8192
    st = ta.QuantizedKvSdpa(axis=2).state()
    kq_np, vq_np = seeded_f16(cfg_seed(2, "k"), (B, HKV, Tc, D)), seeded_f16(cfg_seed(2, "v"), (B, HKV, Tc, D))
    kq, vq = ta.DeviceTensor.from_numpy(kq_np), ta.DeviceTensor.from_numpy(vq_np)
    st.k = kivi.KiviCache(kivi.KIVI_RUNNING_CHANNEL, 8, 0, B, HKV, D)
    st.v = kivi.KiviCache(kivi.KIVI_PER_TOKEN, 8, 0, B, HKV, D)
    st.k.append(kq), st.v.append(vq)

    def prompt():
        st.k.reset()
        st.k.append(kq)

    res["prompt_push_running_keys_8x8x8192x128"] = {"us": round(time_calls(ta, prompt, 8), 2),
                                                    "note": "chunked scan over 64-token chunks (two passes with 128-bit rows, one scan of the chunk results between them), incl. the reset of the running parameters; the scratch belongs to the store"}
    q1_np = (seeded_f16(cfg_seed(2, "q") + 1, (B, HQ, 1, D)).astype(np.float32) / np.sqrt(D)).astype(np.float16)
    q1 = ta.DeviceTensor.from_numpy(q1_np)
    out = ta.DeviceTensor((B, HQ, 1, D), np.float16)
    us = time_calls(ta, lambda: st.eval([q1, tok, tok], out=out), 32)
    T_end = st.k.len()
    step_bytes = B * HKV * (Tc + (T_end - Tc) // 2) * (2 * D + 8) + B * HKV * D * 8 + 2 * B * HQ * D * 2
    case = {"us": round(us, 2), "bytes": step_bytes, "gbs": round(step_bytes / us / 1e3, 1),
            "note": "the new token's K and V rows pushed by one launch + attention straight over the u8 codes (TROCM_KIVI_FUSED=0: push + dequantise K and V + f16 attention)"}
    # after the timing: the last step's output for one kv head against the oracle's attention over its own stores
    b0, h0, g = 5, 3, HQ // HKV
    tok_np = tok.to_numpy()
    kc, vc = orc.KiviCache(True, running=True), orc.KiviCache(False, running=True)
    kc.ingest(kq_np[b0:b0 + 1, h0:h0 + 1]), vc.ingest(vq_np[b0:b0 + 1, h0:h0 + 1])
    for _ in range(T_end - Tc):
        kc.ingest(tok_np[b0:b0 + 1, h0:h0 + 1]), vc.ingest(tok_np[b0:b0 + 1, h0:h0 + 1])
    want = orc.flash_sdpa(q1_np[b0:b0 + 1, h0 * g:(h0 + 1) * g].astype(np.float32), kc.dequantized(), vc.dequantized(), causal=False)
    case["parity_max_abs_vs_oracle"] = float(np.abs(out.to_numpy()[b0:b0 + 1, h0 * g:(h0 + 1) * g].astype(np.float32) - want).max())
    res["quantized_kv_sdpa_step_b8_ctx8192"] = case
    head = res["dequantize_key_block_channel_8bit_8x8x16384x128"]
    roof = {"bound": "hbm", "kernel": "kivi_dequant_kernel<f16, 8>", "achieved": head["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(head["gbs"] / HBM_PEAK_GBS, 4), "traffic": None}
    return base_line(args, "kivi: KIVI-style affine quantised caches (8 x 8 kv heads x 16384 tokens x 128, f16): ingest into per-token "
                     "Value and block x channel Key stores at 8 / 4 bits, the dequantising read of the whole cache, one QuantizedKvSdpa "
                     "decode step at 8192 tokens (attention over the codes); headline = the 8-bit Key cache read", head["gbs"], "GB/s", round(head["us"] / 1e3, 5),
                     "u8->f16", roof, {"cases": res})


def run_ops(ta, args):
    """The ops either side of the cache (RoPE, cast) and the sliding-window decode step, each against
    its HBM roofline, with the oracle timed on the host for the same ops (smaller sample)."""
    from oracle import oracle as orc
    res = {}
    rng = np.random.default_rng(7)
    # RoPE on a prefill chunk: Q [1, 32, 4096, 128] f16 against [4096, 128] tables, rotating over 8 inputs (> 256 MB)
    S = 4096
    xs = [ta.DeviceTensor.from_numpy(rng.standard_normal((1, HQ, S, D)).astype(np.float16)) for _ in range(8)]
    ang = rng.uniform(-3, 3, (S, D)).astype(np.float32)
    cos, sin = ta.DeviceTensor.from_numpy(np.cos(ang).astype(np.float16)), ta.DeviceTensor.from_numpy(np.sin(ang).astype(np.float16))
    out = ta.DeviceTensor((1, HQ, S, D), np.float16)
    rope, turn = ta.ApplyRope(), [0]

    def one_rope():
        rope.eval(xs[turn[0] % 8], cos, sin, out=out)
        turn[0] += 1

    us = time_calls(ta, one_rope, 80)
    by = 2 * HQ * S * D * 2 + 2 * S * D * 2   # x read, y written, tables once
    res["apply_rope_f16_1x32x4096x128"] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": by}
    # cast f32 -> f16, 64 Mi elements, rotating over 4 inputs
    n = 64 << 20
    cs = [ta.DeviceTensor.from_numpy(rng.standard_normal(n, dtype=np.float32)) for _ in range(4)]
    cast = ta.Cast(np.float16)
    us = time_calls(ta, lambda: cast.eval(cs[0]), 3)   # warm the allocator path once
    dst = ta.DeviceTensor((n,), np.float16)
    from tract_amd._lib import call

    def one_cast():
        call("trocm_cast", cs[turn[0] % 4].ptr, 0, dst.ptr, 1, n, None)
        turn[0] += 1

    us = time_calls(ta, one_cast, 40)
    res["cast_f32_f16_64Mi"] = {"us": round(us, 2), "gbs": round(n * 6 / us / 1e3, 1), "bytes": n * 6}
    # sliding-window decode step: batch 8, window 4096, full ring (append wraps), 4 layers
    W, B = 4096, 8
    sts = [ta.WindowKvSdpa(axis=2, window=W).state() for _ in range(4)]
    k0 = rng.standard_normal((B, HKV, W + 100, D)).astype(np.float16)
    q0 = ta.DeviceTensor.from_numpy((rng.standard_normal((B, HQ, W + 100, D)) / np.sqrt(D)).astype(np.float16))
    for st in sts:
        st.eval([q0, k0, k0])
    del q0
    q1 = ta.DeviceTensor.from_numpy((rng.standard_normal((B, HQ, 1, D)) / np.sqrt(D)).astype(np.float16))
    k1 = ta.DeviceTensor.from_numpy(rng.standard_normal((B, HKV, 1, D)).astype(np.float16))
    o1 = ta.DeviceTensor((B, HQ, 1, D), np.float16)

    def one_win():
        sts[turn[0] % 4].eval([q1, k1, k1], out=o1)
        turn[0] += 1

    us = time_calls(ta, one_win, 100)
    by = algorithmic_bytes(B, W)
    res["window_kv_sdpa_step_b8_w4096"] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": int(by)}
    del sts, xs, cs
    # the attention block of a decoder layer's step as an exported graph states it: ApplyRope on Q, ApplyRope on K_new,
    # InPlaceKvSdpa -- as three calls (three launches) and through the entry point that rotates both inside the attention
    # launch; cfg2's shape at 8192 tokens over 4 layers' caches, batch 8 and batch 1
    for Bs, fmt, tag in ((8, None, ""), (1, None, ""), (8, ta.Q4_0, "_q4_0")):
        T0 = 8192
        lay = [ta.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state() for _ in range(4)]
        kk = rng.standard_normal((Bs, HKV, T0, D)).astype(np.float16)
        for st in lay:
            for c in (st.k, st.v):
                c.reserve(T0 + 1024, like=(kk.shape, kk.dtype))
                c.push(kk)
        del kk
        qd = ta.DeviceTensor.from_numpy((rng.standard_normal((Bs, HQ, 1, D)) / np.sqrt(D)).astype(np.float16))
        kd = ta.DeviceTensor.from_numpy(rng.standard_normal((Bs, HKV, 1, D)).astype(np.float16))
        angs = rng.uniform(-3, 3, (Bs, 1, 1, D)).astype(np.float32)
        cd, sd = ta.DeviceTensor.from_numpy(np.cos(angs).astype(np.float16)), ta.DeviceTensor.from_numpy(np.sin(angs).astype(np.float16))
        qr, kr = ta.DeviceTensor(qd.shape, np.float16), ta.DeviceTensor(kd.shape, np.float16)
        od = ta.DeviceTensor(qd.shape, np.float16)

        # (raw C calls with their arguments built once: at batch 1 the host mirror's Python would be what is timed)
        import ctypes as C
        ws = ta.Workspace(Bs, HQ, 1, D)
        nanf = C.c_float(float("nan"))
        qshape, kshape = (C.c_int64 * 4)(Bs, HQ, 1, D), (C.c_int64 * 4)(Bs, HKV, 1, D)
        cstr = (C.c_int64 * 4)(D, 0, D, 1)
        hk, hv = [st.k.handle for st in lay], [st.v.handle for st in lay]

        def three_calls():
            i = turn[0] % 4
            call("trocm_apply_rope", qd.ptr, cd.ptr, sd.ptr, qr.ptr, 1, 4, qshape, None, cstr, None, None)
            call("trocm_apply_rope", kd.ptr, cd.ptr, sd.ptr, kr.ptr, 1, 4, kshape, None, cstr, None, None)
            call("trocm_inplace_kv_sdpa_eval", qr.ptr, kr.ptr, kd.ptr, 1, HQ, 1, None, hk[i], hv[i], od.ptr, nanf, 1, ws.ptr, ws.nbytes, None)
            turn[0] += 1

        def one_call():
            i = turn[0] % 4
            call("trocm_inplace_kv_sdpa_eval_rope", qd.ptr, kd.ptr, kd.ptr, cd.ptr, sd.ptr, D, 1, HQ, 1, hk[i], hv[i], od.ptr, nanf, 1,
                 ws.ptr, ws.nbytes, None, 0, None)
            turn[0] += 1

        def plain_step():   # the step without any rotation, for scale
            i = turn[0] % 4
            call("trocm_inplace_kv_sdpa_eval", qd.ptr, kd.ptr, kd.ptr, 1, HQ, 1, None, hk[i], hv[i], od.ptr, nanf, 1, ws.ptr, ws.nbytes, None)
            turn[0] += 1

        us3 = time_calls(ta, three_calls, 100)
        us1 = time_calls(ta, one_call, 100)
        us0 = time_calls(ta, plain_step, 100)
        res[f"rope_rope_step_b{Bs}_ctx8192{tag}"] = {"three_calls_us": round(us3, 2), "fused_us": round(us1, 2), "step_without_rope_us": round(us0, 2),
                                                "note": "ApplyRope(Q), ApplyRope(K_new), InPlaceKvSdpa step: three launches against one"}
        del lay
    # mask inputs on the fast attention kernels: decode (batch 8, 8192 tokens, padding mask [8,1,1,T]) over
    # 4 layers' K/V, and a 512-query chunk over 4096 keys with the causal mask stated as an input [1,1,512,4096]
    T = 8192
    kvs = [(ta.DeviceTensor.from_numpy(rng.standard_normal((B, HKV, T, D)).astype(np.float16)),
            ta.DeviceTensor.from_numpy(rng.standard_normal((B, HKV, T, D)).astype(np.float16))) for _ in range(4)]
    pad = np.zeros((B, 1, 1, T), np.float16)
    for b in range(B):
        pad[b, :, :, T - 37 * b:] = np.finfo(np.float16).min
    pad = ta.DeviceTensor.from_numpy(pad)
    sd = ta.Sdpa(datum_type=np.float16)

    def one_masked(masked):
        kk, vv = kvs[turn[0] % 4]
        sd.eval(q1, kk, vv, pad if masked else None, out=o1)
        turn[0] += 1

    by = algorithmic_bytes(B, T)
    for name, masked in (("decode_b8_ctx8192_padding_mask", True), ("decode_b8_ctx8192_no_mask", False)):
        us = time_calls(ta, lambda: one_masked(masked), 100)
        res[name] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": int(by)}
    # the reference's statement of a ragged batch: padded to 8192 tokens, sequence b holds 8192 - 1024 * b of them
    pad2 = np.zeros((B, 1, 1, T), np.float16)
    for b in range(B):
        pad2[b, :, :, T - 1024 * b:] = np.finfo(np.float16).min
    pad, by2 = ta.DeviceTensor.from_numpy(pad2), sum(algorithmic_bytes(1, T - 1024 * b) for b in range(B))
    us = time_calls(ta, lambda: one_masked(True), 100)
    res["decode_b8_padded_to_8192_lens_8192_down_to_1024"] = {"us": round(us, 2), "gbs": round(by2 / us / 1e3, 1), "bytes": int(by2)}
    Sq, Sk = 512, 4096
    qp = ta.DeviceTensor.from_numpy((rng.standard_normal((1, HQ, Sq, D)) / np.sqrt(D)).astype(np.float16))
    op = ta.DeviceTensor((1, HQ, Sq, D), np.float16)
    cm = np.where(np.arange(Sk)[None, :] > np.arange(Sq)[:, None] + (Sk - Sq), np.finfo(np.float16).min, 0).astype(np.float16)
    cm = ta.DeviceTensor.from_numpy(cm.reshape(1, 1, Sq, Sk))
    kk, vv = kvs[0]
    kp = ta.DeviceTensor.from_numpy(kk.to_numpy()[:1, :, :Sk].copy())
    vp = ta.DeviceTensor.from_numpy(vv.to_numpy()[:1, :, :Sk].copy())
    sc = ta.Sdpa(datum_type=np.float16, is_causal=True)
    fl = 4.0 * HQ * D * (Sq * Sk - Sq * (Sq - 1) / 2)
    us = time_calls(ta, lambda: sd.eval(qp, kp, vp, cm, out=op), 50)
    res["prefill_512x4096_causal_as_mask_input"] = {"us": round(us, 2), "tflops": round(fl / us / 1e6, 1)}
    us = time_calls(ta, lambda: sc.eval(qp, kp, vp, out=op), 50)
    res["prefill_512x4096_is_causal"] = {"us": round(us, 2), "tflops": round(fl / us / 1e6, 1)}
    # the same chunk over Q8_0 / Q4_0 caches of 4096 tokens (blocks dequantised while the tiles are staged)
    for name, fmt in (("q8_0", ta.Q8_0), ("q4_0", ta.Q4_0)):
        stq = ta.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state()
        stq.k.push(kp), stq.v.push(vp)
        us = time_calls(ta, lambda: stq.attend(qp, out=op), 50)
        res[f"prefill_512x4096_{name}_cache"] = {"us": round(us, 2), "tflops": round(fl / us / 1e6, 1)}
        del stq
    del kvs, kp, vp
    # Q4_0 weights x one activation row (the decode-time projections of an 8B-class decoder), f16; each
    # shape rotates over 8 weight matrices so that launches read HBM
    gemm = ta.GgmlGemm()
    for n_, k_ in ((14336, 4096), (4096, 14336), (4096, 4096), (1024, 4096), (128256, 4096)):
        # (1024 x 4096, the key / value projection: a matrix this small holds tiles and planes, rows 1 and 2 run over the
        # planes; 64 matrices in rotation)
        nw = 3 if n_ > 100000 else 64 if n_ < 2048 else 8
        blob = rng.integers(0, 256, (n_, k_ // 32 * 18), dtype=np.uint8)
        blob[:, 1::18] = (blob[:, 1::18] & 0x03) | 0x28      # scales: small finite f16 values
        ws = [ta.Q40Weights(blob, 1, n_, k_) for _ in range(nw)]
        # 1..16 f16 rows against the tiles, and against the same matrices as planes of codes and scales (what a matrix
        # that is not whole tiles of 16 rows x 128 features is held as)
        os.environ["TROCM_Q4_TILED"] = "0"
        wp = [ta.Q40Weights(blob, 1, n_, k_) for _ in range(nw)]
        del os.environ["TROCM_Q4_TILED"]
        for m_ in (1, 2, 4, 8, 16):
            xp = ta.DeviceTensor.from_numpy(rng.standard_normal((1, m_, k_)).astype(np.float16))
            op = ta.DeviceTensor((1, m_, n_), np.float16)
            row = {}
            for tag, mats in (("tiles_us", ws), ("planes_us", wp)):
                def one_rows():
                    gemm.eval(xp, mats[turn[0] % nw], out=op)
                    turn[0] += 1

                row[tag] = round(time_calls(ta, one_rows, 200), 2)
            row["tiles_gbs"] = round((n_ * (k_ // 32) * 18 + m_ * 2 * (k_ + n_)) / row["tiles_us"] / 1e3, 1)
            res[f"q4_0_rows_f16_m{m_}_n{n_}_k{k_}"] = row
        del wp
        # f32 activations: one and four rows (three bf16 parts per activation as rows of the matrix instruction)
        for m_ in (1, 4):
            xf = ta.DeviceTensor.from_numpy(rng.standard_normal((1, m_, k_)).astype(np.float32))
            of = ta.DeviceTensor((1, m_, n_), np.float32)

            def one_f32():
                gemm.eval(xf, ws[turn[0] % nw], out=of)
                turn[0] += 1

            res[f"q4_0_matvec_f32_m{m_}_n{n_}_k{k_}"] = {"us": round(time_calls(ta, one_f32, 200), 2)}
        if n_ > 100000:
            del ws
            continue
        xa = ta.DeviceTensor.from_numpy(rng.standard_normal((1, 1, k_)).astype(np.float16))
        oa = ta.DeviceTensor((1, 1, n_), np.float16)

        def one_mv():
            gemm.eval(xa, ws[turn[0] % nw], out=oa)
            turn[0] += 1

        us = time_calls(ta, one_mv, 200)
        by = n_ * (k_ // 32) * 18 + 2 * k_ + 2 * n_
        res[f"q4_0_matvec_f16_n{n_}_k{k_}"] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": by}
        # the same weights x the 8 rows of a batch-8 decode step: 16 weight rows x 8 activation rows per matrix
        # instruction, still bound by the weights' bytes
        x8 = ta.DeviceTensor.from_numpy(rng.standard_normal((1, 8, k_)).astype(np.float16))
        o8 = ta.DeviceTensor((1, 8, n_), np.float16)

        def one_mv8():
            gemm.eval(x8, ws[turn[0] % nw], out=o8)
            turn[0] += 1

        us = time_calls(ta, one_mv8, 200)
        by8 = n_ * (k_ // 32) * 18 + 8 * 2 * k_ + 8 * 2 * n_
        res[f"q4_0_matvec_f16_m8_n{n_}_k{k_}"] = {"us": round(us, 2), "gbs": round(by8 / us / 1e3, 1), "bytes": by8}
        # the same weights x the rows of a batch-32 step and of a prefill chunk (128, 512, 2048): the matrix-matrix arm
        for m_ in (32, 128, 512, 2048):
            xm = ta.DeviceTensor.from_numpy(rng.standard_normal((1, m_, k_)).astype(np.float16))
            om = ta.DeviceTensor((1, m_, n_), np.float16)

            def one_mm():
                gemm.eval(xm, ws[turn[0] % nw], out=om)
                turn[0] += 1

            us = time_calls(ta, one_mm, 50)
            res[f"q4_0_matmul_f16_m{m_}_n{n_}_k{k_}"] = {"us": round(us, 2), "tflops": round(2.0 * m_ * n_ * k_ / us / 1e6, 1)}
            del xm, om
        del ws
    # ragged decode step over quantised caches: 32 sequences of 512..32768 tokens, their new tokens quantised
    # by one launch and attention by another
    n_seq = 32
    lens = np.random.default_rng(cfg_seed(5, "q") + 3).integers(512, 32768, size=n_seq, endpoint=True)
    for fmt, name, rb in ((ta.Q8_0, "q8_0", 136), (ta.Q4_0, "q4_0", 72)):
        pool = ta.KvPool(int(lens.sum()) * HKV * rb * 2 * 3 + (64 << 20))
        kcs, vcs = [], []
        for n_ in lens:
            kk = rng.standard_normal((1, HKV, int(n_), D), dtype=np.float32).astype(np.float16)
            kc, vc = ta.InPlaceKvCache(2, fmt, pool=pool), ta.InPlaceKvCache(2, fmt, pool=pool)
            kc.push(kk), vc.push(kk)
            kcs.append(kc), vcs.append(vc)
        wsr = ta.Workspace(n_seq, HQ, 1, D)
        qr = ta.DeviceTensor.from_numpy((rng.standard_normal((n_seq, HQ, 1, D)) / np.sqrt(D)).astype(np.float16))
        knr = ta.DeviceTensor.from_numpy(rng.standard_normal((n_seq, HKV, 1, D)).astype(np.float16))
        outr = ta.DeviceTensor((n_seq, HQ, 1, D), np.float16)
        us = time_calls(ta, lambda: ta.inplace_kv_sdpa_eval_ragged(qr, knr, knr, kcs, vcs, workspace=wsr, out=outr), 16)
        by = 2 * HKV * int(sum(c.len() for c in kcs)) * rb
        res[f"ragged_step_{name}_32seq"] = {"us": round(us, 2), "gbs": round(by / us / 1e3, 1), "bytes": by}
        del kcs, vcs, pool
    # the oracle on the host for the same ops, on a bounded sample
    xh = rng.standard_normal((1, 4, S, D)).astype(np.float16)
    t0 = time.perf_counter()
    orc.apply_rope(xh, np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16))
    t_rope = (time.perf_counter() - t0) * (HQ / 4)
    cpu = {"value": round(res["apply_rope_f16_1x32x4096x128"]["bytes"] / t_rope / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
           "sample": "ApplyRope of 4 of the 32 heads with the scalar C restatement, scaled to 32"}
    head = res["apply_rope_f16_1x32x4096x128"]
    roof = {"bound": "hbm", "kernel": "apply_rope_vec_kernel<f16>", "achieved": head["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(head["gbs"] / HBM_PEAK_GBS, 4), "traffic": None}
    line = base_line(args, "ops: ApplyRope on a 4096-token prefill chunk (32 heads, d=128, f16), cast f32->f16 of 64 Mi "
                     "elements, sliding-window decode step (batch 8, window 4096); inputs rotate so that launches read HBM",
                     head["gbs"], "GB/s", round(head["us"] / 1e3, 5), "f16", roof, {"cases": res})
    line["cpu_baseline"] = cpu
    return line


def run_floors(ta, args):
    """What a short launch costs before any kernel logic: an empty kernel and a read-only streaming kernel
    (non-temporal 128-bit loads, eight in flight per thread, nothing written) on the decode kernels' launch
    shapes, over the byte counts of the short decode launches; then those decode launches themselves as a
    fraction of the streaming kernel's time on the same bytes."""
    from tract_amd._lib import call
    res = {}
    rng = np.random.default_rng(11)
    sizes = {"33.6MB (f16, batch 1, 8192 tokens)": 2 * 1 * HKV * 8192 * D * 2 + 2 * HQ * D * 2,
             "37.8MB (Q4_0, batch 8, 4096 tokens)": 2 * 8 * HKV * 4096 * D * 18 // 32 + 2 * 8 * HQ * D * 2,
             "71.3MB (Q8_0, batch 8, 4096 tokens)": 2 * 8 * HKV * 4096 * D * 34 // 32 + 2 * 8 * HQ * D * 2,
             "268.6MB (f16, batch 8, 8192 tokens)": 2 * 8 * HKV * 8192 * D * 2 + 2 * 8 * HQ * D * 2}
    big = max(sizes.values())
    n_buf = 4   # every launch reads another buffer; short sizes stride through all of them: nothing is found in a cache
    bufs = [ta.DeviceTensor.from_numpy(rng.integers(0, 255, ((big + 15) // 16 * 16,), dtype=np.uint8)) for _ in range(n_buf)]
    sink = ta.DeviceTensor((4,), np.uint8)
    turn = [0]
    shapes = [(256, 256), (512, 256), (1024, 256), (2048, 256), (512, 512), (256, 1024)]
    for wg, th in shapes:
        us = time_calls(ta, lambda: call("trocm_launch_floor", 0, None, 0, wg, th, None, None), 200)
        res[f"empty_kernel_{wg}x{th}"] = {"us": round(us, 2)}
    floor = {}
    for name, nbytes in sizes.items():
        nb16 = nbytes // 16 * 16
        per_buf = max(1, big // nb16)   # disjoint windows of one buffer, then the next buffer
        best = None
        for wg, th in shapes:
            def one():
                i = turn[0]
                turn[0] += 1
                b = bufs[(i // per_buf) % n_buf]
                call("trocm_launch_floor", 1, b.ptr.value + (i % per_buf) * nb16, nb16, wg, th, sink.ptr, None)
            us = time_calls(ta, one, 100)
            res[f"stream_read_{name.split(' ')[0]}_{wg}x{th}"] = {"us": round(us, 2), "gbs": round(nb16 / us / 1e3, 1)}
            best = us if best is None else min(best, us)
        floor[name] = best
    del bufs
    # the decode launches over the same bytes (attention launch only; caches of several layers in turn)
    def decode_case(B, T, fmt, layers):
        sts = [ta.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state() for _ in range(layers)]
        k = seeded_f16(cfg_seed(4, "k") + T + B, (B, HKV, T, D))
        for st in sts:
            for c in (st.k, st.v):
                c.reserve(T + 1024, like=(k.shape, k.dtype))
                c.push(k)
        q = ta.DeviceTensor.from_numpy((seeded_f16(cfg_seed(4, "q"), (B, HQ, 1, D)).astype(np.float32) / np.sqrt(D)).astype(np.float16))
        out = ta.DeviceTensor((B, HQ, 1, D), np.float16)

        def one():
            sts[turn[0] % layers].attend(q, out=out)
            turn[0] += 1
        return time_calls(ta, one, 200)
    cases = {"33.6MB (f16, batch 1, 8192 tokens)": (1, 8192, None, 10), "37.8MB (Q4_0, batch 8, 4096 tokens)": (8, 4096, ta.Q4_0, 8),
             "71.3MB (Q8_0, batch 8, 4096 tokens)": (8, 4096, ta.Q8_0, 5), "268.6MB (f16, batch 8, 8192 tokens)": (8, 8192, None, 2)}
    for name, (B, T, fmt, layers) in cases.items():
        us = decode_case(B, T, fmt, layers)
        res[f"decode_{name.split(' ')[0]}"] = {"us": round(us, 2), "gbs": round(sizes[name] / us / 1e3, 1), "best_stream_read_us": round(floor[name], 2),
                                                "stream_read_time_over_decode_time": round(floor[name] / us, 3)}
    head = res["decode_33.6MB"]
    roof = {"bound": "hbm", "kernel": "sdpa_decode_mfma_kernel<128,8,F16,false,true,0> at batch 1", "achieved": head["gbs"], "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(head["gbs"] / HBM_PEAK_GBS, 4), "traffic": None}
    return base_line(args, "floors: an empty kernel and a read-only streaming kernel on the decode launch shapes over the byte counts "
                     "of the short decode launches, and those launches beside them (headline: batch-1 decode over 8192 tokens)",
                     head["gbs"], "GB/s", round(head["us"] / 1e3, 5), "f16", roof, {"cases": res})


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8, help="headline batch size")
    ap.add_argument("--other-batches", type=str, default="1,32")
    ap.add_argument("--kernel-iters", type=int, default=200)
    ap.add_argument("--windows", type=int, default=5, help="how many times the timed window of --steps steps is taken (median reported)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--workload", default="cfg2", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "ops", "append", "kivi", "floors"],
                    help="cfg2 (default) is the configuration the metric is quoted on; the others print one line "
                         "of the same shape for the remaining configurations")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this path is measured on one GPU; --gpus {args.gpus} is not supported "
              "(no sharding, no collectives in this build)", file=sys.stderr)
        sys.exit(2)

    import tract_amd as ta
    rt = ta.runtime_for_name("rocm")
    if args.workload != "cfg2":
        line = {"cfg1": run_cfg1, "cfg3": run_cfg3, "cfg4": run_cfg4, "cfg5": run_cfg5, "ops": run_ops, "append": run_append, "kivi": run_kivi, "floors": run_floors}[args.workload](ta, args)
        line["device"] = rt.device_name
        print(json.dumps(line))
        return
    main_res = run_batch(ta, args.batch, args.steps, args.warmup, args.kernel_iters, windows=args.windows)

    # parity spot check of the last output against the oracle (checker only)
    from oracle import oracle as orc
    st = main_res.pop("state")
    kd, vd = st.k.valid_contiguous(), st.v.valid_contiguous()
    want = orc.flash_sdpa(main_res["last_q"][:1], kd[:1], vd[:1], causal=True, threads=8)
    err = float(np.abs(want.astype(np.float32) - main_res["last_out"][:1].astype(np.float32)).max())
    del kd, vd, st
    main_res.pop("last_out"), main_res.pop("last_q")

    others = {}
    for b in [int(x) for x in args.other_batches.split(",") if x]:
        r = run_batch(ta, b, args.steps, args.warmup, args.kernel_iters, windows=args.windows)
        for key in ("state", "last_out", "last_q"):
            r.pop(key)
        others[str(b)] = {k: (round(v, 3) if isinstance(v, float) else v) for k, v in r.items()}

    # HBM traffic of a launch: counted at batch 8 with 8226 tokens in the kernel loop; K and V make up all but
    # 0.3 % of it, so another context at batch 8 is that figure scaled by the algorithmic bytes.  Not counted for
    # other batch sizes.
    traffic, traffic_note = None, "counted at batch 8 only"
    if args.batch == 8:
        traffic = int(PMC_TRAFFIC_BYTES_B8_CTX8226 * main_res["step_bytes"] / PMC_ALGORITHMIC_BYTES_B8_CTX8226)
        traffic_note = ("rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE per launch at batch 8, 8226 tokens "
                        f"({PMC_TRAFFIC_BYTES_B8_CTX8226} bytes for {PMC_ALGORITHMIC_BYTES_B8_CTX8226} algorithmic), scaled by this run's "
                        "algorithmic bytes per launch")
    line = {
        "metric": "decode-attn over KV cache: achieved HBM GB/s (% of peak) + us/token at 8k ctx",
        "value": round(main_res["step_gbs"], 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_res["ms_per_step"], 5),
        "us_per_token": round(main_res["us_per_token"], 2),
        "wall_ms_per_step": round(main_res["wall_ms_per_step"], 5),
        "wall_value": round(main_res["wall_step_gbs"], 2),
        "timing": {"value_clock": "HIP events on the stream around each window of --steps steps, median window",
                   "windows": main_res["windows"], "window_ms_per_step_min_max": main_res["window_ms_per_step_min_max"],
                   "wall_clock": "time.perf_counter around the same window between two device synchronisations "
                                 "(adds one launch + one synchronisation latency per window)"},
        "pct_of_hbm_peak": round(100 * main_res["step_gbs"] / HBM_PEAK_GBS, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"cfg2: GQA decode layer 32q/8kv d=128 f16, batch {args.batch}, KV caches of {LAYERS} layers "
                               f"prefilled to {CTX} tokens, {args.steps} steps (single-token append + decode "
                               f"attention) visiting the layers round-robin; {PREWARM_LAUNCHES} untimed attention launches "
                               f"before the warm-up steps bring the device to steady clocks; value = algorithmic bytes of a "
                               f"step / device time per step (HIP events on the stream around the {args.steps} steps, median of "
                               f"{args.windows} such windows); wall_value = the same over the host's clock; each layer's one capacity "
                               f"doubling (8192 -> 16384) falls into the warm-up steps and is reported under capacity_doubling",
                   "batch": args.batch, "layers": LAYERS, "context": CTX, "q_heads": HQ, "kv_heads": HKV, "head_dim": D,
                   "prewarm_launches": PREWARM_LAUNCHES},
        "device": rt.device_name,
        "parity_max_abs_vs_oracle": err,
        "roofline": {
            "bound": "hbm",
            "kernel": "sdpa_decode_mfma_kernel<128,8,F16,false,true> (one launch per step: attention with the new token's append fused in)",
            "achieved": round(main_res["step_gbs"], 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(main_res["step_gbs"] / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_note": traffic_note,
            "kernel_us": round(main_res["us_per_token"], 3),
            "kernel_us_note": "average launch duration = the timed windows' event time / steps (a step is this one launch), median window",
            "algorithmic_bytes_per_launch": main_res["step_bytes"],
            "attention_only_loop": {"us": round(main_res["kernel_us"], 3), "us_min_max": main_res["kernel_us_min_max"],
                                    "gbs": round(main_res["kernel_gbs"], 2), "bytes": main_res["kernel_bytes"],
                                    "note": "the same kernel without the append (windows of launches of `attend`, median)"},
            "cache_resident_achieved": round(main_res["cache_resident_kernel_gbs"], 2),
            "cache_resident_kernel_us": round(main_res["cache_resident_kernel_us"], 3),
        },
        "capacity_doubling": {"step_us_with_growth": round(main_res["growth_step_us"], 2),
                              "us_per_token_amortised_over_128_steps": round(main_res["growth_us_per_token_over_128_steps"], 3),
                              "generation_us_per_token": round(main_res["us_per_token"] + main_res["growth_us_per_token_over_128_steps"], 3),
                              "note": "each layer's one doubling 8192 -> 16384 (K and V moved to new planes) happens in its first "
                                      "step, which is a warm-up step here and timed on its own; generation_us_per_token = steady step + "
                                      "that cost spread over cfg2's 128 steps"},
        "other_batches": others,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args.batch)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
