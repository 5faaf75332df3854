#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

Primary workload (the JSON line's value): single-token attention, Qwen3-30B-A3B
shapes — 16 sequences x 8192 cached tokens, 32 query / 4 KV heads, head_dim 128,
fp16, dimension-first cache.  One step = one Attention::run(position 8191,
interval 1, batch 16).  K/V are already resident in HBM; four cache copies are
rotated between steps so a step never re-reads lines still sitting in the
256 MB infinity cache.

Also reported on the same line (`also`): the 32k-token causal GQA prefill
(TFLOP/s against the dense fp16 MFMA peak) and single-token attention over one
128k-token cache.

`cpu_baseline` times the CPU oracle (a port of the reference's per-row
recurrence, binary32) on this machine's host cores.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu] [--only NAME]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a plain
# copy of known size; summaries and commands under profiles/).  Not measurable from inside
# this script; null for workloads without a counter run.
TRAFFIC_BYTES = {
    "decode": (2 * 131928 + 2252) * 1024,      # 16 x 8192
    "decode128k": (2 * 131745 + 2261) * 1024,  # 1 x 131072
    "lastchunk": (2 * (198592 + 15674) + 31309 + 3120) * 1024,   # 16 tokens x 24: stream kernel + merge launch
    "mixed_decode": (2 * 2257752 + 3286) * 1024,                 # 32 sequences U{1024..131072}, seed 7
    "prefill": (1363516 + 319881) * 1024,
    "kvwrite": (73808 + 65536) * 1024,
    "qkv": (1130126 + 327680) * 1024,          # fetched past the L2s (mostly from the last-level cache) + written
    "stepproj": (2 * 10695 + 1318) * 1024,
    # 48 layers of the fused step, 16 x 8192: raw Q/K/V sums + attention finishing them + output projection
    "layerstep_16x8192": 48 * (2 * (10534 + 131938 + 8990) + 320 + 2378 + 128) * 1024,
}
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA, published
D = 128


def _dev_normal(shape, dtype, seed, scale=1.0):
    import torch

    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    x = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32)
    if scale != 1.0:
        x *= scale
    return x.to(dtype)


MIN_TIMED_MS = 100.0   # a measurement repeats its K-step pass until this much has been timed
MAX_PASSES = 400
_last_passes = 0


def _time_steps(fn, steps, warmup, min_ms=None):
    """W untimed steps, then passes of exactly K steps each, every pass between two
    synchronisation points, repeated until MIN_TIMED_MS of device time has been measured
    (a 20-step pass of a 47 us kernel is 1 ms: one preemption or clock ramp moves it by
    several per cent).  Returns ([median launch duration in ms], median host-clock ms per step).

    Per pass the host clock brackets the K steps with torch.cuda.synchronize() on both sides,
    and two HIP events recorded on the launch stream (the library launches on torch's current
    stream, where the events are recorded too) bracket the same K launches: one step of a
    single-kernel workload is one launch and the launches run back to back, so elapsed / K
    is that kernel's average duration (an event pair around every single launch adds several
    microseconds of command-processor work per step and overstates a 50 us kernel by 10 %).
    The number of passes of the last call is left in _last_passes."""
    import statistics

    import torch

    global _last_passes
    if min_ms is None:
        min_ms = MIN_TIMED_MS
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    host, dev, total = [], [], 0.0
    n = warmup
    while True:
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record()
        for i in range(steps):
            fn(n + i)
        stop.record()
        torch.cuda.synchronize()
        host.append((time.perf_counter() - t0) * 1e3 / steps)
        ms = start.elapsed_time(stop)
        dev.append(ms / steps)
        total += ms
        n += steps
        if total >= min_ms or len(dev) >= MAX_PASSES:
            break
    _last_passes = len(dev)
    return [statistics.median(dev)], statistics.median(host)


def bench_decode(batch, length, steps, warmup, hq=32, hkv=4, copies=4):
    import torch

    import ellm_amd

    cap = length
    scale = 1.0 / D ** 0.5
    ops = []
    for c in range(copies):
        k = _dev_normal((batch, hkv, cap, D), torch.float16, 100 + c)
        v = _dev_normal((batch, hkv, cap, D), torch.float16, 200 + c)
        q = _dev_normal((1, batch, hq, D), torch.float16, 300 + c)
        out = torch.zeros_like(q)
        lse = torch.zeros((1, batch, hq), dtype=torch.float32, device="cuda")
        op = ellm_amd.Attention(q, k, v, out, batch, hq, hkv, D, [hkv * cap * D, cap * D, D, 1],
                                scale, lse=lse, sequence_capacity=cap, max_position_interval=1)
        ops.append(op)
    per, step_ms = _time_steps(lambda i: ops[i % copies].run(length - 1, 1, batch), steps, warmup)
    alg_bytes = 2 * batch * hkv * length * D * 2 + 2 * batch * hq * D * 2
    kern_ms = sum(per) / len(per)
    for op in ops:
        op.close()
    return {
        "alg_bytes": alg_bytes,
        "ms_per_step": step_ms,
        "kernel_ms": kern_ms,
        "gbs": alg_bytes / (step_ms * 1e-3) / 1e9,
        "kernel_gbs": alg_bytes / (kern_ms * 1e-3) / 1e9,
        "passes": _last_passes,
    }


def _board_sensors():
    """hwmon files of every card the kernel driver shows: power (uW), power cap (uW), engine clock (Hz)."""
    import glob

    cards = []
    for dev in sorted(glob.glob("/sys/class/drm/card*/device")):
        for hw in glob.glob(os.path.join(dev, "hwmon", "hwmon*")):
            f = {}
            for key, names in (("power", ("power1_input", "power1_average")), ("cap", ("power1_cap",)),
                               ("sclk", ("freq1_input",))):
                for n in names:
                    if os.path.exists(os.path.join(hw, n)):
                        f[key] = os.path.join(hw, n)
                        break
            if "sclk" not in f and os.path.exists(os.path.join(dev, "pp_dpm_sclk")):
                f["dpm_sclk"] = os.path.join(dev, "pp_dpm_sclk")   # lines "n: <MHz>Mhz", the current one starred
            if "power" in f:
                cards.append(f)
    return cards


def board_power_during(run_pass, seconds=1.0, period=0.02):
    """Board power and engine clock, read from the driver's hwmon files every `period` seconds on a
    second thread while run_pass() (a batch of launches ending in a synchronisation) is repeated for
    `seconds`.  Not part of any timed region.  With several cards visible the one that draws most is
    taken.  None where the files are missing or unreadable."""
    import statistics
    import threading

    cards = _board_sensors()
    if not cards:
        return None

    def read(path):
        try:
            return float(open(path).read().strip())
        except (OSError, ValueError):
            return None

    def read_clock(c):
        if "sclk" in c:
            return read(c["sclk"])
        if "dpm_sclk" in c:
            try:
                for line in open(c["dpm_sclk"]).read().splitlines():
                    if "*" in line:
                        return float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip()) * 1e6
            except (OSError, ValueError, IndexError):
                pass
        return None

    rows, stop = [], threading.Event()

    def poll():
        while not stop.is_set():
            rows.append([(read(c["power"]), read_clock(c)) for c in cards])
            stop.wait(period)

    th = threading.Thread(target=poll, daemon=True)
    th.start()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        run_pass()
    stop.set()
    th.join()
    rows = rows[len(rows) // 4:]      # the first quarter: clocks and the sensor's average still moving
    best = None
    for i, c in enumerate(cards):
        watts = [r[i][0] / 1e6 for r in rows if r[i][0] is not None]
        if not watts:
            continue
        mhz = [r[i][1] / 1e6 for r in rows if r[i][1] is not None]
        cap = read(c["cap"]) if "cap" in c else None
        entry = {"watts": round(statistics.mean(watts), 1), "watts_max": round(max(watts), 1),
                 "cap_watts": round(cap / 1e6, 1) if cap else None,
                 "engine_mhz": round(statistics.mean(mhz), 0) if mhz else None, "samples": len(watts)}
        if best is None or entry["watts"] > best["watts"]:
            best = entry
    return best


def bench_prefill(seq, steps, warmup, hq=32, hkv=4, dtype_name="f16", p0=0, zero_kv=False, batch=1, copies=1,
                  power_seconds=0.0):
    import torch

    import ellm_amd

    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    cap = p0 + seq
    scale = 1.0 / D ** 0.5
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    qs = torch.rand((1, 1, hq, 1), generator=g, device="cuda") * 1.5 + 0.5   # per-head scale U[0.5, 2]
    ks = torch.rand((1, hkv, 1, 1), generator=g, device="cuda") * 1.5 + 0.5
    vs = torch.rand((1, hkv, 1, 1), generator=g, device="cuda") * 1.5 + 0.5
    ops = []
    for c in range(copies):     # several cache sets in rotation where a step should find nothing cached
        q = (_dev_normal((seq, batch, hq, D), torch.float32, 11 + 10 * c) * qs).to(dt)
        k = (_dev_normal((batch, hkv, cap, D), torch.float32, 12 + 10 * c) * ks).to(dt)
        v = (_dev_normal((batch, hkv, cap, D), torch.float32, 13 + 10 * c) * vs).to(dt)
        if zero_kv:  # diagnostic: same instruction stream, operands that toggle nothing
            k.zero_()
            v.zero_()
        out = torch.zeros_like(q)
        lse = torch.zeros((seq, batch, hq), dtype=torch.float32, device="cuda")
        ops.append((ellm_amd.Attention(q, k, v, out, batch, hq, hkv, D, [hkv * cap * D, cap * D, D, 1], scale,
                                       lse=lse, sequence_capacity=cap, max_position_interval=seq), q, k, v, out, lse))
    per, step_ms = _time_steps(lambda i: ops[i % copies][0].run(p0, seq, batch), steps, warmup)
    flops = batch * 4 * D * hq * (seq * p0 + seq * (seq + 1) // 2)
    kern_ms = sum(per) / len(per)
    passes = _last_passes
    power = None
    if power_seconds > 0:       # after the timed passes, not inside them
        def run_pass():
            for i in range(8):
                ops[i % copies][0].run(p0, seq, batch)
            torch.cuda.synchronize()
        power = board_power_during(run_pass, power_seconds)
    for op in ops:
        op[0].close()
    return {
        "flops": flops,
        "ms_per_step": step_ms,
        "kernel_ms": kern_ms,
        "tflops": flops / (step_ms * 1e-3) / 1e12,
        "kernel_tflops": flops / (kern_ms * 1e-3) / 1e12,
        "passes": passes,
        "power": power,
    }


def bench_ragged_decode(batch, lo, hi, steps, warmup, hq=32, hkv=4, seed=7):
    """One single-token step over `batch` sequences whose cache lengths are drawn
    uniformly from [lo, hi] (per-sequence positions on the device)."""
    import numpy as np
    import torch

    import ellm_amd

    rng = np.random.default_rng(seed)
    lengths = rng.integers(lo, hi + 1, size=batch)
    cap = int(hi)
    scale = 1.0 / D ** 0.5
    k = torch.empty((batch, hkv, cap, D), dtype=torch.float16, device="cuda").normal_()
    v = torch.empty((batch, hkv, cap, D), dtype=torch.float16, device="cuda").normal_()
    q = _dev_normal((1, batch, hq, D), torch.float16, 301)
    out = torch.zeros_like(q)
    pos = torch.tensor((lengths - 1).astype(np.int32), dtype=torch.int32, device="cuda")
    op = ellm_amd.Attention(q, k, v, out, batch, hq, hkv, D, [hkv * cap * D, cap * D, D, 1], scale,
                            sequence_capacity=cap, max_position_interval=1)
    max_pos = int(lengths.max() - 1)
    per, step_ms = _time_steps(lambda i: op.run_ragged(pos, max_pos, batch), steps, warmup)
    alg_bytes = int(2 * hkv * D * 2 * lengths.sum() + 2 * batch * hq * D * 2)
    kern_ms = sum(per) / len(per)
    op.close()
    return {
        "alg_bytes": alg_bytes,
        "ms_per_step": step_ms,
        "kernel_ms": kern_ms,
        "gbs": alg_bytes / (step_ms * 1e-3) / 1e9,
        "kernel_gbs": alg_bytes / (kern_ms * 1e-3) / 1e9,
        "tokens": int(lengths.sum()),
    }


def bench_kv_write(n_tokens, steps, warmup, hkv=4, seqs=1):
    """Key rows RMS-normalised and rotated, value rows copied, both written to their
    token coordinates of the cache (the step before attention in a layer)."""
    import torch

    import ellm_amd

    cap = n_tokens
    copies = 6   # sources and cache layers rotate (6 x 128 MiB) so that no step finds its rows cached
    cache = ellm_amd.KVCache(copies, seqs, hkv, cap, ellm_amd.DTYPE_F16)
    ks = [_dev_normal((n_tokens, seqs, hkv, D), torch.float16, 21 + c) for c in range(copies)]
    vs = [_dev_normal((n_tokens, seqs, hkv, D), torch.float16, 41 + c) for c in range(copies)]
    j = torch.arange(D // 2, device="cuda", dtype=torch.float64)
    ang = torch.arange(cap, device="cuda", dtype=torch.float64)[:, None] * (1.0e6 ** (-2.0 * j / D))[None, :]
    rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).reshape(cap, D).to(torch.float16)
    per, step_ms = _time_steps(
        lambda i: cache.append_norm_rope(i % copies, 0, ks[i % copies], vs[i % copies], rope),
        steps, warmup)
    rows = n_tokens * seqs * hkv
    alg_bytes = rows * D * 2 * 4 + cap * D * 2          # K, V read and written; the table read once
    kern_ms = sum(per) / len(per)
    # yardsticks on the same buffers: the library's plain write (ellm_kv_append: the same rows copied,
    # nothing computed) and the runtime's own device-to-device copy of the same bytes
    per_plain, _ = _time_steps(lambda i: cache.append(i % copies, 0, ks[i % copies], vs[i % copies]), steps, warmup)
    dst = [torch.empty((2,) + tuple(ks[0].shape), dtype=torch.float16, device="cuda") for _ in range(copies)]
    src = [torch.stack((ks[c], vs[c])) for c in range(copies)]
    per_copy, _ = _time_steps(lambda i: dst[i % copies].copy_(src[i % copies]), steps, warmup)
    copy_bytes = rows * D * 2 * 4
    cache.close()
    return {"alg_bytes": alg_bytes, "ms_per_step": step_ms, "kernel_ms": kern_ms,
            "gbs": alg_bytes / (step_ms * 1e-3) / 1e9,
            "kernel_gbs": alg_bytes / (kern_ms * 1e-3) / 1e9,
            "plain_append_gbs": copy_bytes / (sum(per_plain) / len(per_plain) * 1e-3) / 1e9,
            "device_copy_gbs": copy_bytes / (sum(per_copy) / len(per_copy) * 1e-3) / 1e9}


def bench_mixed_step(layers, prefill_tokens, batch, lo, hi, steps, warmup, hidden=2048, hq=32, hkv=4, seed=7):
    """One step of the mixed configuration end to end: for each layer the fused Q/K/V projection
    (random-init weights of the layer, norm + rotation, K/V written into the cache) and the
    attention of a `prefill_tokens`-token prefill of one sequence, and the same two for one new
    token of `batch` other sequences with cache lengths U{lo..hi}; all launches on one stream,
    issued one by one and replayed from one recorded graph.
    Every layer has its own weights and its own K/V: one cache object of `layers` layers whose
    1 + batch sequences have their own capacities (the prefill's length, and each drawn length
    rounded up to 64), so the resident set is what the sequences need (~223 GB for 48 layers)
    rather than 33 x 131072 positions a layer.  Activations (hidden rows, Q, attention output)
    are layer-shared scratch, as in the reference (src/memory/cache.rs:76-91)."""
    import numpy as np
    import torch

    import ellm_amd

    dt = torch.float16
    rng = np.random.default_rng(seed)
    lengths = rng.integers(lo, hi + 1, size=batch)
    caps = [prefill_tokens] + [int((n + 63) // 64 * 64) for n in lengths]
    scale = 1.0 / D ** 0.5
    torch.cuda.empty_cache()     # the cache below is allocated by the library, not by torch
    cache = ellm_amd.KVCache.ragged(layers, caps, hkv, ellm_amd.DTYPE_F16)
    cap = max(caps)
    j = torch.arange(D // 2, device="cuda", dtype=torch.float64)
    ang = torch.arange(cap, device="cuda", dtype=torch.float64)[:, None] * (1.0e6 ** (-2.0 * j / D))[None, :]
    rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).reshape(cap, D).to(dt)
    del ang
    x_dec = _dev_normal((1, batch, hidden), dt, 300)
    q = torch.zeros((1, batch, hq, D), dtype=dt, device="cuda")
    out = torch.zeros_like(q)
    pos = torch.tensor((lengths - 1).astype(np.int32), dtype=torch.int32, device="cuda")
    max_pos = int(lengths.max() - 1)
    x_pre = _dev_normal((prefill_tokens, 1, hidden), dt, 310)
    pq = torch.zeros((prefill_tokens, 1, hq, D), dtype=dt, device="cuda")
    pout = torch.zeros_like(pq)
    ops, keep = [], []
    for layer in range(layers):
        kt, vt = cache.layer_flat_tensors(layer, dt)
        kt.normal_()             # the sequences' caches already hold their tokens
        vt.normal_()
        v0, v1 = cache.layer_ragged(layer, 0), cache.layer_ragged(layer, 1)
        w = [_dev_normal((h * D, hidden), dt, 700 + 3 * layer + i, scale=hidden ** -0.5) for i, h in enumerate((hq, hkv, hkv))]
        keep.append((w, kt, vt))
        ops.append((ellm_amd.MatMul3(x_pre, w[0], pq, w[1], kt, w[2], vt, rope, D, 1, hq, hkv, v0.strides, 0,
                                     seq_table=v0),
                    ellm_amd.Attention(pq, kt, vt, pout, 1, hq, hkv, D, v0.strides, scale,
                                       max_position_interval=prefill_tokens, seq_table=v0),
                    ellm_amd.MatMul3(x_dec, w[0], q, w[1], kt, w[2], vt, rope, D, batch, hq, hkv, v1.strides, 0,
                                     seq_table=v1),
                    ellm_amd.Attention(q, kt, vt, out, batch, hq, hkv, D, v1.strides, scale,
                                       max_position_interval=1, seq_table=v1)))

    def step(_=None):
        for qkv_pre, att_pre, qkv_dec, att_dec in ops:
            qkv_pre.run(0, prefill_tokens, 1)
            att_pre.run(0, prefill_tokens, 1)
            qkv_dec.run_ragged(pos, max_pos, batch)
            att_dec.run_ragged(pos, max_pos, batch)

    stream = torch.cuda.Stream()
    side = ellm_amd.SideStream()

    def step_side_by_side():
        # the two halves of a layer share nothing: the single-token half on the library's side
        # stream, joined before the next layer
        for qkv_pre, att_pre, qkv_dec, att_dec in ops:
            side.fork(stream)
            qkv_dec.run_ragged(pos, max_pos, batch, stream=side)
            att_dec.run_ragged(pos, max_pos, batch, stream=side)
            qkv_pre.run(0, prefill_tokens, 1, stream=stream)
            att_pre.run(0, prefill_tokens, 1, stream=stream)
            side.join(stream)

    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        _, eager_ms = _time_steps(step, steps, warmup)
        with ellm_amd.StepGraph(stream) as graph:
            step()
        _, graph_ms = _time_steps(lambda _i: graph.launch(), steps, warmup)
        graph.close()
        with ellm_amd.StepGraph(stream) as graph:
            step_side_by_side()
        _, side_ms = _time_steps(lambda _i: graph.launch(), steps, warmup)
    graph.close()
    side.close()
    flops = layers * 4 * D * hq * (prefill_tokens * (prefill_tokens + 1) // 2)
    proj_flops = layers * 2 * (prefill_tokens + batch) * hidden * (hq + 2 * hkv) * D
    nbytes = layers * int(2 * hkv * D * 2 * lengths.sum() + 2 * batch * hq * D * 2)
    for group in ops:
        for op in group:
            op.close()
    resident = 2 * layers * hkv * sum(caps) * D * 2
    del keep
    cache.close()
    return {"eager_ms": eager_ms, "graph_ms": graph_ms, "side_by_side_ms": side_ms, "flops": flops, "proj_flops": proj_flops,
            "bytes": nbytes, "tokens": int(lengths.sum()), "resident_bytes": resident}


def bench_token_step(layers, batch, length, steps, warmup, hq=32, hkv=4):
    """One single-token step of a whole model's attention: per layer the fused cache write of
    the new key / value rows (key RMS norm + rotation) and the attention over the cache, the
    per-sequence positions advanced on the device at the end; launched eagerly (2 launches a
    layer + 1) and replayed from a graph recorded once through the library."""
    import torch

    import ellm_amd

    cap = length + 2 * (steps + warmup) + 8
    scale = 1.0 / D ** 0.5
    stream = torch.cuda.Stream()
    cache = ellm_amd.KVCache(layers, batch, hkv, cap, ellm_amd.DTYPE_F16)
    j = torch.arange(D // 2, device="cuda", dtype=torch.float64)
    ang = torch.arange(cap, device="cuda", dtype=torch.float64)[:, None] * (1.0e6 ** (-2.0 * j / D))[None, :]
    rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).reshape(cap, D).to(torch.float16)
    q = _dev_normal((1, batch, hq, D), torch.float16, 401)
    k1 = _dev_normal((1, batch, hkv, D), torch.float16, 402)
    v1 = _dev_normal((1, batch, hkv, D), torch.float16, 403)
    out = torch.zeros_like(q)
    ops = []
    for layer in range(layers):
        kt, vt = cache.layer_tensors(layer, torch.float16)
        kt.normal_()
        vt.normal_()
        _, _, strides = cache.layer(layer)
        ops.append(ellm_amd.Attention(q, kt, vt, out, batch, hq, hkv, D, strides, scale,
                                      sequence_capacity=cap, max_position_interval=1))
    pos = torch.full((batch,), length - 1, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()

    def step(_=None):
        for layer in range(layers):
            cache.append_norm_rope(layer, 0, k1, v1, rope, positions=pos, max_position=cap - 1)
            ops[layer].run_ragged(pos, cap - 1, batch)
        ellm_amd.positions_advance(pos, 1)

    def fused_step(_=None):     # the write inside the attention launch (ellm_kv_append_attn_run_ragged)
        for layer in range(layers):
            cache.append_norm_rope_with_attention(layer, ops[layer], 0, k1, v1, rope, positions=pos, max_position=cap - 1)
        ellm_amd.positions_advance(pos, 1)

    with torch.cuda.stream(stream):
        _, eager_ms = _time_steps(step, steps, warmup)
        pos.fill_(length - 1)
        stream.synchronize()
        with ellm_amd.StepGraph(stream) as graph:
            step()
        _, graph_ms = _time_steps(lambda _i: graph.launch(), steps, warmup)
        pos.fill_(length - 1)
        stream.synchronize()
        with ellm_amd.StepGraph(stream) as fused_graph:
            fused_step()
        _, fused_ms = _time_steps(lambda _i: fused_graph.launch(), steps, warmup)
    graph.close()
    fused_graph.close()
    for op in ops:
        op.close()
    cache.close()
    nbytes = layers * (2 * batch * hkv * length * D * 2 + 2 * batch * hq * D * 2)
    return {"eager_ms": eager_ms, "graph_ms": graph_ms, "fused_ms": fused_ms, "bytes": nbytes}


def bench_qkv_projection(tokens, steps, warmup, hidden=2048, hq=32, hkv=4, dtype_name="f16", batch=1):
    """Fused Q/K/V projection of `tokens` token rows (x `batch` sequences): C = X . [Wq; Wk; Wv]^T
    with RMS norm + rotary rotation of the query and key heads, query rows to the Q scratch,
    key / value rows to their token coordinates of the cache."""
    import torch

    import ellm_amd

    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    cap = tokens
    x = _dev_normal((tokens, batch, hidden), dt, 71)
    wq = _dev_normal((hq * D, hidden), dt, 72, scale=hidden ** -0.5)
    wk = _dev_normal((hkv * D, hidden), dt, 73, scale=hidden ** -0.5)
    wv = _dev_normal((hkv * D, hidden), dt, 74, scale=hidden ** -0.5)
    j = torch.arange(D // 2, device="cuda", dtype=torch.float64)
    ang = torch.arange(cap, device="cuda", dtype=torch.float64)[:, None] * (1.0e6 ** (-2.0 * j / D))[None, :]
    rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).reshape(cap, D).to(dt)
    q = torch.zeros((tokens, batch, hq, D), dtype=dt, device="cuda")
    cache = ellm_amd.KVCache(1, batch, hkv, cap,
                             ellm_amd.DTYPE_F16 if dtype_name == "f16" else ellm_amd.DTYPE_BF16)
    kt, vt = cache.layer_tensors(0, dt)
    _, _, strides = cache.layer(0)
    op = ellm_amd.MatMul3(x, wq, q, wk, kt, wv, vt, rope, D, batch, hq, hkv, strides, cap)
    per, step_ms = _time_steps(lambda i: op.run(0, tokens, batch), steps, warmup)
    flops = 2 * tokens * batch * hidden * (hq + 2 * hkv) * D
    kern_ms = sum(per) / len(per)
    op.close()
    cache.close()
    return {"flops": flops, "ms_per_step": step_ms, "kernel_ms": kern_ms,
            "tflops": flops / (step_ms * 1e-3) / 1e12, "kernel_tflops": flops / (kern_ms * 1e-3) / 1e12}


def bench_output_projection(tokens, steps, warmup, hidden=2048, hq=32, dtype_name="f16"):
    """Output projection with residual: Y = R + A . Wo^T, A = the attention output rows."""
    import torch

    import ellm_amd

    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    a = _dev_normal((tokens, 1, hq * D), dt, 81)
    w = _dev_normal((hidden, hq * D), dt, 82, scale=(hq * D) ** -0.5)
    r = _dev_normal((tokens, 1, hidden), dt, 83)
    out = torch.zeros_like(r)
    op = ellm_amd.MatMulAdd(a, w, r, out)
    per, step_ms = _time_steps(lambda i: op.run(0, tokens, 1), steps, warmup)
    flops = 2 * tokens * hidden * hq * D
    kern_ms = sum(per) / len(per)
    op.close()
    return {"flops": flops, "ms_per_step": step_ms, "kernel_ms": kern_ms,
            "tflops": flops / (step_ms * 1e-3) / 1e12, "kernel_tflops": flops / (kern_ms * 1e-3) / 1e12}


def bench_step_projections(batch, steps, warmup, hidden=2048, hq=32, hkv=4, copies=8):
    """The two projections of a single-token step (one token row per sequence): fused Q/K/V
    and output + residual.  The weights rotate over `copies` sets (8 x 21 MB and 8 x 17 MB)
    so that a step streams them from HBM, as a model with many layers does."""
    import torch

    import ellm_amd

    dt = torch.float16
    cap = 1024
    x = _dev_normal((1, batch, hidden), dt, 91)
    j = torch.arange(D // 2, device="cuda", dtype=torch.float64)
    ang = torch.arange(cap, device="cuda", dtype=torch.float64)[:, None] * (1.0e6 ** (-2.0 * j / D))[None, :]
    rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).reshape(cap, D).to(dt)
    q = torch.zeros((1, batch, hq, D), dtype=dt, device="cuda")
    cache = ellm_amd.KVCache(1, batch, hkv, cap, ellm_amd.DTYPE_F16)
    kt, vt = cache.layer_tensors(0, dt)
    _, _, strides = cache.layer(0)
    qkv, keep = [], []
    for c in range(copies):
        w = [_dev_normal((h * D, hidden), dt, 100 + 3 * c + i, scale=hidden ** -0.5) for i, h in enumerate((hq, hkv, hkv))]
        keep.append(w)
        qkv.append(ellm_amd.MatMul3(x, w[0], q, w[1], kt, w[2], vt, rope, D, batch, hq, hkv, strides, cap))
    per, qkv_ms = _time_steps(lambda i: qkv[i % copies].run(7, 1, batch), steps, warmup)
    qkv_kernel_ms = per[0]
    a = _dev_normal((1, batch, hq * D), dt, 92)
    r = _dev_normal((1, batch, hidden), dt, 93)
    out = torch.zeros_like(r)
    oproj = []
    for c in range(copies):
        w = _dev_normal((hidden, hq * D), dt, 200 + c, scale=(hq * D) ** -0.5)
        keep.append(w)
        oproj.append(ellm_amd.MatMulAdd(a, w, r, out))
    per, o_ms = _time_steps(lambda i: oproj[i % copies].run(7, 1, batch), steps, warmup)
    for op in qkv + oproj:
        op.close()
    cache.close()
    qkv_bytes = (hq + 2 * hkv) * D * hidden * 2 + batch * hidden * 2 + batch * (hq + 2 * hkv) * D * 2
    o_bytes = hidden * hq * D * 2 + batch * hq * D * 2 + 2 * batch * hidden * 2
    return {"qkv_ms": qkv_ms, "qkv_kernel_ms": qkv_kernel_ms, "qkv_bytes": qkv_bytes,
            "o_ms": o_ms, "o_kernel_ms": per[0], "o_bytes": o_bytes}


def bench_layer_steps(layers, cases, steps, warmup, hidden=2048, hq=32, hkv=4):
    """The attention block of every layer for one new token per sequence: fused Q/K/V projection
    (norm + rotation, K/V written into the cache), attention over the cache, output projection +
    residual; every layer has its own weights and cache; positions advance on the device.
    Issued launch by launch and replayed from a graph recorded once through the library.
    cases: (sequences, cached tokens) pairs; the layers' weights are made once and shared by the
    cases, every case has its own caches."""
    import torch

    import ellm_amd

    dt = torch.float16
    scale = 1.0 / D ** 0.5
    stream = torch.cuda.Stream()
    keep = []
    for layer in range(layers):
        w = [_dev_normal((h * D, hidden), dt, 600 + 4 * layer + i, scale=hidden ** -0.5) for i, h in enumerate((hq, hkv, hkv))]
        wo = _dev_normal((hidden, hq * D), dt, 603 + 4 * layer, scale=(hq * D) ** -0.5)
        keep.append((w, wo))
    results = {}
    for batch, length in cases:
        n_steps = min(steps, 20)
        cap = length + 512     # positions advance once per step; the kernels clamp them to cap - 1
        cache = ellm_amd.KVCache(layers, batch, hkv, cap, ellm_amd.DTYPE_F16)
        j = torch.arange(D // 2, device="cuda", dtype=torch.float64)
        ang = torch.arange(cap, device="cuda", dtype=torch.float64)[:, None] * (1.0e6 ** (-2.0 * j / D))[None, :]
        rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).reshape(cap, D).to(dt)
        x = [_dev_normal((1, batch, hidden), dt, 501), torch.zeros((1, batch, hidden), dtype=dt, device="cuda")]
        q = torch.zeros((1, batch, hq, D), dtype=dt, device="cuda")
        att = torch.zeros_like(q)
        ops = []
        for layer in range(layers):
            kt, vt = cache.layer_tensors(layer, dt)
            kt.normal_()
            vt.normal_()
            _, _, strides = cache.layer(layer)
            w, wo = keep[layer]
            src, dst = x[layer & 1], x[1 - (layer & 1)]
            ops.append((ellm_amd.MatMul3(src, w[0], q, w[1], kt, w[2], vt, rope, D, batch, hq, hkv, strides, cap),
                        ellm_amd.Attention(q, kt, vt, att, batch, hq, hkv, D, strides, scale,
                                           sequence_capacity=cap, max_position_interval=1),
                        ellm_amd.MatMulAdd(att.view(1, batch, hq * D), wo, src, dst)))
        pos = torch.full((batch,), length - 1, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()

        def step(_=None):
            for qkv, attn, oproj in ops:
                qkv.run_ragged(pos, cap - 1, batch)
                attn.run_ragged(pos, cap - 1, batch)
                oproj.run(0, 1, batch)
            ellm_amd.positions_advance(pos, 1)

        # short steps: fewer timed passes, so that the positions stay near `length`
        min_ms = MIN_TIMED_MS if length >= 4096 else 30.0
        with torch.cuda.stream(stream):
            _, eager_ms = _time_steps(step, n_steps, warmup, min_ms=min_ms)
            pos.fill_(length - 1)
            stream.synchronize()
            with ellm_amd.StepGraph(stream) as graph:
                step()
            dev, graph_ms = _time_steps(lambda _i: graph.launch(), n_steps, warmup, min_ms=min_ms)
            graph.close()
            # the same step with the projection and the attention of a layer as one fused call
            # (the attention launch finishes the head rows the projection leaves raw)
            pos.fill_(length - 1)
            stream.synchronize()

            def fused_step(_=None):
                for qkv, attn, oproj in ops:
                    qkv.run_with_attention(attn, cap - 1, batch, positions=pos)
                    oproj.run(0, 1, batch)
                ellm_amd.positions_advance(pos, 1)

            with ellm_amd.StepGraph(stream) as graph:
                fused_step()
            fdev, fused_ms = _time_steps(lambda _i: graph.launch(), n_steps, warmup, min_ms=min_ms)
        graph.close()
        for group in ops:
            for op in group:
                op.close()
        cache.close()
        del rope, ang
        kv_bytes = layers * (2 * batch * hkv * length * D * 2)
        w_bytes = layers * ((hq + 2 * hkv) * D * hidden * 2 + hidden * hq * D * 2)
        results[(batch, length)] = {"eager_ms": eager_ms, "graph_ms": graph_ms, "graph_dev_ms": dev[0],
                                    "fused_ms": fused_ms, "fused_dev_ms": fdev[0],
                                    "kv_bytes": kv_bytes, "w_bytes": w_bytes, "steps": n_steps}
    return results


def cpu_baseline_layer_step(batch, length, layers=48, hidden=2048, hq=32, hkv=4):
    """One layer's attention block of a single-token step on the CPU oracle (fused Q/K/V projection,
    attention over the cache, output projection + residual: the oracle's scalar restatements, one
    thread), times the layer count."""
    import numpy as np
    import oracle_lib as orc

    cap = length
    x = _cpu_normal((1, batch, hidden), "f16", 31)
    w = [_cpu_normal((h * D, hidden), "f16", 32 + i) for i, h in enumerate((hq, hkv, hkv))]
    wo = _cpu_normal((hidden, hq * D), "f16", 36)
    k = _cpu_normal((batch, hkv, cap, D), "f16", 37)
    v = _cpu_normal((batch, hkv, cap, D), "f16", 38)
    ang = np.arange(cap)[:, None] * (1.0e6 ** (-2.0 * np.arange(D // 2) / D))[None, :]
    rope32 = np.empty((cap, D), dtype=np.float32)
    rope32[:, 0::2], rope32[:, 1::2] = np.cos(ang), np.sin(ang)
    rope = orc.to_storage(rope32, orc.F16)
    q = np.zeros((1, batch, hq, D), dtype=np.float16)
    strides = [hkv * cap * D, cap * D, D, 1]
    t0 = time.perf_counter()
    assert orc.matmul3(x, w[0], w[1], w[2], q, k, v, rope, strides, cap, length - 1, 1, orc.F16) == 0
    att, _ = orc.attention(q, k, v, 1.0 / D ** 0.5, orc.F16, position_index=length - 1, n_threads=1)
    orc.matmul_add(att.reshape(1, batch, hq * D), wo, x, orc.F16)
    t = time.perf_counter() - t0
    return {"value": round(t * layers * 1e3, 2), "unit": "ms", "cores": 1, "kind": "port",
            "sample": f"one layer of {layers} on one thread ({t * 1e3:.1f} ms), x {layers}"}


def bench_chunk_block(positions, batch, p0, steps, warmup, hidden=2048, hq=32, hkv=4):
    """The attention block of one layer for a prompt chunk of `positions` tokens x `batch` sequences
    on caches that already hold `p0` tokens: fused Q/K/V projection (K/V written into the cache at
    p0..), chunk attention over 0..p0 + positions, output projection + residual."""
    import torch

    import ellm_amd

    dt = torch.float16
    cap = p0 + positions
    scale = 1.0 / D ** 0.5
    cache = ellm_amd.KVCache(1, batch, hkv, cap, ellm_amd.DTYPE_F16)
    kt, vt = cache.layer_tensors(0, dt)
    kt.normal_()
    vt.normal_()
    _, _, strides = cache.layer(0)
    j = torch.arange(D // 2, device="cuda", dtype=torch.float64)
    ang = torch.arange(cap, device="cuda", dtype=torch.float64)[:, None] * (1.0e6 ** (-2.0 * j / D))[None, :]
    rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).reshape(cap, D).to(dt)
    x = _dev_normal((positions, batch, hidden), dt, 701)
    y = torch.zeros_like(x)
    q = torch.zeros((positions, batch, hq, D), dtype=dt, device="cuda")
    att = torch.zeros_like(q)
    w = [_dev_normal((h * D, hidden), dt, 702 + i, scale=hidden ** -0.5) for i, h in enumerate((hq, hkv, hkv))]
    wo = _dev_normal((hidden, hq * D), dt, 705, scale=(hq * D) ** -0.5)
    qkv = ellm_amd.MatMul3(x, w[0], q, w[1], kt, w[2], vt, rope, D, batch, hq, hkv, strides, cap)
    attn = ellm_amd.Attention(q, kt, vt, att, batch, hq, hkv, D, strides, scale, sequence_capacity=cap,
                              max_position_interval=positions)
    oproj = ellm_amd.MatMulAdd(att.view(positions, batch, hq * D), wo, x, y)
    parts = {}
    for name, fn in (("qkv", lambda i: qkv.run(p0, positions, batch)),
                     ("attention", lambda i: attn.run(p0, positions, batch)),
                     ("output", lambda i: oproj.run(p0, positions, batch))):
        per, _ = _time_steps(fn, steps, warmup)
        parts[name] = sum(per) / len(per)

    def block(_i):
        qkv.run(p0, positions, batch)
        attn.run(p0, positions, batch)
        oproj.run(p0, positions, batch)

    _, block_ms = _time_steps(block, steps, warmup)
    for op in (qkv, attn, oproj):
        op.close()
    cache.close()
    rows = positions * batch
    flops = (2 * rows * hidden * (hq + 2 * hkv) * D + 2 * rows * hidden * hq * D
             + 4 * D * hq * batch * (positions * p0 + positions * (positions + 1) / 2))
    return {"block_ms": block_ms, "parts_ms": parts, "flops": flops}


def _host_info():
    """CPU model, logical cores of the machine, and the threads the CPU baselines use: one per
    core this process may run on, at most the CPU share the environment states
    (OMP_NUM_THREADS, which a shared GPU box sets to its per-GPU share of the host)."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = os.cpu_count() or 1
    share = os.environ.get("OMP_NUM_THREADS", "")
    cores = min(allowed, int(share)) if share.isdigit() and int(share) > 0 else allowed
    return {"cpu_model": model, "host_cores": os.cpu_count() or 1, "cores": max(1, cores)}


def _cpu_normal(shape, dtype_name, seed):
    """N(0,1) on the host in the storage type, as a numpy array of bit patterns."""
    import numpy as np
    import torch

    g = torch.Generator()
    g.manual_seed(seed)
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    x = torch.randn(shape, generator=g, dtype=torch.float32).to(dt)
    a = x.view(torch.int16).numpy()
    return a.view(np.float16) if dtype_name == "f16" else a.view(np.uint16)


def cpu_baseline_decode(batch, length, hq=32, hkv=4, budget_s=1.5):
    """The CPU oracle on the full single-token workload, repeated for about `budget_s` seconds
    of wall time (x the threads: 20-odd core-seconds of CPU work); one pinned thread per core
    with the reference's static split and barrier (src/serving/start.rs:43-77)."""
    import oracle_lib as orc

    host = _host_info()
    cores = host["cores"]
    q = _cpu_normal((1, batch, hq, D), "f16", 1)
    k = _cpu_normal((batch, hkv, length, D), "f16", 2)
    v = _cpu_normal((batch, hkv, length, D), "f16", 3)
    import numpy as np
    out = np.zeros_like(q)
    op = orc.Operator(q, k, v, out, None, batch, hq, hkv, D, [hkv * length * D, length * D, D, 1],
                      1.0 / D ** 0.5, orc.F16)
    t1 = op.run_threads(length - 1, 1, batch, cores, pin=True)
    repeats = max(1, min(200, int(budget_s / max(t1, 1e-3))))
    t = op.run_threads(length - 1, 1, batch, cores, pin=True, repeats=repeats) / repeats
    alg_bytes = 2 * batch * hkv * length * D * 2 + 2 * batch * hq * D * 2
    return {
        "value": alg_bytes / t / 1e9,
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "pinned": True,
        "sample": f"full workload, {repeats} passes, {t * 1e3:.1f} ms per pass, one pinned thread per core",
    }


def _cpu_sampled_rows(op, position_index, pick_rows, row_macs, cores, budget_s, positions=None):
    """Times the oracle on a seeded sample of (token, sequence, head) rows sized for about
    `budget_s` seconds of wall time: a pilot of 2 rows per thread gives the rate, then the
    sample.  pick_rows(n) -> uint32 [n, 3]; row_macs(rows) -> multiply-adds of those rows.
    Returns (seconds, multiply-adds of the sample, rows)."""
    pilot = pick_rows(2 * cores)
    _, _, t0 = op.run_rows(position_index, pilot, cores, positions=positions, pin=True)
    rate = row_macs(pilot) / max(t0, 1e-4)
    n = int(min(200000, max(4 * cores, rate * budget_s / (row_macs(pilot) / len(pilot)))))
    rows = pick_rows(n)
    _, _, t = op.run_rows(position_index, rows, cores, positions=positions, pin=True)
    return t, row_macs(rows), len(rows)


def cpu_baseline_chunk(seq, p0, hq, hkv, dtype_name, budget_s=1.5, seed=17):
    """The CPU oracle on a seeded subset of the (token, head) rows of a causal chunk of `seq`
    tokens on a cache that already holds `p0`, extrapolated to the whole chunk by the count of
    multiply-adds (a row at position p costs 2 x 128 x (p + 1) of them); the full chunk is
    10^12 to 10^13 multiply-adds, hours of CPU time."""
    import numpy as np
    import oracle_lib as orc

    host = _host_info()
    cores = host["cores"]
    cap = p0 + seq
    code = orc.F16 if dtype_name == "f16" else orc.BF16
    k = _cpu_normal((1, hkv, cap, D), dtype_name, seed)
    v = _cpu_normal((1, hkv, cap, D), dtype_name, seed + 1)
    q = np.zeros((seq, 1, hq, D), dtype=k.dtype)       # untouched pages cost nothing
    out = np.zeros((1, 1, hq, D), dtype=k.dtype)       # run_rows returns its own rows
    op = orc.Operator(q, k, v, out, None, 1, hq, hkv, D, [hkv * cap * D, cap * D, D, 1],
                      1.0 / D ** 0.5, code)
    rng = np.random.default_rng(seed)
    qrow = _cpu_normal((D,), dtype_name, seed + 2)

    def pick_rows(n):
        rows = np.stack((rng.integers(0, seq, size=n), np.zeros(n, dtype=np.int64),
                         rng.integers(0, hq, size=n)), axis=1).astype(np.uint32)
        q[rows[:, 0], 0, rows[:, 2]] = qrow
        return rows

    def row_macs(rows):
        return float(2 * D * (p0 + rows[:, 0].astype(np.float64) + 1).sum())

    t, macs, n = _cpu_sampled_rows(op, p0, pick_rows, row_macs, cores, budget_s)
    full_macs = 2.0 * D * hq * (seq * p0 + seq * (seq + 1) / 2)
    factor = full_macs / macs
    return {
        "value": 2 * full_macs / (t * factor) / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "pinned": True,
        "sample": f"{n} seeded (token, head) rows, {macs / 1e9:.2f} of {full_macs / 1e9:.0f} G multiply-adds in "
                  f"{t:.2f} s; x {factor:.0f} by multiply-add count",
        "extrapolation_factor": factor,
        "seconds_extrapolated": t * factor,
    }


def cpu_baseline_ragged_decode(lengths, hq=32, hkv=4, sample_seqs=4, seed=19):
    """The CPU oracle on a single-token step over `sample_seqs` of the drawn sequences (all their
    query heads), extrapolated to all of them by cached-token count."""
    import numpy as np
    import oracle_lib as orc

    host = _host_info()
    cores = host["cores"]
    rng = np.random.default_rng(seed)
    chosen = np.sort(rng.choice(len(lengths), size=min(sample_seqs, len(lengths)), replace=False))
    lens = np.asarray(lengths)[chosen]
    cap = int(lens.max())
    b = len(chosen)
    k = _cpu_normal((b, hkv, cap, D), "f16", seed)
    v = _cpu_normal((b, hkv, cap, D), "f16", seed + 1)
    q = _cpu_normal((1, b, hq, D), "f16", seed + 2)
    out = np.zeros_like(q)
    op = orc.Operator(q, k, v, out, None, b, hq, hkv, D, [hkv * cap * D, cap * D, D, 1],
                      1.0 / D ** 0.5, orc.F16)
    pos = (lens - 1).astype(np.uint32)
    t = op.run_threads(0, 1, b, cores, positions=pos, pin=True)
    factor = float(np.sum(lengths)) / float(lens.sum())
    nbytes = float(2 * hkv * D * 2 * np.sum(lengths) + 2 * len(lengths) * hq * D * 2)
    return {
        "value": nbytes / (t * factor) / 1e9,
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "pinned": True,
        "sample": f"{b} of {len(lengths)} sequences, all heads, {t * 1e3:.0f} ms; x {factor:.2f} by cached-token count",
        "extrapolation_factor": factor,
        "seconds_extrapolated": t * factor,
    }


def bench_mfma_stream(mode, dtype_name, n_cu, seconds=0.6, zeros=False, per_cu=1):
    """What a pure stream of v_mfma_f32_32x32x16 sustains on N(0,1) operands on this box now
    (libellm_diag.so: one wave per SIMD, four accumulators, no global memory access in the loop;
    mode 0 register operands, mode 1 the A operand re-read from LDS for every MFMA, mode 2 the
    same plus the vector instructions of a soft-max of that tile shape in the same wave)."""
    import ctypes

    import torch

    path = os.path.join(ROOT, "ellm_amd", "lib", "libellm_diag.so")
    lib = ctypes.CDLL(path)
    fn = lib.ellm_diag_mfma_stream
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                   ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(ctypes.c_double)]
    dt = torch.float16 if dtype_name == "f16" else torch.bfloat16
    ops = _dev_normal((16, 256, 8), dt, 91)
    if zeros:   # the same instruction stream on operands that toggle nothing: what the schedule allows
        ops.zero_()
    n_wg = n_cu * per_cu     # per_cu = 2: two waves per SIMD, so one wave's vector work overlaps the other's MFMAs
    sink = torch.zeros((n_wg * 256,), dtype=torch.float32, device="cuda")
    flops = ctypes.c_double()
    iters = 4000      # 128000 MFMAs a wave: ~2.5 ms a launch
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def launch(_i):
        rc = fn(mode, 0 if dtype_name == "f16" else 1, ops.data_ptr(), sink.data_ptr(), n_wg, iters // per_cu, stream,
                ctypes.byref(flops))
        if rc:
            raise RuntimeError(f"ellm_diag_mfma_stream returned {rc}")

    # long enough for the part's power management to settle on its sustained clock
    per, _ = _time_steps(launch, 40, 40, min_ms=seconds * 1e3)
    return flops.value / (per[0] * 1e-3) / 1e12


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--only", default="", help="decode | prefill | decode128k | chunk | smallchunk | lastchunk | mixed | mixed48 | kvwrite | tokenstep | layerstep | qkv | oproj | chunkproj | chunkblock | stepproj")
    ap.add_argument("--prefill-zero-kv", action="store_true",
                    help="diagnostic for --only prefill: K and V all zero (the kernel issues the same "
                         "instructions; separates its cycle count from the clock the part sustains "
                         "under dense random operands); the line it prints is not a benchmark result")
    ap.add_argument("--layer-cases", default="",
                    help="for --only layerstep: comma-separated SEQxLEN pairs instead of the default five (profiling)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first run one plain 256 MiB device copy (a known-traffic dispatch "
                         "for scaling rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import ellm_amd

    ellm_amd.load_library()  # fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    if args.copy_calibration:
        src = torch.ones(256 * 1024 * 1024 // 4, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)      # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    also = []
    last_entries = []   # the two headline targets: appended last, where a truncated record still shows them
    targets = {}        # compact copies of the headline figures, inside the line's `roofline` object
    dec = None
    host = _host_info()
    if args.only in ("", "decode"):
        dec = bench_decode(16, 8192, args.steps, args.warmup)
        targets["decode_16x8192"] = {
            "us": round(dec["kernel_ms"] * 1e3, 2), "gbs": round(dec["kernel_gbs"], 1),
            "frac": round(dec["kernel_gbs"] / HBM_PEAK_GBS, 4), "target_frac": 0.7}
    if args.only in ("", "prefill"):
        pf_steps = max(3, min(args.steps, 10))
        pf = bench_prefill(32768, pf_steps, min(args.warmup, 2), zero_kv=args.prefill_zero_kv, power_seconds=1.0)
        # the same launch on zero K and V: same instruction stream, operands that toggle nothing
        # (not a result: it shows what the operand values cost in clock under the board's power cap)
        pf_zero = None if args.prefill_zero_kv else bench_prefill(32768, 3, 1, zero_kv=True, power_seconds=1.0)
        # the ceiling this box gives any MFMA kernel on dense random fp16 operands, timed right
        # after the kernel it is compared with
        n_cu = torch.cuda.get_device_properties(0).multi_processor_count
        stream_reg = bench_mfma_stream(0, "f16", n_cu)
        stream_lds = bench_mfma_stream(1, "f16", n_cu)
        stream_mix = bench_mfma_stream(2, "f16", n_cu, per_cu=2)
        stream_mix0 = bench_mfma_stream(2, "f16", n_cu, seconds=0.3, zeros=True, per_cu=2)
        stream_reg0 = bench_mfma_stream(0, "f16", n_cu, seconds=0.3, zeros=True)
        stream_lds0 = bench_mfma_stream(1, "f16", n_cu, seconds=0.3, zeros=True)
        pf_cpu = None if args.skip_cpu else cpu_baseline_chunk(32768, 0, 32, 4, "f16")
        last_entries.append({
            "workload": "prefill: 1 seq x 32768 tokens, 32q/4kv heads, fp16, causal (configs[2])"
                        + (" [DIAGNOSTIC: K = V = 0]" if args.prefill_zero_kv else ""),
            "metric": "prefill attn TFLOP/s", "value": round(pf["tflops"], 2), "unit": "TFLOP/s",
            "ms_per_step": round(pf["ms_per_step"], 4), "kernel_ms": round(pf["kernel_ms"], 4), "steps": pf_steps,
            "roofline": {"bound": "mfma", "achieved": round(pf["kernel_tflops"], 2),
                         "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(pf["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4),
                         "traffic": TRAFFIC_BYTES["prefill"]},
            "passes": pf["passes"],
            # board power / engine clock (hwmon, 20 ms samples, 1 s after the timed passes) for this
            # launch and for the same launch on K = V = 0
            "board_power": {
                "this_workload": pf["power"],
                "zero_kv": None if pf_zero is None else dict(pf_zero["power"] or {}, ms_per_step=round(pf_zero["ms_per_step"], 4),
                                                             tflops=round(pf_zero["tflops"], 1)),
            },
            # pure v_mfma_f32_32x32x16_f16 streams on N(0,1) operands on every compute unit, timed in
            # this run (libellm_diag.so): operands in registers / A operand from LDS / LDS-fed plus
            # the vector instructions of a soft-max of the same tile shape
            "mfma_stream_on_n01_fp16": {
                "register_operands_tflops": round(stream_reg, 1),
                "a_operand_from_lds_tflops": round(stream_lds, 1),
                "lds_fed_with_softmax_vector_mix_tflops": round(stream_mix, 1),
                "same_streams_on_zero_operands_tflops": [round(stream_reg0, 1), round(stream_lds0, 1),
                                                         round(stream_mix0, 1)],
                "kernel_frac_of_mix_stream": round(pf["kernel_tflops"] / stream_mix, 4),
                "frac_of_published_peak": round(stream_reg / MFMA_F16_PEAK_TFLOPS, 4),
                "kernel_frac_of_register_stream": round(pf["kernel_tflops"] / stream_reg, 4),
                "kernel_frac_of_lds_fed_stream": round(pf["kernel_tflops"] / stream_lds, 4),
            },
            "cpu_baseline": pf_cpu,
        })
        targets["prefill_32k"] = {
            "ms": round(pf["kernel_ms"], 4), "tflops": round(pf["kernel_tflops"], 1),
            "frac": round(pf["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4), "target_frac": 0.5,
            "mix_stream_tflops": round(stream_mix, 1), "register_stream_tflops": round(stream_reg, 1),
            "frac_of_mix_stream": round(pf["kernel_tflops"] / stream_mix, 4),
            "engine_mhz": (pf["power"] or {}).get("engine_mhz"), "watts": (pf["power"] or {}).get("watts"),
        }
    if args.only in ("", "decode128k"):
        d128 = bench_decode(1, 131072, args.steps, args.warmup)
        targets["decode_1x131072"] = {
            "us": round(d128["kernel_ms"] * 1e3, 2), "gbs": round(d128["kernel_gbs"], 1),
            "frac": round(d128["kernel_gbs"] / HBM_PEAK_GBS, 4), "target_frac": 0.7}
        last_entries.append({
            "workload": "decode: 1 seq x 131072 cached tokens, 32q/4kv heads, fp16",
            "metric": "decode attn HBM GB/s", "value": round(d128["gbs"], 1), "unit": "GB/s",
            "ms_per_step": round(d128["ms_per_step"], 5), "kernel_ms": round(d128["kernel_ms"], 5), "steps": args.steps,
            "roofline": {"bound": "hbm", "achieved": round(d128["kernel_gbs"], 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(d128["kernel_gbs"] / HBM_PEAK_GBS, 4),
                         "traffic": TRAFFIC_BYTES["decode128k"]},
            "passes": d128["passes"],
        })

        # the batch of configs[1] at the full cache length: 4.3 GB of K/V a step, far beyond
        # every cache, so one set of buffers is enough
        b128_steps = max(3, min(args.steps, 20))
        b128 = bench_decode(16, 131072, b128_steps, min(args.warmup, 3), copies=1)
        targets["decode_16x131072"] = {
            "us": round(b128["kernel_ms"] * 1e3, 1), "gbs": round(b128["kernel_gbs"], 1),
            "frac": round(b128["kernel_gbs"] / HBM_PEAK_GBS, 4)}
        also.append({
            "workload": "decode: 16 seq x 131072 cached tokens, 32q/4kv heads, fp16",
            "metric": "decode attn HBM GB/s", "value": round(b128["gbs"], 1), "unit": "GB/s",
            "ms_per_step": round(b128["ms_per_step"], 5), "steps": b128_steps,
            "roofline": {"bound": "hbm", "achieved": round(b128["kernel_gbs"], 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(b128["kernel_gbs"] / HBM_PEAK_GBS, 4),
                         "traffic": None},
        })

    if args.only in ("", "chunk"):
        ck_steps = max(3, min(args.steps, 5))
        ck = bench_prefill(8192, ck_steps, min(args.warmup, 1), hq=64, hkv=8, dtype_name="bf16",
                           p0=120000)
        ck_cpu = None if args.skip_cpu else cpu_baseline_chunk(8192, 120000, 64, 8, "bf16")
        also.append({
            "workload": "chunk: 8192 tokens on a 120000-token cache, 64q/8kv, bf16 (configs[3])",
            "metric": "prefill attn TFLOP/s", "value": round(ck["tflops"], 2), "unit": "TFLOP/s",
            "ms_per_step": round(ck["ms_per_step"], 4), "steps": ck_steps,
            "roofline": {"bound": "mfma", "achieved": round(ck["kernel_tflops"], 2),
                         "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(ck["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4),
                         "traffic": None},
            "passes": ck["passes"],
            "cpu_baseline": ck_cpu,
        })
    if args.only in ("", "smallchunk"):
        # a short chunk of one sequence on a long cache: 8 row-block workgroups, so the key range
        # is split over workgroups and merged by a second small launch
        sc = bench_prefill(64, args.steps, min(args.warmup, 5), p0=8192)
        also.append({
            "workload": "chunk: 64 tokens x 1 seq on an 8192-token cache, 32q/4kv, fp16 (keys split + merge)",
            "metric": "prefill attn TFLOP/s", "value": round(sc["tflops"], 2), "unit": "TFLOP/s",
            "ms_per_step": round(sc["ms_per_step"], 5), "steps": args.steps,
            "kv_gbs": round(2 * 4 * (8192 + 64) * D * 2 / (sc["ms_per_step"] * 1e-3) / 1e9, 1),
        })

    if args.only in ("", "lastchunk"):
        # the reference's serving loop ends a prompt with a chunk of (prompt % 64) positions x 24 sequences
        # (src/serving/start copy.rs:71-101): few query rows per K/V plane over thousands of cached tokens
        lc_dec = bench_decode(24, 8192, args.steps, min(args.warmup, 5), copies=3)
        lc = {t: bench_prefill(t, args.steps, min(args.warmup, 5), p0=8192, batch=24, copies=3) for t in (2, 8, 16, 24, 33, 48, 64)}
        kv_bytes = 2 * 24 * 4 * 8192 * D * 2
        # the same launches on K = V = 0 (same instruction stream, operands that toggle nothing) with the
        # board's power and engine clock beside them: what the operand values cost under the power cap
        lc_pw = {}
        for t in (16, 64):
            real = bench_prefill(t, 5, 2, p0=8192, batch=24, copies=3, power_seconds=0.6)
            zero = bench_prefill(t, 5, 2, p0=8192, batch=24, copies=3, zero_kv=True, power_seconds=0.6)
            lc_pw[str(t)] = {"us": round(real["kernel_ms"] * 1e3, 1), "zero_kv_us": round(zero["kernel_ms"] * 1e3, 1),
                             "watts": (real["power"] or {}).get("watts"), "engine_mhz": (real["power"] or {}).get("engine_mhz"),
                             "zero_kv_watts": (zero["power"] or {}).get("watts"),
                             "zero_kv_engine_mhz": (zero["power"] or {}).get("engine_mhz"),
                             "cap_watts": (real["power"] or {}).get("cap_watts")}
        also.append({
            "workload": "last chunk: 2-64 tokens x 24 seq on 8192-token caches, 32q/4kv, fp16; value = 16 tokens",
            "metric": "chunk attention us per call", "unit": "us",
            "value": round(lc[16]["ms_per_step"] * 1e3, 1),
            "us_by_tokens": {str(t): round(r["ms_per_step"] * 1e3, 1) for t, r in lc.items()},
            "single_token_us": round(lc_dec["ms_per_step"] * 1e3, 1),
            "board_power_by_tokens": lc_pw,
            "kv_gbs_by_tokens": {str(t): round(kv_bytes / (r["ms_per_step"] * 1e-3) / 1e9, 1) for t, r in lc.items()},
            "steps": args.steps,
            "roofline": {"bound": "hbm", "achieved": round(kv_bytes / (lc[16]["kernel_ms"] * 1e-3) / 1e9, 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(kv_bytes / (lc[16]["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                         "traffic": TRAFFIC_BYTES["lastchunk"]},
        })
        targets["lastchunk_24x8192"] = {"us_by_tokens": {str(t): round(r["kernel_ms"] * 1e3, 1) for t, r in lc.items()},
                                        "single_token_us": round(lc_dec["kernel_ms"] * 1e3, 1),
                                        "zero_kv_us": {t: v["zero_kv_us"] for t, v in lc_pw.items()},
                                        "engine_mhz": {t: v["engine_mhz"] for t, v in lc_pw.items()}}

    if args.only in ("", "mixed"):
        # one layer of the mixed-step configuration: a 16384-token prefill and a single-token step over 32
        # sequences with cache lengths U{1024..131072}; the configuration runs this 48 times a step
        mx_steps = max(3, min(args.steps, 10))
        mp = bench_prefill(16384, mx_steps, min(args.warmup, 2))
        md = bench_ragged_decode(32, 1024, 131072, mx_steps, min(args.warmup, 2))
        mq = bench_qkv_projection(16384, mx_steps, min(args.warmup, 2))
        msp = bench_step_projections(32, mx_steps, min(args.warmup, 2))
        mx_cpu = None
        if not args.skip_cpu:
            import numpy as np
            lengths = np.random.default_rng(7).integers(1024, 131072 + 1, size=32)   # as bench_ragged_decode
            cp = cpu_baseline_chunk(16384, 0, 32, 4, "f16", budget_s=1.0)
            cd = cpu_baseline_ragged_decode(lengths)
            mx_cpu = {"value": round((cp["seconds_extrapolated"] + cd["seconds_extrapolated"]) * 1e3, 1),
                      "unit": "ms", "cores": cp["cores"], "kind": "port", "pinned": True,
                      "sample": "prefill: " + cp["sample"] + "; single token: " + cd["sample"],
                      "prefill_tflops": cp["value"], "decode_gbs": cd["value"]}
        also.append({
            "workload": "mixed step, 1 of 48 layers (configs[4]): 16384-token prefill + 32 seq U{1024..131072}",
            "metric": "attention ms per layer",
            "value": round(mp["ms_per_step"] + md["ms_per_step"], 4), "unit": "ms",
            "prefill_ms": round(mp["ms_per_step"], 4), "prefill_tflops": round(mp["tflops"], 1),
            "prefill_frac_of_mfma_peak": round(mp["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4),
            "decode_ms": round(md["ms_per_step"], 4), "decode_gbs": round(md["gbs"], 1),
            "decode_cached_tokens": md["tokens"], "steps": mx_steps,
            "prefill_projection_ms": round(mq["ms_per_step"], 4),
            "prefill_projection_frac_of_mfma_peak": round(mq["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4),
            "decode_projection_ms": round(msp["qkv_ms"], 5),
            "decode_projection_frac_of_hbm_peak": round(
                msp["qkv_bytes"] / (msp["qkv_kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "roofline": {"bound": "hbm", "achieved": round(md["kernel_gbs"], 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(md["kernel_gbs"] / HBM_PEAK_GBS, 4),
                         "traffic": TRAFFIC_BYTES["mixed_decode"]},
            "cpu_baseline": mx_cpu,
        })

    if args.only in ("", "mixed48"):
        try:
            ms = bench_mixed_step(48, 16384, 32, 1024, 131072, 3, 1)
        except (ellm_amd.EllmError, RuntimeError) as e:   # e.g. 223 GB of cache not available on this box
            ms = None
            also.append({"workload": "mixed step end to end (BASELINE configs[4])", "error": str(e)[:300]})
        if ms is not None:
            # every flop at the MFMA peak plus every cache byte at the HBM peak, one after the other
            floor_ms = ((ms["flops"] + ms["proj_flops"]) / (MFMA_F16_PEAK_TFLOPS * 1e12) + ms["bytes"] / (HBM_PEAK_GBS * 1e9)) * 1e3
            also.append({
                "workload": "mixed step, 48 layers, projections + attention (configs[4]); value = one stream, one graph",
                "metric": "attention ms per step", "value": round(ms["graph_ms"], 3), "unit": "ms",
                "eager_ms": round(ms["eager_ms"], 3), "graph_ms": round(ms["graph_ms"], 3),
                "side_by_side_ms": round(ms["side_by_side_ms"], 3),
                "steps": 3, "prefill_tflop_per_step": round(ms["flops"] / 1e12, 2),
                "projection_tflop_per_step": round(ms["proj_flops"] / 1e12, 2),
                "decode_gb_per_step": round(ms["bytes"] / 1e9, 1),
                "cache_resident_gb": round(ms["resident_bytes"] / 1e9, 1),
                "floor_ms_at_both_peaks": round(floor_ms, 2), "frac_of_floor": round(floor_ms / ms["graph_ms"], 4),
            })
            targets["mixed48"] = {"ms_one_stream": round(ms["graph_ms"], 2), "ms_two_streams": round(ms["side_by_side_ms"], 2),
                                  "floor_ms": round(floor_ms, 2), "frac_of_floor": round(floor_ms / ms["graph_ms"], 4)}
    if args.only in ("", "kvwrite"):
        kw = bench_kv_write(32768, args.steps, args.warmup)
        also.append({
            "workload": "cache write, key RMS norm + rotation: 32768 tokens x 4 kv heads, fp16",
            "metric": "kv write HBM GB/s", "value": round(kw["gbs"], 1), "unit": "GB/s",
            "ms_per_step": round(kw["ms_per_step"], 5), "steps": args.steps,
            # the same rows through ellm_kv_append (copied, nothing computed) and the same bytes through
            # the runtime's device-to-device copy, timed in this run
            "plain_append_gbs": round(kw["plain_append_gbs"], 1), "device_copy_gbs": round(kw["device_copy_gbs"], 1),
            "roofline": {"bound": "hbm", "achieved": round(kw["kernel_gbs"], 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(kw["kernel_gbs"] / HBM_PEAK_GBS, 4),
                         "traffic": TRAFFIC_BYTES["kvwrite"]},
        })

    if args.only in ("", "tokenstep"):
        for (tb, tl) in ((16, 8192), (4, 1024)):
            ts = bench_token_step(48, tb, tl, min(args.steps, 20), min(args.warmup, 3))
            also.append({
                "workload": f"token step, 48 layers: cache write + attention, {tb} seq x {tl} cached tokens; value = one launch a layer",
                # fused: the write inside the attention launch (ellm_kv_append_attn_run_ragged), one graph;
                # two_calls: ellm_kv_append_norm_rope then ellm_attn_run_ragged, eagerly and from one graph
                "metric": "attention ms per token step", "value": round(ts["fused_ms"], 4), "unit": "ms",
                "fused_ms": round(ts["fused_ms"], 4), "two_calls_ms": round(ts["graph_ms"], 4),
                "two_calls_eager_ms": round(ts["eager_ms"], 4),
                "steps": min(args.steps, 20),
                "gbs": round(ts["bytes"] / (ts["fused_ms"] * 1e-3) / 1e9, 1),
            })
            targets[f"tokenstep_{tb}x{tl}"] = {"ms": round(ts["fused_ms"], 4), "two_calls_ms": round(ts["graph_ms"], 4),
                                               "frac": round(ts["bytes"] / (ts["fused_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    if args.only in ("", "qkv"):
        pj_steps = max(3, min(args.steps, 20))
        pj = bench_qkv_projection(32768, pj_steps, min(args.warmup, 3))
        also.append({
            "workload": "fused Q/K/V projection: 32768 rows x 2048 -> 5120, norm + rotation, K/V to the cache, fp16",
            "metric": "projection TFLOP/s", "value": round(pj["tflops"], 2), "unit": "TFLOP/s",
            "ms_per_step": round(pj["ms_per_step"], 4), "steps": pj_steps,
            "roofline": {"bound": "mfma", "achieved": round(pj["kernel_tflops"], 2),
                         "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(pj["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4),
                         "traffic": TRAFFIC_BYTES["qkv"]},
        })
    if args.only in ("", "oproj"):
        pj_steps = max(3, min(args.steps, 20))
        po = bench_output_projection(32768, pj_steps, min(args.warmup, 3))
        also.append({
            "workload": "output projection + residual: 32768 tokens x 4096 -> 2048, fp16",
            "metric": "projection TFLOP/s", "value": round(po["tflops"], 2), "unit": "TFLOP/s",
            "ms_per_step": round(po["ms_per_step"], 4), "steps": pj_steps,
            "roofline": {"bound": "mfma", "achieved": round(po["kernel_tflops"], 2),
                         "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(po["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None},
        })

    if args.only in ("", "chunkproj"):
        # the reference's serving shape: chunks of 64 positions x 24 sequences (src/serving/start copy.rs:30)
        cq = bench_qkv_projection(64, args.steps, min(args.warmup, 5), batch=24)
        co = bench_output_projection(64 * 24, args.steps, min(args.warmup, 5))
        also.append({
            "workload": "projections at 1536 rows (64 positions x 24 seq): Q/K/V 2048 -> 5120, output 4096 -> 2048, fp16",
            "metric": "projection TFLOP/s (Q/K/V)", "value": round(cq["tflops"], 2), "unit": "TFLOP/s",
            "ms_per_step": round(cq["ms_per_step"], 5), "steps": args.steps,
            "output_projection_ms": round(co["ms_per_step"], 5),
            "output_projection_tflops": round(co["tflops"], 2),
            "roofline": {"bound": "mfma", "achieved": round(cq["kernel_tflops"], 2),
                         "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(cq["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None},
        })
        targets["chunkproj_1536"] = {
            "qkv_us": round(cq["kernel_ms"] * 1e3, 2), "output_us": round(co["kernel_ms"] * 1e3, 2),
            "qkv_frac": round(cq["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4),
            "output_frac": round(co["kernel_tflops"] / MFMA_F16_PEAK_TFLOPS, 4)}

    if args.only in ("", "chunkblock"):
        cb = bench_chunk_block(64, 24, 4096, min(args.steps, 30), min(args.warmup, 5))
        also.append({
            "workload": "layer block, chunk of 64 positions x 24 seq on 4096-token caches: Q/K/V + attention + output",
            "metric": "attention-block ms per chunk", "value": round(cb["block_ms"], 5), "unit": "ms",
            "steps": min(args.steps, 30),
            "qkv_ms": round(cb["parts_ms"]["qkv"], 5), "attention_ms": round(cb["parts_ms"]["attention"], 5),
            "output_ms": round(cb["parts_ms"]["output"], 5),
            "tflops": round(cb["flops"] / (cb["block_ms"] * 1e-3) / 1e12, 1),
        })

    if args.only in ("", "stepproj"):
        sp = bench_step_projections(16, args.steps, args.warmup)
        also.append({
            "workload": "projections of a token step, 16 seq: Q/K/V 2048 -> 5120, output 4096 -> 2048, weights from HBM",
            "metric": "weight stream GB/s (Q/K/V projection)", "unit": "GB/s",
            "value": round(sp["qkv_bytes"] / (sp["qkv_ms"] * 1e-3) / 1e9, 1),
            "ms_per_step": round(sp["qkv_ms"], 5), "steps": args.steps,
            "output_projection_ms": round(sp["o_ms"], 5),
            "output_projection_gbs": round(sp["o_bytes"] / (sp["o_ms"] * 1e-3) / 1e9, 1),
            "roofline": {"bound": "hbm", "achieved": round(sp["qkv_bytes"] / (sp["qkv_kernel_ms"] * 1e-3) / 1e9, 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(sp["qkv_bytes"] / (sp["qkv_kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                         "traffic": TRAFFIC_BYTES["stepproj"]},
        })
        targets["stepproj_16"] = {
            "qkv_us": round(sp["qkv_kernel_ms"] * 1e3, 2), "output_us": round(sp["o_kernel_ms"] * 1e3, 2),
            "qkv_frac": round(sp["qkv_bytes"] / (sp["qkv_kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "output_frac": round(sp["o_bytes"] / (sp["o_kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    if args.only in ("", "layerstep"):
        # 16 x 8192: BASELINE configs[1] with its projections; 4 x 1024: a small batch; 1 x 512 / 256 / 128:
        # the operating point of the reference's own published numbers (decode at batch 1 after a prompt
        # of 128 / 256 / 512 tokens, README.md:92-116; its figures include the MoE blocks, these do not)
        cases = [(16, 8192), (4, 1024), (1, 512), (1, 256), (1, 128)]
        if args.layer_cases:
            cases = [tuple(int(v) for v in c.split("x")) for c in args.layer_cases.split(",")]
        lsr = bench_layer_steps(48, cases, args.steps, min(args.warmup, 3))
        for (lb, ll) in cases:
            ls = lsr[(lb, ll)]
            nbytes = ls["kv_bytes"] + ls["w_bytes"]
            ls_cpu = None
            if not args.skip_cpu and (lb == 1 or (lb, ll) == (16, 8192)):
                ls_cpu = cpu_baseline_layer_step(lb, ll)
            dev_ms = min(ls["fused_dev_ms"], ls["graph_dev_ms"])
            also.append({
                "workload": f"layer step, 48 layers: Q/K/V projection + attention + output projection, {lb} seq x {ll} cached tokens",
                "metric": "attention-block ms per token step", "value": round(min(ls["fused_ms"], ls["graph_ms"]), 4), "unit": "ms",
                # fused: projection + attention of a layer through ellm_matmul3_attn_run (2 launches,
                # no exchange between the projection's workgroups); three_calls: the three operators
                # one by one; both replayed from one recorded graph
                "fused_ms": round(ls["fused_ms"], 4), "three_calls_ms": round(ls["graph_ms"], 4),
                "three_calls_eager_ms": round(ls["eager_ms"], 4),
                "kernel_ms": round(dev_ms, 4), "us_per_layer": round(dev_ms * 1e3 / 48, 2),
                "steps": ls["steps"],
                "cache_gb_per_step": round(ls["kv_bytes"] / 1e9, 3), "weight_gb_per_step": round(ls["w_bytes"] / 1e9, 3),
                "roofline": {"bound": "hbm", "achieved": round(nbytes / (dev_ms * 1e-3) / 1e9, 1),
                             "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(nbytes / (dev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                             "traffic": TRAFFIC_BYTES.get(f"layerstep_{lb}x{ll}")},
                "cpu_baseline": ls_cpu,
            })
            targets[f"layerstep_{lb}x{ll}"] = {
                "ms": round(dev_ms, 4), "us_per_layer": round(dev_ms * 1e3 / 48, 2),
                "three_calls_us_per_layer": round(ls["graph_dev_ms"] * 1e3 / 48, 2),
                "fused_us_per_layer": round(ls["fused_dev_ms"] * 1e3 / 48, 2),
                "frac": round(nbytes / (dev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    cpu = None
    if not args.skip_cpu and dec is not None:
        cpu = cpu_baseline_decode(16, 8192)

    also += last_entries
    if dec is None:  # partial run for profiling
        print(json.dumps({"targets": targets, "also": also}))
        return
    line = {
        "metric": "decode attn HBM GB/s (Qwen3 GQA, 1 GPU)",
        "value": round(dec["gbs"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dec["ms_per_step"], 5),
        # value = algorithmic bytes / ms_per_step (host clock around the K steps); roofline.achieved and
        # .frac = the same bytes / kernel_ms (HIP events on the launch stream around the same K launches)
        "kernel_ms": round(dec["kernel_ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "decode: 16 seq x 8192 cached tokens, 32q/4kv heads, fp16 (BASELINE configs[1])",
                   "batch": 16, "cache_len": 8192, "q_heads": 32, "kv_heads": 4},
        "roofline": {"bound": "hbm", "achieved": round(dec["kernel_gbs"], 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(dec["kernel_gbs"] / HBM_PEAK_GBS, 4),
                     "traffic": TRAFFIC_BYTES["decode"], "timer": "kernel_ms (HIP events)",
                     # the headline figures of the other workloads (their full entries are in `also`)
                     "targets": targets},
        "cpu_baseline": cpu,
        "passes": dec["passes"],
        "cpu_model": host["cpu_model"],
        "host_cores": host["host_cores"],
        "also": also,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
