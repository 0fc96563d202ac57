#!/usr/bin/env python3
"""Benchmark of the paged q8_0 KV decode step on one MI355X: append one token per sequence, then paged GQA decode
attention, on the batched ragged configuration (64 sequences, context lengths uniform in [1024, 65536], 24 Q / 4 KV
heads, head_dim 256, 64-token pages from one shared shuffled pool sized to fit exactly).

Prints ONE JSON line. `value` is the algorithmic KV bytes of a step (sum of context lengths x 2176 B) over the wall
time of a step with everything resident in HBM; `roofline` is the same bytes over the split-K kernel's own duration,
measured with HIP events on the launch stream; `cpu_baseline` is the CPU oracle's decode attention on a bounded
sample of the same sequences, on this box's host cores.
"""
import argparse
import ctypes
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    # name: (format, batch, lo, hi, outlier channels)
    "ragged_b64_q8_0": dict(fmt=8, batch=64, lo=1024, hi=65536, seed=4),
    # one sequence's KV (71 MB) would stay in the 256 MB last-level cache from step to step: the steps rotate over
    # eight layers' pools, as the layers of a model do
    "b1_ctx32k_q8_0": dict(fmt=8, batch=1, lo=32768, hi=32768, seed=4, layers=8),
    # (this kernel runs as fast as the shader clock up to about 2.1 GHz, and after an idle GPU the clock falls from 2.4 to
    # 1.3 GHz within 3 ms and is back at the 2.1 GHz it holds under this kernel some 30 ms later: the default warm-up
    # waits for that, and the line's after_idle object holds the steps timed right after an idle period)
    "b16_ctx128k_q4_0": dict(fmt=4, batch=16, lo=131072, hi=131072, seed=4, outliers=8, warmup=80),
    # chunked prefill: every sequence holds `lo` tokens and takes a chunk of `chunk` more per step (the first six
    # launches of the attention kernel after an idle GPU run up to 25 % longer than the later ones)
    "prefill_b8_ctx16k_chunk2k_q8_0": dict(fmt=8, batch=8, lo=16384, hi=16384, seed=4, chunk=2048, warmup=10),
    "prefill_b8_ctx16k_chunk2k_q4_0": dict(fmt=4, batch=8, lo=16384, hi=16384, seed=4, chunk=2048, warmup=10),
    # the unquantized f16 twins of the decode path (4096 B per token)
    "b16_ctx128k_f16": dict(fmt=16, batch=16, lo=131072, hi=131072, seed=4),
    "ragged_b64_f16": dict(fmt=16, batch=64, lo=1024, hi=65536, seed=4),
    "prefill_b8_ctx16k_chunk2k_f16": dict(fmt=16, batch=8, lo=16384, hi=16384, seed=4, chunk=2048, warmup=10),
    # the reference's own KV format (kv8a16: 2336 B per token, 256-token pages), the same ragged batch
    "ragged_b64_kv8a16": dict(fmt=816, batch=64, lo=1024, hi=65536, seed=4),
    "b1_ctx32k_kv8a16": dict(fmt=816, batch=1, lo=32768, hi=32768, seed=4, layers=8),
    "prefill_b8_ctx16k_chunk2k_kv8a16": dict(fmt=816, batch=8, lo=16384, hi=16384, seed=4, chunk=2048, warmup=10),
    # ... and in its 4-bit sibling, kv4a16 (H256-rotated K in 16 levels per 32-dim group, V in 15 levels per tile)
    "ragged_b64_kv4a16": dict(fmt=416, batch=64, lo=1024, hi=65536, seed=4, warmup=80),
    "b16_ctx128k_kv4a16": dict(fmt=416, batch=16, lo=131072, hi=131072, seed=4, warmup=80),
    "prefill_b8_ctx16k_chunk2k_kv4a16": dict(fmt=416, batch=8, lo=16384, hi=16384, seed=4, chunk=2048, warmup=10),
}
MFMA_F16_PEAK_TFLOPS = 2500.0
EVENT_EVERY = 4      # decode workloads: HIP events around the split-K kernel on every fourth timed step
NQ, NKV, HD, PT = 24, 4, 256, 64
# HBM bytes per launch of each workload's dominant kernel from rocprofv3 counters (FETCH_SIZE + WRITE_SIZE, each scaled
# by what the counter reads for a plain 1 GiB copy): measurements made outside this script, kept in a tracked table that
# names the commit each was taken at.
def load_traffic():
    table = {}
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.md")) as f:
            for line in f:
                cols = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cols) == 5 and cols[0] in WORKLOADS:
                    table[cols[0]] = (float(cols[1]), "%s (kernel %s, measured at commit %s)" % (cols[4], cols[2], cols[3]))
    except (OSError, ValueError):
        pass
    return table


TRAFFIC = load_traffic()

def fnv1a(b):
    h = 0xCBF29CE484222325
    for x in np.frombuffer(b, np.uint8)[:65536]:
        h = ((h ^ int(x)) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return f"{h:016x}"


def build_state(yahkv, torch, wl, total_steps):
    rng = np.random.default_rng(wl["seed"])
    lens = rng.integers(wl["lo"], wl["hi"] + 1, wl["batch"]).astype(np.int32)
    total_steps = wl.get("chunk", total_steps)       # prefill: room for one chunk, rewritten by every step
    pages = (lens + total_steps + PT - 1) // PT
    n_pages = int(pages.sum())                       # the pool fits the job exactly
    g = yahkv.geometry(wl["fmt"], NQ, NKV, HD, PT, n_pages)
    alloc = yahkv.PagePool(n_pages)
    alloc.shuffle(12345)
    table = np.zeros((wl["batch"], int(pages.max())), np.int32)
    for s, n in enumerate(pages):
        table[s, :n] = alloc.alloc(int(n))
    assert alloc.free_count == 0
    yahkv.validate_page_table(g, table, lens + total_steps)
    layers = [yahkv.DevicePools(g) for _ in range(wl.get("layers", 1))]
    t_table = torch.from_numpy(table).cuda()
    gen = torch.Generator(device="cuda").manual_seed(wl["seed"])
    chunk = 8192
    outl = None
    if wl.get("outliers"):
        outl = torch.ones(NKV, HD, device="cuda")
        for h in range(NKV):
            outl[h, torch.from_numpy(rng.permutation(HD)[:wl["outliers"]]).cuda()] = 20.0
    for pools in layers:                             # fill the prefix through the library's own append
        for s in range(wl["batch"]):
            for o in range(0, int(lens[s]), chunk):
                n = min(chunk, int(lens[s]) - o)
                k = torch.randn((1, n, NKV, HD), generator=gen, device="cuda", dtype=torch.float32)
                if outl is not None:
                    k = k * outl
                v = torch.randn((1, n, NKV, HD), generator=gen, device="cuda", dtype=torch.float32)
                yahkv.append(pools, t_table[s:s + 1], torch.tensor([o], dtype=torch.int32, device="cuda"),
                             k.to(torch.bfloat16), v.to(torch.bfloat16))
    torch.cuda.synchronize()
    return g, layers, lens, table, t_table, gen


def clock_trace(yahkv, torch, launch, n=60, idle_s=3.0):
    """After `idle_s` seconds without GPU work: n launches of `launch` (a callable that queues the workload's dominant
    kernel), each followed by the library's clock probe. Returns per launch its duration (HIP events) and the shader
    clock right after it. An extra figure for instruction-bound kernels, whose speed follows the clock."""
    res = torch.zeros((n, 2), dtype=torch.int64, device="cuda")
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    torch.cuda.synchronize()
    time.sleep(idle_s)
    for i in range(n):
        ev[i][0].record()
        launch()
        ev[i][1].record()
        yahkv.shader_clock_probe(res[i], 2000)       # 20 us
    torch.cuda.synchronize()
    r = res.cpu().numpy().astype(np.float64)
    trace = {"idle_s": idle_s, "kernel_ms": [round(a.elapsed_time(b), 4) for a, b in ev],
             "shader_mhz": [int(round(x)) for x in r[:, 0] / np.maximum(r[:, 1], 1) * 100.0],
             "note": "launches of the dominant kernel back to back after an idle GPU, the shader clock after each"}
    # The clock WHILE the kernel runs: the same launches back to back (the GPU is warm now), and probes of 0.5 ms each on
    # a second stream beside them. The probe's wave shares a CU with the kernel's workgroups, so the launches run a
    # little slower than alone (much slower where one workgroup per CU holds a fixed share of the work).
    per = float(np.median(trace["kernel_ms"][n // 2:]))
    n_load = max(int(120.0 / per), 8)                  # about 120 ms of load
    n_probe = int(n_load * per / 0.5) + 20
    side = torch.cuda.Stream()
    res = torch.zeros((n_probe, 2), dtype=torch.int64, device="cuda")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(n_load):
        launch()
    e1.record()
    side.wait_event(e0)
    with torch.cuda.stream(side):
        for i in range(n_probe):
            yahkv.shader_clock_probe(res[i], 50000)
    torch.cuda.synchronize()
    total = e0.elapsed_time(e1)
    r = res.cpu().numpy().astype(np.float64)
    mhz = (r[:, 0] / np.maximum(r[:, 1], 1) * 100.0)[:max(min(int(total / 0.5) - 2, n_probe), 1)]
    trace["under_load"] = {"shader_mhz_median": int(np.median(mhz[len(mhz) // 2:])),
                           "shader_mhz_p10_p90": [int(np.percentile(mhz[len(mhz) // 2:], 10)),
                                                  int(np.percentile(mhz[len(mhz) // 2:], 90))],
                           "kernel_ms_beside_the_probe": round(total / n_load, 4), "launches": n_load,
                           "note": "probes of 0.5 ms on a second stream while the launches run; second half of them"}
    return trace


def closed_form_err(Kd, Vd, qs, scale, got):
    """max |got - want| / max |want| of one sequence against softmax(q K^T scale) V in float64 (Kd, Vd [n][H][D])."""
    Kd, Vd, qs = Kd.astype(np.float64), Vd.astype(np.float64), qs.astype(np.float64)
    want = np.zeros((NQ, HD))
    for h in range(NQ):
        sc = Kd[:, h // (NQ // NKV)] @ qs[h] * scale
        p = np.exp(sc - sc.max())
        want[h] = (p / p.sum()) @ Vd[:, h // (NQ // NKV)]
    return float(np.abs(got - want).max() / np.abs(want).max())


def parity_check(yahkv, torch, g, pools, t_table, lens, q, out, scale, rows):
    """Closed-form float64 attention on the library's own gathered blocks, for a few sequences, before timing."""
    import oracle
    worst = 0.0
    for s in rows:
        n = int(lens[s])
        k, v = yahkv.gather_blocks(pools, t_table[s], n)
        bb = k.shape[-1]
        deq = oracle.dequantize_q8_0 if g.format == 8 else oracle.dequantize_q4_0
        Kd = deq(k.cpu().numpy().reshape(-1, bb)).reshape(n, NKV, HD).astype(np.float64)
        Vd = deq(v.cpu().numpy().reshape(-1, bb)).reshape(n, NKV, HD).astype(np.float64)
        qs = q[s].float().cpu().numpy().astype(np.float64)
        want = np.zeros((NQ, HD))
        for h in range(NQ):
            sc = Kd[:, h // (NQ // NKV)] @ qs[h] * scale
            p = np.exp(sc - sc.max())
            want[h] = (p / p.sum()) @ Vd[:, h // (NQ // NKV)]
        got = out[s].cpu().numpy()
        worst = max(worst, float(np.abs(got - want).max() / np.abs(want).max()))
    return worst


CPU_REPS = 5
APPEND_REPS = 20


def time_repeated(torch, fn, reps=APPEND_REPS):
    """ms per call of a short, repeatable piece of GPU work: `reps` calls back to back between one pair of HIP events
    (a pair of events around a single call adds about 6 us of its own, a third of what a chunk append takes)."""
    fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def median_time(fn, reps=CPU_REPS):
    fn()                                                       # warm-up
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return float(np.median(times))


def cpu_decode_case(oracle, fmt, n_q, n_kv, hd, pt, lens, seed, q_kind):
    """The oracle's append + decode attention on one configuration; returns (seconds per attention, tokens, bytes)."""
    rng = np.random.default_rng(seed)
    lens = np.asarray(lens, np.int32)
    pages = (lens + pt - 1) // pt
    g = oracle.geometry(fmt, n_q, n_kv, hd, pt, int(pages.sum()))
    perm = rng.permutation(g.n_pages).astype(np.int32)
    table = np.zeros((len(lens), int(pages.max())), np.int32)
    o = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[o:o + n]
        o += n
    host = oracle.HostPools(g)
    t0 = time.perf_counter()
    for i, n in enumerate(lens):
        oracle.append(host, table[i:i + 1], [0], None, rng.standard_normal((1, int(n), n_kv, hd), np.float32),
                      rng.standard_normal((1, int(n), n_kv, hd), np.float32))
    t_quant = time.perf_counter() - t0
    q = rng.standard_normal((len(lens), n_q, hd)).astype(np.float32)
    scale = 1.0 / float(np.sqrt(hd))
    t = median_time(lambda: oracle.decode_attend(host, table, lens, q, scale))
    h = fnv1a(oracle.decode_attend(host, table, lens, q, scale).tobytes())
    bpt = 2 * n_kv * (hd // 32) * ((32 if fmt == 8 else 16) + 2)
    return t, int(lens.sum()), int(lens.sum()) * bpt, t_quant, h


def cpu_baseline(wl, lens, scale, budget_tokens=150000):
    """The CPU oracle (a port: the reference has no CPU paged attention), rebuilt for this box's host cores with the
    reference's host flags (-O3 -march=native -ffp-contract=off, engine/build_hrx.sh:26), all host cores: decode
    attention on the first sequences of the batch whose lengths add up to about budget_tokens, and on the two small
    configurations; median of 5 after a warm-up."""
    import oracle
    build = oracle.use_native_build()
    take, tot = [], 0
    for s, n in enumerate(lens):
        if take and tot + int(n) > budget_tokens:
            break
        take.append(s)
        tot += int(n)
    t, tot, nbytes, t_quant, h = cpu_decode_case(oracle, wl["fmt"], NQ, NKV, HD, PT, lens[take], 99, "bf16")
    rng = np.random.default_rng(99)
    ref_append = None
    if wl["fmt"] == 8 and oracle.ref() is not None:
        # the reference's own CPU code on this path: QuantizeQ8_0 (engine/core/gguf_quant.cpp:310-320), compiled from its
        # sources into oracle/_ref; scalar, one thread, as the reference runs it
        import ctypes as C
        n_el = 1 << 22
        x = rng.standard_normal(n_el).astype(np.float32)
        dst = np.empty(n_el // 32 * 34, np.uint8)
        fn = oracle.ref().ref_quantize_q8_0
        fn.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p]
        tr = median_time(lambda: fn(x.ctypes.data, n_el, dst.ctypes.data))
        ref_append = {"blocks_per_s": round(n_el / 32 / tr, 0), "kind": "reference", "cores": 1,
                      "sample": f"the reference's QuantizeQ8_0 on {n_el // 32} blocks of N(0,1), median of {CPU_REPS}"}
    res = {"value": round(nbytes / t / 1e9, 3), "unit": "GB/s", "cores": oracle.threads(), "kind": "port", "build": build,
           "sample": f"oracle decode attention on the first {len(take)} sequences of the batch ({tot} tokens, "
                     f"{nbytes / 1e6:.0f} MB of KV), median of {CPU_REPS} after a warm-up",
           "tok_per_s": round(len(take) / t, 2), "out_fnv1a": h,
           "append_blocks_per_s": round(tot * 2 * NKV * (HD // 32) / t_quant, 0),
           "append_note": "oracle scalar block quantizer + page scatter, 1 thread",
           "append_reference": ref_append}
    if wl["fmt"] == 8:
        # the two configurations a CPU runs whole: the tiny one (8 Q / 2 KV heads of 128 dims, 16-token pages, 513 keys)
        # and one sequence of 32768 tokens at the benchmark's geometry
        t1, n1, b1, _, h1 = cpu_decode_case(oracle, 8, 8, 2, 128, 16, [513], 1, "f16")
        t2, n2, b2, _, h2 = cpu_decode_case(oracle, 8, NQ, NKV, HD, PT, [32768], 2, "bf16")
        res["configs"] = {
            "config1_tiny": {"ms": round(t1 * 1e3, 4), "GB/s": round(b1 / t1 / 1e9, 3), "tokens": n1, "out_fnv1a": h1},
            "config2_b1_ctx32k": {"ms": round(t2 * 1e3, 3), "GB/s": round(b2 / t2 / 1e9, 3), "tokens": n2,
                                  "out_fnv1a": h2}}
    return res


def prefill_cpu_baseline(wl, scale, prefix=2048, chunk=64):
    """The CPU oracle's chunked-prefill attention (f32 operands) on one short sequence, all host cores."""
    import oracle
    rng = np.random.default_rng(98)
    n = prefix + chunk
    g = oracle.geometry(wl["fmt"], NQ, NKV, HD, PT, (n + PT - 1) // PT)
    table = rng.permutation(g.n_pages).astype(np.int32)[None]
    host = oracle.HostPools(g)
    oracle.append(host, table, [0], None, rng.standard_normal((1, n, NKV, HD), np.float32),
                  rng.standard_normal((1, n, NKV, HD), np.float32))
    q = rng.standard_normal((1, chunk, NQ, HD)).astype(np.float32)
    build = oracle.use_native_build()
    t = median_time(lambda: oracle.prefill_attend(host, table, [prefix], q, scale))
    flops = NQ * chunk * (prefix + (chunk + 1) / 2) * HD * 4
    return {"value": round(flops / t / 1e12, 5), "unit": "TFLOP/s", "cores": oracle.threads(), "kind": "port",
            "build": build,
            "sample": f"oracle prefill attention, 1 sequence, prefix {prefix} + chunk {chunk}, median of {CPU_REPS} "
                      "after a warm-up", "tok_per_s": round(chunk / t, 1)}


def run_f16(a, wl, torch, yahkv):
    """A step on unquantized f16 pools: append one token per sequence + decode attention (partials, then their merge)."""
    rng = np.random.default_rng(wl["seed"])
    B = wl["batch"]
    lens = rng.integers(wl["lo"], wl["hi"] + 1, B).astype(np.int32)
    total = a.warmup + a.steps + 1
    pages = (lens + total + PT - 1) // PT
    n_pages = int(pages.sum())
    g = yahkv.f16_geometry(NQ, NKV, HD, PT, n_pages)
    perm = rng.permutation(n_pages).astype(np.int32)
    table = np.zeros((B, int(pages.max())), np.int32)
    o = 0
    for s, n in enumerate(pages):
        table[s, :n] = perm[o:o + n]
        o += n
    pools = yahkv.F16Pools(g)
    t_table = torch.from_numpy(table).cuda()
    gen = torch.Generator(device="cuda").manual_seed(wl["seed"])
    for s in range(B):                                   # fill the prefix through the library's own append
        for o in range(0, int(lens[s]), 8192):
            n = min(8192, int(lens[s]) - o)
            k = torch.randn((1, n, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            v = torch.randn((1, n, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            yahkv.f16_append(pools, t_table[s:s + 1], torch.tensor([o], dtype=torch.int32, device="cuda"), k, v)
    scale = 1.0 / float(np.sqrt(HD))
    max_len = int(lens.max()) + total
    len_rows = torch.from_numpy(lens[None, :] + np.arange(total + 1, dtype=np.int32)[:, None]).cuda()
    q = torch.randn((B, NQ, HD), generator=gen, device="cuda").to(torch.bfloat16)
    knew = torch.randn((total, B, 1, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    vnew = torch.randn((total, B, 1, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.empty((B, NQ, HD), dtype=torch.float32, device="cuda")
    ws = torch.empty(yahkv.lib.yahkv_f16_decode_workspace_bytes(g, B, max_len, None), dtype=torch.uint8, device="cuda")
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]

    def step(i, pair=None):
        yahkv.f16_append(pools, t_table, len_rows[i], knew[i], vnew[i])
        if pair:
            pair[0].record()
        yahkv.f16_decode_attend(pools, t_table, len_rows[i + 1], max_len, q, scale, out=out, workspace=ws)
        if pair:
            pair[1].record()

    # parity before timing: the shortest sequence against the float64 closed form over the pools' own f16 values
    step(0)
    torch.cuda.synchronize()
    first_hash = fnv1a(out.cpu().numpy().tobytes())
    s0 = int(np.argmin(lens))
    n0 = int(lens[s0]) + 1
    kp, vp = pools.k.view(torch.float16), pools.v.view(torch.float16)
    kp = kp.view(n_pages, NKV, HD // 16, PT, 16)
    run = min(PT, 32)                                    # V^T lies in runs of at most 32 keys
    vp = vp.view(n_pages, NKV, PT // run, HD, run)
    pg = t_table[s0, :(n0 + PT - 1) // PT].long()
    Kd = kp[pg].permute(0, 3, 1, 2, 4).reshape(-1, NKV, HD)[:n0].double().cpu().numpy()
    Vd = vp[pg].permute(0, 2, 4, 1, 3).reshape(-1, NKV, HD)[:n0].double().cpu().numpy()
    qs = q[s0].double().cpu().numpy()
    err = 0.0
    for h in range(NQ):
        sc = Kd[:, h // (NQ // NKV)] @ qs[h] * scale
        p = np.exp(sc - sc.max())
        want = (p / p.sum()) @ Vd[:, h // (NQ // NKV)]
        err = max(err, float(np.abs(out[s0, h].cpu().numpy() - want).max() / np.abs(want).max()))
    if not err < 2e-3:
        raise SystemExit(f"bench.py: parity check failed before timing: max relative error {err:.3e}")
    for i in range(a.warmup):
        step(1 + i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(1 + a.warmup + i, ev[i])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / a.steps * 1e3
    kern_ms = float(np.mean([p[0].elapsed_time(p[1]) for p in ev]))
    kv_bytes = float(np.sum(lens + a.warmup + 1 + (a.steps + 1) / 2)) * 2 * NKV * HD * 2
    gbs, kgbs = kv_bytes / (ms * 1e-3) / 1e9, kv_bytes / (kern_ms * 1e-3) / 1e9
    return {
        "metric": "paged f16 KV decode-attn HBM GB/s (% of peak) + tok/s", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "ctx_min": int(lens.min()), "ctx_max": int(lens.max()),
                   "ctx_sum": int(lens.sum()), "n_q_heads": NQ, "n_kv_heads": NKV, "head_dim": HD, "page_tokens": PT,
                   "n_pages": n_pages, "kv_format": "f16", "step": "append 1 token/seq + paged decode attention"},
        "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2), "tok_per_s": round(B / (ms * 1e-3), 1),
        "kv_bytes_per_step": int(kv_bytes), "parity_max_rel_err": float(f"{err:.3e}"), "out_fnv1a": first_hash,
        "roofline": {"bound": "hbm", "achieved": round(kgbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(kgbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC.get(a.workload, (None, None))[0],
                     "traffic_source": TRAFFIC.get(a.workload, (None, None))[1],
                     "kernel": "PartF16<%d, %d> + ReduceF16" % (HD, PT), "kernel_ms": round(kern_ms, 4)},
        "cpu_baseline": None}


def run_kv8(a, wl, torch, yahkv):
    """A step on kv8a16 pools (the reference's own format): one new token per sequence and the attention over the
    sequence with it, LoomDecoder::Step's kappend, vappend, part_q, reduce (loom_decoder.hpp:253-268) in two dispatches:
    split-K partials over the closed 16-key tiles, then the merge, which takes the open tile's keys, quantizes the new
    token's K row, puts its V row into the open tile and closes the tile on its 16th key."""
    rng = np.random.default_rng(wl["seed"])
    B, PG = wl["batch"], 256
    lens = rng.integers(wl["lo"], wl["hi"] + 1, B).astype(np.int32)
    total = a.warmup + a.steps + 1
    pages = (lens + total + PG - 1) // PG
    n_layers = wl.get("layers", 1)
    n_pages = int(pages.sum())                       # the pool fits the job exactly
    bits = 4 if wl["fmt"] == 416 else 8
    g = yahkv.kv8_geometry(NQ, NKV, n_pages, bits, bits)
    alloc = yahkv.PagePool(n_pages)
    alloc.shuffle(12345)
    table = np.zeros((B, int(pages.max())), np.int32)
    for s, n in enumerate(pages):
        table[s, :n] = alloc.alloc(int(n))
    assert alloc.free_count == 0
    layers = [yahkv.Kv8Pools(g) for _ in range(n_layers)]
    t_table = torch.from_numpy(table).cuda()
    gen = torch.Generator(device="cuda").manual_seed(wl["seed"])
    for pools in layers:                             # the prefix through the library's own kmean + chunk append
        for s in range(B):
            for o in range(0, int(lens[s]), 8192):
                n = min(8192, int(lens[s]) - o)
                k = (torch.randn((1, n, NKV, HD), generator=gen, device="cuda") + 0.5).to(torch.bfloat16)
                v = torch.randn((1, n, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
                if o == 0:
                    yahkv.kv8_kmean(pools, t_table[s:s + 1], k)
                yahkv.kv8_append(pools, t_table[s:s + 1], torch.tensor([o], dtype=torch.int32, device="cuda"), k, v)
    scale = 1.0 / float(np.sqrt(HD))
    max_len = int(lens.max()) + total
    len_rows = torch.from_numpy(lens[None, :] + np.arange(total + 1, dtype=np.int32)[:, None]).cuda()
    q = torch.randn((B, NQ, HD), generator=gen, device="cuda").to(torch.bfloat16)
    knew = torch.randn((total, B, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    vnew = torch.randn((total, B, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.empty((B, NQ, HD), dtype=torch.float32, device="cuda")
    opt = yahkv.decode_options(deterministic=a.deterministic, min_chunk_tiles=a.min_chunk_tiles)
    if a.first_come:
        opt.deterministic = -1
    ws = torch.empty(yahkv.lib.yahkv_kv8_decode_workspace_bytes(g, B, max_len, opt), dtype=torch.uint8, device="cuda")
    xcd = (yahkv.kv8_decode_calibrate(layers[0], t_table, len_rows[0], max_len, q, ws, opt, rounds=3)
           if not a.no_calibrate else None)            # set-up, as a server does once (equal shares without it)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]

    def step(i, pair=None):
        pools = layers[i % n_layers]
        seq_len = len_rows[i + 1]
        if pair:
            pair[0].record()
        yahkv.kv8_decode_part(pools, t_table, seq_len, max_len, q, scale, ws, opt=opt)
        if pair:
            pair[1].record()
        yahkv.kv8_decode_reduce(pools, t_table, seq_len, max_len, q, scale, out, ws, knew[i], vnew[i], opt=opt)

    # parity before timing: the first step's output of the shortest, the median and the longest sequence against the
    # float64 closed form over the oracle's dequantized model of those sequences' pages
    step(0)
    torch.cuda.synchronize()
    first_hash = fnv1a(out.cpu().numpy().tobytes())
    from oracle import kv8 as okv8
    order = np.argsort(lens)
    rows = sorted({int(order[0]), int(order[len(order) // 2]), int(order[-1])})
    err = 0.0
    for s in rows:
        n = int(lens[s]) + 1
        hp, row = okv8.pools_of_sequence(layers[0], table[s], n)
        Kd, Vd = okv8.dense(hp, row, n)
        qs = q[s].float().cpu().numpy()
        if bits == 4:                                # 4-bit K is stored rotated: the scores are taken against H256 q / 16
            qs = okv8.rotate_q(qs)
        err = max(err, closed_form_err(Kd, Vd, qs, scale, out[s].cpu().numpy()))
    if not err < 2e-3:
        raise SystemExit(f"bench.py: parity check failed before timing: max relative error {err:.3e}")
    for i in range(a.warmup):
        step(1 + i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(1 + a.warmup + i, ev[i] if i % EVENT_EVERY == 0 else None)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / a.steps * 1e3
    kern_ms = float(np.mean([p[0].elapsed_time(p[1]) for p in ev[::EVENT_EVERY]]))
    kern_how = "HIP events around the part kernel of every %d-th timed step" % EVENT_EVERY
    if kern_ms < 0.1:
        # A pair of events around one launch adds about 6 us of its own: the timed steps' part launches again, one
        # behind the other between a single pair of events (they only write partials; the layers rotate as in the steps).
        it = iter(range(a.steps))

        def part_only():
            i = 1 + a.warmup + next(it, 0)
            yahkv.kv8_decode_part(layers[i % n_layers], t_table, len_rows[i + 1], max_len, q, scale, ws, opt=opt)
        again = time_repeated(torch, part_only, reps=a.steps - 1)
        if again < kern_ms:                              # (not below when the host cannot queue them fast enough)
            kern_ms, kern_how = again, "the timed steps' part launches back to back between one pair of HIP events"
    bpt = 2336 if bits == 8 else 1408                    # kq 1024 + ks 32 + vq 1024 + vs 256; 512 + 128 + 512 + 256 (architecture.md:219-220)
    tokens = [int(lens.sum()) + B * (2 + a.warmup + i) for i in range(a.steps)]
    kv_bytes = float(np.mean(tokens)) * bpt
    gbs, kgbs = kv_bytes / (ms * 1e-3) / 1e9, kv_bytes / (kern_ms * 1e-3) / 1e9
    res = {
        "metric": "paged kv%da16 KV decode-attn HBM GB/s (%% of peak) + tok/s" % bits, "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "ctx_min": int(lens.min()), "ctx_max": int(lens.max()),
                   "ctx_sum": int(lens.sum()), "n_q_heads": NQ, "n_kv_heads": NKV, "head_dim": HD, "page_tokens": PG,
                   "n_pages": n_pages, "layers_rotated": n_layers, "kv_format": "kv%da16" % bits, "xcd_weight": xcd,
                   "step": "append 1 token/seq + paged decode attention (part, reduce with the open tile and the append in it)"},
        "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2), "tok_per_s": round(B / (ms * 1e-3), 1),
        "kv_bytes_per_step": int(kv_bytes), "parity_max_rel_err": float(f"{err:.3e}"), "parity_rows": rows,
        "out_fnv1a": first_hash,
        "roofline": {"bound": "hbm", "achieved": round(kgbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(kgbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC.get(a.workload, (None, None))[0],
                     "traffic_source": TRAFFIC.get(a.workload, (None, None))[1],
                     "kernel": "Kv8Part<%d, %d>" % (bits, bits), "kernel_ms": round(kern_ms, 4),
                     "kernel_ms_from": kern_how},
        "cpu_baseline": None}
    # the same number of steps again right after three idle seconds, without warm-up (see run_decode): an extra figure
    time.sleep(3.0)
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(1 + i)
    torch.cuda.synchronize()
    cold_ms = (time.perf_counter() - t0) / a.steps * 1e3
    res["after_idle"] = {"ms_per_step": round(cold_ms, 4), "GB/s": round(kv_bytes / (cold_ms * 1e-3) / 1e9, 1),
                         "note": "%d steps right after 3 idle seconds, no warm-up" % a.steps}
    return res


def run_prefill_kv8(a, wl, torch, yahkv):
    """The prefill step on kv8a16 pools: quantize + scatter the chunk (K rows around the sequence's channel means, V in
    16-key tiles), then one call that decodes prefix + chunk to f16 tile images and runs the causal attention."""
    B, chunk, prefix, PG = wl["batch"], wl["chunk"], wl["lo"], 256
    per_seq = (prefix + chunk + PG - 1) // PG
    bits = 4 if wl["fmt"] == 416 else 8
    g = yahkv.kv8_geometry(NQ, NKV, B * per_seq, bits, bits)
    alloc = yahkv.PagePool(g.n_pages)
    alloc.shuffle(12345)
    table = np.stack([alloc.alloc(per_seq) for _ in range(B)]).astype(np.int32)
    pools = yahkv.Kv8Pools(g)
    t_table = torch.from_numpy(table).cuda()
    gen = torch.Generator(device="cuda").manual_seed(wl["seed"])
    for s in range(B):
        for o in range(0, prefix, 8192):
            n = min(8192, prefix - o)
            k = (torch.randn((1, n, NKV, HD), generator=gen, device="cuda") + 0.5).to(torch.bfloat16)
            v = torch.randn((1, n, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            if o == 0:
                yahkv.kv8_kmean(pools, t_table[s:s + 1], k)
            yahkv.kv8_append(pools, t_table[s:s + 1], torch.tensor([o], dtype=torch.int32, device="cuda"), k, v)
    scale = 1.0 / float(np.sqrt(HD))
    t_prefix = torch.full((B,), prefix, dtype=torch.int32, device="cuda")
    q = torch.randn((B, chunk, NQ, HD), generator=gen, device="cuda").to(torch.bfloat16)
    knew = (torch.randn((B, chunk, NKV, HD), generator=gen, device="cuda") + 0.5).to(torch.bfloat16)
    vnew = torch.randn((B, chunk, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.empty(q.shape, dtype=torch.float16, device="cuda")
    ws = torch.empty(yahkv.lib.yahkv_kv8_prefill_workspace_bytes(g, B, prefix, chunk), dtype=torch.uint8, device="cuda")
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]

    def step(pair=None):
        yahkv.kv8_append(pools, t_table, t_prefix, knew, vnew)
        if pair:
            pair[0].record()
        yahkv.kv8_prefill_attend(pools, t_table, t_prefix, prefix, q, scale, out=out, workspace=ws)
        if pair:
            pair[1].record()

    # parity before timing: float64 closed form over the oracle's model of what the prefill kernels decode (f16 values)
    step()
    torch.cuda.synchronize()
    first_hash = fnv1a(out.view(torch.int16).cpu().numpy().tobytes())
    from oracle import kv8 as okv8
    n = prefix + chunk
    err = 0.0
    for s_ in (0, B - 1):
        hp, row = okv8.pools_of_sequence(pools, table[s_], n)
        Kd, Vd = okv8.dense(hp, row, n, as_f16=True)
        for t in (0, 1, chunk // 3, chunk // 2, chunk - 65, chunk - 1):
            for h in (0, 7, 13, NQ - 1):
                kv = h // (NQ // NKV)
                qv = q[s_, t, h].float().cpu().numpy()
                if bits == 4:                        # as the rotation kernel leaves it: H256 q / 16 rounded to f16
                    qv = okv8.rotate_q(qv).astype(np.float16)
                qv = qv.astype(np.float64)
                sc = Kd[:prefix + t + 1, kv].astype(np.float64) @ qv * scale
                p = np.exp(sc - sc.max())
                want = (p / p.sum()) @ Vd[:prefix + t + 1, kv].astype(np.float64)
                got = out[s_, t, h].float().cpu().numpy()
                err = max(err, float(np.abs(got - want).max() / np.abs(want).max()))
    if not err < 2e-3:
        raise SystemExit(f"bench.py: parity check failed before timing: max relative error {err:.3e}")
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(ev[i])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / a.steps * 1e3
    kern_ms = float(np.mean([p[0].elapsed_time(p[1]) for p in ev]))
    # (the chunk's rows go to the same places again: the pools stay as they are)
    app_ms = time_repeated(torch, lambda: yahkv.kv8_append(pools, t_table, t_prefix, knew, vnew))
    app_bytes = B * chunk * (2 * NKV * HD * 2 + (2336 if bits == 8 else 1408))   # bf16 rows in, codes + scales + stats out
    flops = float(B) * NQ * chunk * (prefix + (chunk + 1) / 2) * HD * 4
    return {
        "metric": "chunked-prefill attention over paged kv%da16 KV, TFLOP/s (f16 MFMA) + tok/s" % bits,
        "value": round(flops / (ms * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "prefix": prefix, "chunk": chunk, "n_q_heads": NQ,
                   "n_kv_heads": NKV, "head_dim": HD, "page_tokens": PG, "n_pages": g.n_pages, "kv_format": "kv%da16" % bits,
                   "step": "append chunk (quantize + scatter) + decode tiles to f16 + causal attention"},
        "tok_per_s": round(B * chunk / (ms * 1e-3), 1), "flops_per_step": int(flops),
        "parity_max_rel_err": float(f"{err:.3e}"), "out_fnv1a": first_hash,
        "append": {"kernel": "Kv8AppendChunk", "ms": round(app_ms, 4), "bytes": int(app_bytes),
                   "GB/s": round(app_bytes / (app_ms * 1e-3) / 1e9, 1),
                   "frac_of_hbm_peak": round(app_bytes / (app_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                   "note": "quantize + scatter of the chunk: %d calls back to back between one pair of HIP events" % APPEND_REPS},
        "roofline": {"bound": "mfma", "achieved": round(flops / (kern_ms * 1e-3) / 1e12, 1),
                     "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / (kern_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                     "traffic": TRAFFIC.get(a.workload, (None, None))[0],
                     "traffic_source": TRAFFIC.get(a.workload, (None, None))[1],
                     "kernel": ("Kv4RotateQ + " if bits == 4 else "") + "PrefillImagesKv8<0> + PrefillAttendImg<%d, 3, 1, 6>" % HD,
                     "kernel_ms": round(kern_ms, 4)},
        "cpu_baseline": None}


def run_prefill(a, wl, torch, yahkv):
    """A step: quantize + scatter one chunk per sequence, decode prefix + chunk to f16 tiles, causal attention."""
    g, layers, lens, table, t_table, gen = build_state(yahkv, torch, wl, 0)
    pools = layers[0]
    B, chunk, prefix = wl["batch"], wl["chunk"], int(lens.max())
    scale = 1.0 / float(np.sqrt(HD))
    t_prefix = torch.from_numpy(lens).cuda()
    q = torch.randn((B, chunk, NQ, HD), generator=gen, device="cuda").to(torch.bfloat16)
    knew = torch.randn((B, chunk, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    vnew = torch.randn((B, chunk, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.empty(q.shape, dtype=torch.float16, device="cuda")   # the reference's kernel writes f16 (gen_attn_fa.py:1589-1595)
    ws = torch.empty(yahkv.prefill_workspace_bytes(g, B, prefix, chunk), dtype=torch.uint8, device="cuda")
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]

    def step(pair=None):
        yahkv.append(pools, t_table, t_prefix, knew, vnew)
        if a.one_pass:                      # no workspace: the kernel that decodes each tile while staging it
            if pair:
                pair[0].record()
            yahkv.prefill_attend(pools, t_table, t_prefix, prefix, q, scale, out=out, workspace=False)
            if pair:
                pair[1].record()
            return
        yahkv.prefill_decode_tiles(pools, t_table, t_prefix, prefix, B, chunk, ws)
        if pair:
            pair[0].record()
        yahkv.prefill_attend_tiles(pools, t_table, t_prefix, prefix, q, scale, out, ws)
        if pair:
            pair[1].record()

    # parity before timing: float64 closed form on the library's own gathered blocks (exact arithmetic, nothing of the
    # matrix unit's f16 operands modelled), a few (query, head) rows of two sequences
    step()
    torch.cuda.synchronize()
    first_hash = fnv1a(out.view(torch.int16).cpu().numpy().tobytes())
    import oracle
    n = prefix + chunk
    err = 0.0
    for s_ in (0, B - 1):
        k, v = yahkv.gather_blocks(pools, t_table[s_], n)
        deq, bb = (oracle.dequantize_q8_0, 34) if wl["fmt"] == 8 else (oracle.dequantize_q4_0, 18)
        Kd = deq(k.cpu().numpy().reshape(-1, bb)).reshape(n, NKV, HD).astype(np.float64)
        Vd = deq(v.cpu().numpy().reshape(-1, bb)).reshape(n, NKV, HD).astype(np.float64)
        for t in (0, 1, chunk // 3, chunk // 2, chunk - 65, chunk - 1):
            for h in (0, 7, 13, NQ - 1):
                sc = Kd[:prefix + t + 1, h // (NQ // NKV)] @ q[s_, t, h].float().cpu().numpy().astype(np.float64) * scale
                p = np.exp(sc - sc.max())
                want = (p / p.sum()) @ Vd[:prefix + t + 1, h // (NQ // NKV)]
                got = out[s_, t, h].float().cpu().numpy()
                err = max(err, float(np.abs(got - want).max() / np.abs(want).max()))
    if not err < 2e-3:
        raise SystemExit(f"bench.py: parity check failed before timing: max relative error {err:.3e}")

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(ev[i])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = dt / a.steps * 1e3
    kern_ms = float(np.mean([p[0].elapsed_time(p[1]) for p in ev]))
    # (the chunk's rows go to the same places again: the pools stay as they are)
    app_ms = time_repeated(torch, lambda: yahkv.append(pools, t_table, t_prefix, knew, vnew))
    app_bytes = B * chunk * (2 * NKV * HD * 2 + 2 * NKV * (HD // 32) * (34 if wl["fmt"] == 8 else 18))   # bf16 rows in, blocks out
    flops = float(B) * NQ * chunk * (prefix + (chunk + 1) / 2) * HD * 4   # both products, causal part counted once
    res = {
        "metric": "chunked-prefill attention over paged q%d KV, TFLOP/s (f16 MFMA) + tok/s" % wl["fmt"],
        "value": round(flops / (ms * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "prefix": prefix, "chunk": chunk, "n_q_heads": NQ,
                   "n_kv_heads": NKV, "head_dim": HD, "page_tokens": PT, "n_pages": g.n_pages,
                   "kv_format": "q%d_0" % wl["fmt"],
                   "step": ("append chunk (quantize + scatter) + causal attention that decodes its tiles itself" if a.one_pass
                            else "append chunk (quantize + scatter) + decode tiles to f16 + causal attention")},
        "tok_per_s": round(B * chunk / (ms * 1e-3), 1), "flops_per_step": int(flops),
        "parity_max_rel_err": float(f"{err:.3e}"), "out_fnv1a": first_hash,
        "append": {"kernel": "AppendPages<%d, 2>" % wl["fmt"], "ms": round(app_ms, 4), "bytes": int(app_bytes),
                   "GB/s": round(app_bytes / (app_ms * 1e-3) / 1e9, 1),
                   "frac_of_hbm_peak": round(app_bytes / (app_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                   "note": "quantize + scatter of the chunk: %d calls back to back between one pair of HIP events" % APPEND_REPS},
        "roofline": {"bound": "mfma", "achieved": round(flops / (kern_ms * 1e-3) / 1e12, 1),
                     "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / (kern_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                     "traffic": None if a.one_pass else TRAFFIC.get(a.workload, (None, None))[0],
                     "traffic_source": None if a.one_pass else TRAFFIC.get(a.workload, (None, None))[1],
                     "kernel": ("PrefillAttendFused<%d, %d, %d>" % (wl["fmt"], HD, PT) if a.one_pass
                                else "PrefillAttendImg<%d, 3, 1, 6>" % HD), "kernel_ms": round(kern_ms, 4)},
    }
    if a.clock_trace:
        res["clock_trace"] = clock_trace(
            yahkv, torch, lambda: yahkv.prefill_attend_tiles(pools, t_table, t_prefix, prefix, q, scale, out, ws), n=24)
    if not a.no_cpu_baseline:
        res["cpu_baseline"] = prefill_cpu_baseline(wl, scale)
    return res


def run_prefill_f16(a, wl, torch, yahkv):
    """The prefill step on unquantized f16 pools: append the chunk, then one call that converts prefix + chunk to
    f16 tiles and runs the causal attention."""
    B, chunk, prefix = wl["batch"], wl["chunk"], wl["lo"]
    rng = np.random.default_rng(wl["seed"])
    per_seq = (prefix + chunk + PT - 1) // PT
    n_pages = B * per_seq
    g = yahkv.f16_geometry(NQ, NKV, HD, PT, n_pages)
    t_table = torch.from_numpy(rng.permutation(n_pages).astype(np.int32).reshape(B, per_seq)).cuda()
    pools = yahkv.F16Pools(g)
    gen = torch.Generator(device="cuda").manual_seed(wl["seed"])
    for s in range(B):
        for o in range(0, prefix, 8192):
            n = min(8192, prefix - o)
            k = torch.randn((1, n, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            v = torch.randn((1, n, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            yahkv.f16_append(pools, t_table[s:s + 1], torch.tensor([o], dtype=torch.int32, device="cuda"), k, v)
    scale = 1.0 / float(np.sqrt(HD))
    t_prefix = torch.full((B,), prefix, dtype=torch.int32, device="cuda")
    q = torch.randn((B, chunk, NQ, HD), generator=gen, device="cuda").to(torch.bfloat16)
    knew = torch.randn((B, chunk, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    vnew = torch.randn((B, chunk, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.empty(q.shape, dtype=torch.float16, device="cuda")
    ws = torch.empty(yahkv.lib.yahkv_f16_prefill_workspace_bytes(g, B, prefix, chunk), dtype=torch.uint8, device="cuda")
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]

    def step(pair=None):
        yahkv.f16_append(pools, t_table, t_prefix, knew, vnew)
        if pair:
            pair[0].record()
        yahkv.f16_prefill_attend(pools, t_table, t_prefix, prefix, q, scale, out=out, workspace=ws)
        if pair:
            pair[1].record()

    # parity before timing: float64 closed form over the pools' own f16 values, a few (query, head) rows of sequence 0
    step()
    torch.cuda.synchronize()
    first_hash = fnv1a(out.view(torch.int16).cpu().numpy().tobytes())
    n = prefix + chunk
    run = min(PT, 32)
    kp = pools.k.view(torch.float16).view(n_pages, NKV, HD // 16, PT, 16)
    vp = pools.v.view(torch.float16).view(n_pages, NKV, PT // run, HD, run)
    pg = t_table[0].long()
    Kd = kp[pg].permute(0, 3, 1, 2, 4).reshape(-1, NKV, HD)[:n].double().cpu().numpy()
    Vd = vp[pg].permute(0, 2, 4, 1, 3).reshape(-1, NKV, HD)[:n].double().cpu().numpy()
    err = 0.0
    for t in (0, chunk // 2, chunk - 1):
        for h in (0, NQ - 1):
            sc = Kd[:prefix + t + 1, h // (NQ // NKV)] @ q[0, t, h].double().cpu().numpy() * scale
            pr = np.exp(sc - sc.max())
            want = (pr / pr.sum()) @ Vd[:prefix + t + 1, h // (NQ // NKV)]
            got = out[0, t, h].float().cpu().numpy()
            err = max(err, float(np.abs(got - want).max() / np.abs(want).max()))
    if not err < 2e-3:
        raise SystemExit(f"bench.py: parity check failed before timing: max relative error {err:.3e}")
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(ev[i])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / a.steps * 1e3
    kern_ms = float(np.mean([p[0].elapsed_time(p[1]) for p in ev]))
    flops = float(B) * NQ * chunk * (prefix + (chunk + 1) / 2) * HD * 4
    return {
        "metric": "chunked-prefill attention over paged f16 KV, TFLOP/s (f16 MFMA) + tok/s",
        "value": round(flops / (ms * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "prefix": prefix, "chunk": chunk, "n_q_heads": NQ,
                   "n_kv_heads": NKV, "head_dim": HD, "page_tokens": PT, "n_pages": n_pages, "kv_format": "f16",
                   "step": "append chunk (f16 rounding + scatter) + f16 pages to tile images + causal attention"},
        "tok_per_s": round(B * chunk / (ms * 1e-3), 1), "flops_per_step": int(flops),
        "parity_max_rel_err": float(f"{err:.3e}"), "out_fnv1a": first_hash,
        "roofline": {"bound": "mfma", "achieved": round(flops / (kern_ms * 1e-3) / 1e12, 1),
                     "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / (kern_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                     "traffic": None, "traffic_source": None,
                     "kernel": "PrefillImagesF16<%d, %d> + PrefillAttendImg<%d, 3, 1, 6>" % (HD, PT, HD),
                     "kernel_ms": round(kern_ms, 4)},
        "cpu_baseline": None}


def run_decode(a, wl, torch, yahkv):
    """A step on quantized pools: one new token per sequence and the attention over the sequence with it. Two dispatches
    (yahkv_decode_step's): split-K partials over the tokens already in the pools, then the merge, which also quantizes
    the new token, writes it to its page and adds its term. --separate-append: three dispatches, the reference's order
    (append, partials, merge)."""
    total = a.warmup + 2 * a.steps + 1                # (the second set of steps: the ones timed after an idle period)
    g, layers, lens, table, t_table, gen = build_state(yahkv, torch, wl, total)
    pools = layers[0]
    B = wl["batch"]
    scale = 1.0 / float(np.sqrt(HD))
    max_len = int(lens.max()) + total
    # Lengths live on the device, one row per step, as the reference preloads its position array
    # (engine/model/loom_decoder.hpp:131-133): no kernel is spent on incrementing them.
    len_rows = torch.from_numpy(lens[None, :] + np.arange(total + 1, dtype=np.int32)[:, None]).cuda()
    q = torch.randn((B, NQ, HD), generator=gen, device="cuda").to(torch.bfloat16)
    knew = torch.randn((total, B, 1, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    vnew = torch.randn((total, B, 1, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.empty((B, NQ, HD), dtype=torch.float32, device="cuda")
    opt = yahkv.decode_options(one_launch=a.one_launch, deterministic=a.deterministic,
                               min_chunk_tiles=a.min_chunk_tiles, wg_partials=a.wg_partials, cut=a.cut)
    if a.first_come:
        opt.deterministic = -1
    ws = torch.empty(yahkv.decode_workspace_bytes(g, B, max_len, opt), dtype=torch.uint8, device="cuda")
    # which instance of the part kernel the library picks (its last template argument): 1 merges in the same launch,
    # 2 leaves one partial per workgroup for a chunk's last pair (the library's rule for a batch with few tiles per wave)
    chunks = torch.cuda.get_device_properties(0).multi_processor_count
    line = -(-max_len // 64) * B * NKV
    few_tiles = line <= chunks * 8 * 4
    # 3: the kernel of its own for q8_0 with at most two tiles per wave (DattnPartWhole: a wave asks for a whole tile at once)
    whole = a.wg_partials in (0, 3) and g.format == 8 and not a.one_launch and line <= chunks * 8 * 2
    part_mode = 1 if a.one_launch else 3 if whole else 2 if a.wg_partials in (1, 3) or (a.wg_partials == 0 and few_tiles) else 0
    # set-up, as a server does once: the XCDs' relative read speeds on this batch (equal shares without it)
    xcd = yahkv.decode_calibrate(pools, t_table, len_rows[0], max_len, q, ws, opt, rounds=3) if not a.no_calibrate else None
    if a.one_launch:
        yahkv.decode_workspace_init(g, B, max_len, ws, opt)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]
    separate = a.separate_append or a.one_launch

    # The step's two calls with their arguments marshalled once per step index, before anything is timed: the timed loop
    # then pays for the C calls alone, as a C++ caller does (building ctypes arguments from tensors costs Python about as
    # much as a small batch's whole step takes on the GPU).
    calls = None if separate else [
        yahkv.decode_step_calls(layers[i % len(layers)], t_table, len_rows[i], len_rows[i + 1], max_len, knew[i][:, 0],
                                vnew[i][:, 0], q, scale, out, ws, opt=opt) for i in range(total)]

    def step(i, pair=None, on=None):        # on: the handle of the stream a graph is being captured on
        seq_len = len_rows[i + 1]
        pools = layers[i % len(layers)]     # (with several layers a layer sees every n-th token; the others stay zero blocks)
        if not separate:
            part, merge = calls[i]
            if pair:
                pair[0].record()
            part(on) if on else part()      # the tokens before the step
            if pair:
                pair[1].record()
            merge(on) if on else merge()    # the step's own token, the partials' merge
            return
        yahkv.append(pools, t_table, len_rows[i], knew[i], vnew[i])    # position = current length (device-resident)
        if pair:
            pair[0].record()
        if not a.one_launch:                # the reference's form: partials, then their merge in a dispatch of its own
            yahkv.decode_part(pools, t_table, seq_len, max_len, q, scale, ws, opt=opt)
            if pair:
                pair[1].record()
            yahkv.decode_reduce(g, t_table.shape[1], seq_len, B, max_len, out, ws, opt=opt)
        else:                               # one launch: the split-K kernel's workgroups merge what they finish last
            yahkv.decode_attend(pools, t_table, seq_len, max_len, q, scale, out=out, workspace=ws, opt=opt)
            if pair:
                pair[1].record()

    # parity before timing: first step; the shortest, a quartile, the median and the longest sequence (the ones that span
    # the most chunks and XCD shares) against the float64 closed form
    step(0)
    torch.cuda.synchronize()
    first_hash = fnv1a(out.cpu().numpy().tobytes())
    order = np.argsort(lens)
    rows = sorted({int(order[0]), int(order[len(order) // 4]), int(order[len(order) // 2]), int(order[-1])})
    err = parity_check(yahkv, torch, g, pools, t_table, lens + 1, q, out, scale, rows)
    if not err < 2e-3:
        raise SystemExit(f"bench.py: parity check failed before timing: max relative error {err:.3e}")

    for i in range(a.warmup):
        step(1 + i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        # (the kernel's own duration is taken on every fourth timed step: a pair of event records costs the stream a few
        # microseconds, which the other steps are spared)
        step(1 + a.warmup + i, ev[i] if i % EVENT_EVERY == 0 else None)
    t_issued = time.perf_counter()          # (what the host took to queue the steps: below the step's time, or its bound)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0

    bpt = yahkv.lib.yahkv_bytes_per_token(g)
    # context lengths seen by timed step i: lens + 1 (parity step) + warmup + i + 1
    tokens = [int(lens.sum()) + B * (2 + a.warmup + i) for i in range(a.steps)]
    kv_bytes = float(np.mean(tokens)) * bpt
    ms = dt / a.steps * 1e3
    kern_ms = float(np.mean([p[0].elapsed_time(p[1]) for p in ev[::EVENT_EVERY]]))
    kern_how = "HIP events around the part kernel of every %d-th timed step" % EVENT_EVERY
    if kern_ms < 0.1 and calls is not None:
        # A pair of events around one launch adds about 6 us of its own, a quarter of a small batch's part kernel: the
        # timed steps' part launches again, one behind the other between a single pair of events (they only write
        # partials; the layers rotate as in the steps, so nothing is read from a cache a step would not find it in).
        it = iter(range(a.steps))
        kern_ms = time_repeated(torch, lambda: calls[1 + a.warmup + next(it, 0)][0](), reps=a.steps - 1)
        kern_how = "the timed steps' part launches back to back between one pair of HIP events"
    gbs = kv_bytes / (ms * 1e-3) / 1e9
    # (in the two-dispatch step the split-K kernel runs over the tokens before the step's own: one fewer per sequence)
    kgbs = (kv_bytes - (0 if separate else B * bpt)) / (kern_ms * 1e-3) / 1e9
    res = {
        "metric": ("paged q8 KV decode-attn HBM GB/s (% of peak) + tok/s, B=64 ragged ctx"
                   if a.workload == "ragged_b64_q8_0" else
                   "paged q%d KV decode-attn HBM GB/s (%% of peak) + tok/s" % wl["fmt"]),
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "host_issue_ms_per_step": round((t_issued - t0) / a.steps * 1e3, 4),
        "dtype": "u8" if wl["fmt"] == 8 else "u4", "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "ctx_min": int(lens.min()), "ctx_max": int(lens.max()),
                   "ctx_sum": int(lens.sum()), "n_q_heads": NQ, "n_kv_heads": NKV, "head_dim": HD, "page_tokens": PT,
                   "n_pages": g.n_pages, "layers_rotated": len(layers), "kv_format": "q8_0" if wl["fmt"] == 8 else "q4_0",
                   "step": "append 1 token/seq + paged decode attention (%s)" %
                           ("append, one launch for part and merge" if a.one_launch else
                            "append, part, reduce" if separate else "part, reduce with the append in it"),
                   "xcd_weight": xcd},
        "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2), "tok_per_s": round(B / (ms * 1e-3), 1),
        "kv_bytes_per_step": int(kv_bytes), "parity_max_rel_err": float(f"{err:.3e}"), "out_fnv1a": first_hash,
        "roofline": {"bound": "hbm", "achieved": round(kgbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(kgbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC.get(a.workload, (None, None))[0],
                     "traffic_source": TRAFFIC.get(a.workload, (None, None))[1],
                     "kernel": "DattnPartWhole" if part_mode == 3 else "DattnPart<%d, %d, %d, %d>" % (wl["fmt"], HD, PT, part_mode),
                     "kernel_ms": round(kern_ms, 4), "kernel_ms_from": kern_how},
    }
    # The same number of steps again, right after three idle seconds and without warm-up: what a server's first steps
    # after a pause cost (the shader clock dips for some tens of milliseconds then; kernels bound by HBM hardly notice,
    # the q4_0 kernel does). An extra figure, not `value`.
    time.sleep(3.0)
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(1 + a.warmup + a.steps + i)
    torch.cuda.synchronize()
    cold_ms = (time.perf_counter() - t0) / a.steps * 1e3
    res["after_idle"] = {"ms_per_step": round(cold_ms, 4), "GB/s": round(kv_bytes / (cold_ms * 1e-3) / 1e9, 1),
                         "note": "%d steps right after 3 idle seconds, no warm-up" % a.steps}
    if a.clock_trace:
        last = a.warmup + a.steps + 1
        res["clock_trace"] = clock_trace(
            yahkv, torch, lambda: yahkv.decode_part(pools, t_table, len_rows[last], max_len, q, scale, ws, opt=opt))
    if a.graph_replay:
        # The same timed steps (same tokens at the same positions: the pools end up as they are) recorded once into
        # a HIP graph, so the launches follow each other without the host in between; an extra figure, not `value`.
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                on = ctypes.c_void_p(side.cuda_stream)
                for i in range(a.steps):
                    step(1 + a.warmup + i, on=on)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) / a.steps * 1e3)
        gms = float(np.median(times))
        res["graph_replay"] = {"ms_per_step": round(gms, 4), "GB/s": round(kv_bytes / (gms * 1e-3) / 1e9, 1),
                               "tok_per_s": round(B / (gms * 1e-3), 1),
                               "note": "the timed steps replayed as one HIP graph, median of 5 replays"}
    if not a.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(wl, lens, scale)
    return res


def run_workload(a, torch, yahkv):
    wl = WORKLOADS[a.workload]
    if "chunk" in wl and wl["fmt"] == 16:
        return run_prefill_f16(a, wl, torch, yahkv)
    if "chunk" in wl and wl["fmt"] in (816, 416):
        return run_prefill_kv8(a, wl, torch, yahkv)
    if "chunk" in wl:
        return run_prefill(a, wl, torch, yahkv)
    if wl["fmt"] == 16:
        return run_f16(a, wl, torch, yahkv)
    if wl["fmt"] in (816, 416):
        return run_kv8(a, wl, torch, yahkv)
    return run_decode(a, wl, torch, yahkv)


# what the default run times besides its own workload: the other configurations of the benchmark that fill a GPU
ALSO = ["b1_ctx32k_q8_0", "prefill_b8_ctx16k_chunk2k_q8_0", "b16_ctx128k_q4_0", "ragged_b64_kv8a16", "ragged_b64_kv4a16",
        "ragged_b64_f16", "prefill_b8_ctx16k_chunk2k_q4_0"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps before the timed ones (default: 3, or what the workload names)")
    ap.add_argument("--workload", default="ragged_b64_q8_0", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-also", action="store_true",
                    help="default workload only: do not time the other configurations for the line's `also` object")
    ap.add_argument("--no-calibrate", action="store_true", help="decode workloads: equal chunk shares for all XCDs")
    ap.add_argument("--deterministic", action="store_true", help="decode workloads: the default (fixed tile pattern per wave)")
    ap.add_argument("--first-come", action="store_true",
                    help="decode workloads: opt.deterministic = -1, a workgroup's tiles handed out first come, first served "
                         "(results then differ in their last bits from run to run)")
    ap.add_argument("--one-launch", action="store_true",
                    help="decode workloads: yahkv_decode_attend with opt.one_launch instead of part + reduce")
    ap.add_argument("--one-pass", action="store_true",
                    help="quantized prefill workloads: no workspace, the attention kernel decodes its tiles itself")
    ap.add_argument("--min-chunk-tiles", type=int, default=0,
                    help="decode workloads: yahkv_decode_options::min_chunk_tiles (0: the library's default)")
    ap.add_argument("--wg-partials", type=int, default=0, choices=[0, 1, 2, 3],
                    help="q8_0 / q4_0 decode workloads: yahkv_decode_options::wg_partials (1: one partial per workgroup for a "
                         "chunk's last pair, 2: one per wave, 3: one per workgroup from waves that ask for whole tiles, "
                         "0: chosen from the batch's size)")
    ap.add_argument("--cut", type=int, default=0, choices=[0, 1, 2],
                    help="q8_0 / q4_0 decode workloads: yahkv_decode_options::cut (1: by (sequence, kv head), 2: by "
                         "(sequence, tile) with the kv heads of a tile on neighbouring waves, 0: the library's choice)")
    ap.add_argument("--separate-append", action="store_true",
                    help="decode workloads: the step's token is appended by a dispatch of its own (three per step)")
    ap.add_argument("--clock-trace", action="store_true",
                    help="also: after the timing and three idle seconds, launches of the dominant kernel back to back with "
                         "the shader clock after each (quantized decode and prefill workloads)")
    ap.add_argument("--graph-replay", action="store_true",
                    help="decode workloads: also replay the timed steps as one HIP graph and report its time per step")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run plain device copies of 1 GiB (to scale rocprofv3's FETCH_SIZE / WRITE_SIZE)")
    a = ap.parse_args()
    if a.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU (the path has no cross-GPU exchange); use --gpus 1")
    import torch
    yahkv = importlib.import_module("yet-another-halo-engine_amd")
    torch.cuda.set_device(0)
    if a.copy_calibration:
        src = torch.ones(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"bytes_read": 1 << 30, "bytes_written": 1 << 30, "copies": 5}}))
        return
    asked_warmup = a.warmup
    headline = a.workload
    a.warmup = asked_warmup if asked_warmup is not None else WORKLOADS[headline].get("warmup", 3)
    if headline == "ragged_b64_q8_0" and not a.no_also:
        a.graph_replay = True   # the default run also says what its steps take as one HIP graph (an extra figure)
    res = run_workload(a, torch, yahkv)
    if headline == "ragged_b64_q8_0" and not a.no_also:
        # the other configurations, timed by the same run with their own default warm-up, a short record each
        res["also"] = {}
        for name in ALSO:
            torch.cuda.empty_cache()
            sub = argparse.Namespace(**vars(a))
            sub.workload, sub.graph_replay, sub.no_cpu_baseline = name, "chunk" not in WORKLOADS[name], True
            sub.warmup, sub.clock_trace = WORKLOADS[name].get("warmup", 3), False
            r = run_workload(sub, torch, yahkv)
            keep = ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "tok_per_s", "parity_max_rel_err", "roofline",
                    "graph_replay", "after_idle", "append", "pct_of_hbm_peak", "out_fnv1a")
            res["also"][name] = {k: r[k] for k in keep if k in r}
    print(json.dumps(res))


if __name__ == "__main__":
    main()
