#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

One "step" is one pass of decode attention over the KV caches of all 30 layers
of a Gemma3n-E2B-shaped model at 4096 context (config 3 of BASELINE.json:
batch 1, 8 query heads / 2 KV heads, head_dim 256, fp16 cache, 16 split-KV
partitions merged by log-sum-exp), issued as one multi-layer launch plus the
merge pass. A single layer is only 8 MiB and would sit in cache, so each step
streams a different set of 30 layer caches out of 4 (1 GiB in total): reads
come from HBM, not from L2 / Infinity Cache.

Prints ONE JSON line. `value` is algorithmic bytes per step / wall time per
step with all inputs resident in HBM. Every leg is timed over a region of at
least 50 ms whatever --steps says (`timed_steps` says how many steps that
took). `sustained` repeats the headline step (and, under `prefill`, the config-2
launch) back to back for 2 s. `roofline` prices the decode attention kernel alone (begin / end stamps
attached to each dispatch, on the stream it runs on) against the 8 TB/s HBM
peak. `decode_graph` replays the same work from HIP graphs: the one multi-layer
launch, and the 30 layers as 30 launches in dependency order (what a forward
pass over a model issues). `prefill` is the 26-layer, 1024-token bf16 prefill of
config 2 in one launch, priced against the 2.5 PFLOP/s dense bf16 MFMA peak.
`cpu_baseline` times the C restatement of the reference CPU op order
(oracle/attn_oracle.c) on a bounded sample of the same decode workload.
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

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
D = 256
METRIC = "decode-attn HBM GB/s (% of 8 TB/s) + prefill-attn TFLOP/s, Gemma3n-E2B shape"
MIN_TIMED_REGION_S = 0.05
SUSTAINED_S = 2.0  # the headline step and the config-2 prefill launch are also run back to back for this long


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def rounded(d):
    return {k: (round(v, 4) if isinstance(v, float) else v) for k, v in d.items()}


def time_steps(torch, step_fn, steps, warmup, min_region_s=MIN_TIMED_REGION_S):
    """Seconds per step over a timed region of at least `min_region_s`: after `warmup` untimed steps a short
    probe sizes the region, then max(steps, what fills the region) steps are queued back to back between
    two synchronisations. Returns (seconds per step, steps timed)."""
    for i in range(warmup):
        step_fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(8):
        step_fn(warmup + i)
    torch.cuda.synchronize()
    est = max((time.perf_counter() - t0) / 8, 1e-7)
    timed = max(steps, int(min_region_s / est) + 1)
    t0 = time.perf_counter()
    for i in range(timed):
        step_fn(warmup + 8 + i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / timed, timed


def kernel_ms(torch, handle, step_fn, first, bursts=6, burst=32):
    """Duration of the kernel itself (begin / end stamps attached to the dispatch) in the steady state of
    back-to-back launches, and the time per step of the very bursts the stamps are read in (stream events
    around each burst): the stamps of each burst's last launch are read. Returns (kernel ms, ms per step of
    those bursts)."""
    handle.set_timing(True)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    total, span, i = 0.0, 0.0, first
    for _ in range(bursts):
        e0.record()
        for _ in range(burst):
            step_fn(i)
            i += 1
        e1.record()
        total += handle.last_kernel_ms()
        e1.synchronize()
        span += e0.elapsed_time(e1) / burst
    handle.set_timing(False)
    return total / bursts, span / bursts


def read_floor_ms(torch, at, nbytes, workgroups, waves, cache_bytes, bursts=4, burst=16):
    """Duration (dispatch stamps) of a launch that only streams `nbytes` of the handle's cache with the decode
    kernel's load pattern through `workgroups` x `waves` waves (mi355_attn_stream_probe), rotating through the
    cache so that nothing is resident: the floor a decode launch of those bytes and that shape is priced against."""
    span = (nbytes // (workgroups * waves) + 32767) // 32768 * 32768 * workgroups * waves
    slots = max(1, cache_bytes // span)
    at.set_timing(True)
    total, i = 0.0, 0
    for _ in range(bursts):
        for _ in range(burst):
            at.stream_probe((i % slots) * span, nbytes, workgroups, waves)
            i += 1
        total += at.last_kernel_ms()
    at.set_timing(False)
    return total / bursts


def load_traffic(key):
    """HBM bytes per launch of a benchmarked kernel as last measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    (each scaled by what the same counter reads for a plain copy of known size): profiles/traffic.json holds the
    figures and the commands that produced them. None when the file has no entry."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(key, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def fill_cache(at, torch, layers, seqs_lens, hkv, dtype, seed):
    """Appends N(0,1) rows (generated on the GPU) to every (layer, sequence)."""
    g = torch.Generator(device="cuda:0").manual_seed(seed)
    for layer in range(layers):
        for seq, n in enumerate(seqs_lens):
            k = torch.randn((n, hkv, D), generator=g, device="cuda:0", dtype=torch.float32).to(dtype)
            v = torch.randn((n, hkv, D), generator=g, device="cuda:0", dtype=torch.float32).to(dtype)
            at.kv_append(layer, seq, 0, k, v)


# ---------------------------------------------------------------------------------------------- decode
def bench_decode_c3(A, torch, steps, warmup, layers=30, rotation=4, splits=16, ctx=4096):
    """Config 3 x 30 layers. Runs on a stream of its own so that the same calls can be captured into HIP graphs."""
    hq, hkv = 8, 2
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        at = A.Attn(layers * rotation, hq, hkv, D, ctx, 1, A.F16, A.F16, stream=side.cuda_stream)
        fill_cache(at, torch, layers * rotation, [ctx], hkv, torch.float16, seed=0xC0FFEE + 2)
        q = torch.randn((rotation, layers, 1, hq, D), device="cuda:0", dtype=torch.float32).half()
        out = torch.empty_like(q)
        lens = A._i32_array([ctx])

        def step(i):
            r = i % rotation
            at.decode(r * layers, lens, q[r], out[r], num_splits=splits, n_layers=layers, batch=1)

        sec, timed = time_steps(torch, step, steps, warmup)
        kms, burst_ms = kernel_ms(torch, at, step, 0)
        # the same steps back to back for SUSTAINED_S seconds: the rate at the clocks and the memory state the part
        # settles into under this load (the 50 ms regions above end before it does)
        sec_long, timed_long = time_steps(torch, step, steps, 0, min_region_s=SUSTAINED_S)
        # algorithmic bytes: K and V once, Q and O once (no partials, no padding)
        per_layer = ctx * hkv * D * 2 * 2 + 2 * hq * D * 2
        step_bytes = per_layer * layers
        floor_ms = read_floor_ms(torch, at, step_bytes, layers * hkv * splits, 1, at.cache_bytes)

        def step1(i):  # single layer, cache resident: latency figure only
            at.decode(0, lens, q[0, 0], out[0, 0], num_splits=splits, batch=1)
        lat, _ = time_steps(torch, step1, 200, 20)

        # The same work replayed from HIP graphs (no allocation happens inside a captured call: the split-KV
        # workspace exists since the eager steps above). One graph per cache set, replayed in turn.
        def capture(fn):
            graphs = []
            for r in range(rotation):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    fn(r)
                graphs.append(g)
            return graphs

        def one_launch(r):
            at.decode(r * layers, lens, q[r], out[r], num_splits=splits, n_layers=layers, batch=1)

        def per_layer_chain(r):  # layer l + 1 of a forward pass needs layer l's output: one launch (+ merge) per layer, in order
            for layer in range(layers):  # (partition count by the library's own rule for a one-layer launch)
                at.decode(r * layers + layer, lens, q[r, layer], out[r, layer], num_splits=0, batch=1)

        sec_chain_eager, _ = time_steps(torch, lambda i: per_layer_chain(i % rotation), steps, 2)
        graph = {}
        try:
            for r in range(rotation):
                one_launch(r)
            torch.cuda.synchronize()
            want = out.clone()
            g1 = capture(one_launch)
            sec_g1, _ = time_steps(torch, lambda i: g1[i % rotation].replay(), steps, warmup)
            ok1 = bool(torch.equal(out, want))
            out.zero_()
            g30 = capture(per_layer_chain)
            sec_g30, _ = time_steps(torch, lambda i: g30[i % rotation].replay(), steps, warmup)
            # (one-layer launches merge four waves per workgroup through LDS, the 30-layer launch runs one wave per
            # workgroup: another summation order, so the two agree to rounding, not bit for bit)
            ok30 = bool((out.float() - want.float()).abs().max().item() <= 2e-3 * want.float().abs().max().item())
            graph = {
                "what": "the headline step replayed from HIP graphs (captured calls of the same C ABI, one graph per cache "
                        "set): `one_launch` = the multi-layer launch + merge; `per_layer_chain` = the 30 layers as 30 "
                        "launches (+ merges) in dependency order, the shape a forward pass over a model issues",
                "one_launch": {"us_per_step": round(sec_g1 * 1e6, 2), "GBps": round(step_bytes / sec_g1 / 1e9, 1),
                               "frac_of_hbm_peak": round(step_bytes / sec_g1 / 1e9 / HBM_PEAK_GBS, 4),
                               "equals_eager_output": ok1},
                "per_layer_chain": {"us_per_step": round(sec_g30 * 1e6, 2), "GBps": round(step_bytes / sec_g30 / 1e9, 1),
                                    "frac_of_hbm_peak": round(step_bytes / sec_g30 / 1e9 / HBM_PEAK_GBS, 4),
                                    "us_per_layer": round(sec_g30 * 1e6 / layers, 2), "matches_one_launch_output": ok30},
                "per_layer_chain_eager": {"us_per_step": round(sec_chain_eager * 1e6, 2),
                                          "GBps": round(step_bytes / sec_chain_eager / 1e9, 1)},
            }
            del g1, g30
        except Exception as e:  # a graph leg that cannot run is reported, never hidden
            graph = {"error": f"{type(e).__name__}: {e}"}
        torch.cuda.synchronize()
        at.close()
    return {"sec_per_step": sec, "timed_steps": timed, "kernel_ms": kms, "burst_ms_per_step": burst_ms,
            "sustained_sec_per_step": sec_long, "sustained_steps": timed_long, "floor_ms": floor_ms,
            "step_bytes": step_bytes, "layers": layers, "single_layer_latency_us": lat * 1e6,
            "tokens_per_s": 1.0 / sec, "graph": graph}


def bench_decode_batch(A, torch, name, kv, lens, steps, warmup, rotation, splits, layers=1):
    """Batched decode (configs 4 and 5): `layers` layers per launch, rotating over `rotation` sets of them."""
    hq, hkv = 8, 2
    B = len(lens)
    stream = torch.cuda.current_stream().cuda_stream
    at = A.Attn(rotation * layers, hq, hkv, D, 4096, B, kv, A.F16, stream=stream)
    g = torch.Generator(device="cuda:0").manual_seed(0xC0FFEE + (3 if kv == A.F16 else 4))
    for layer in range(rotation * layers):
        for b, n in enumerate(lens):
            if kv == A.I8:
                k = torch.randint(-127, 128, (n, hkv, D), generator=g, device="cuda:0", dtype=torch.int8)
                v = torch.randint(-127, 128, (n, hkv, D), generator=g, device="cuda:0", dtype=torch.int8)
                sc = torch.rand((hkv, D), generator=g, device="cuda:0") * 0.02 + 0.02
                at.kv_set_scales(layer, b, sc, sc)
            else:
                k = torch.randn((n, hkv, D), generator=g, device="cuda:0").half()
                v = torch.randn((n, hkv, D), generator=g, device="cuda:0").half()
            at.kv_append(layer, b, 0, k, v)
    q = torch.randn((layers, B, hq, D), device="cuda:0").half()
    out = torch.empty_like(q)
    clens = A._i32_array(lens)

    def step(i):
        at.decode((i % rotation) * layers, clens, q, out, num_splits=splits, n_layers=layers, batch=B)

    sec, timed = time_steps(torch, step, steps, warmup)
    kms, _ = kernel_ms(torch, at, step, 0, bursts=4, burst=16 if layers == 1 else 4)
    esz = 1 if kv == A.I8 else 2
    nbytes = layers * (sum(lens) * hkv * D * 2 * esz + 2 * B * hq * D * 2 + (B * 2 * hkv * D * 4 if kv == A.I8 else 0))
    # the floor: the same bytes through as many one-wave workgroups as the launch has partitions that hold keys
    out_row = {"workload": name, "ms_per_step": sec * 1e3, "timed_steps": timed, "kernel_ms": kms, "bytes": nbytes,
               "GBps": nbytes / sec / 1e9, "kernel_GBps": nbytes / (kms * 1e-3) / 1e9,
               "frac_of_hbm_peak": nbytes / (kms * 1e-3) / 1e9 / HBM_PEAK_GBS, "tokens_per_s": B / sec}
    if layers == 1 and splits > 0:
        per = -(-(-(-max(lens) // splits)) // 64) * 64
        wgs = sum(-(-n // per) for n in lens) * hkv
        floor = read_floor_ms(torch, at, nbytes, wgs, 1, at.cache_bytes)
        out_row.update({"read_floor_ms": floor, "frac_of_read_floor": floor / kms, "read_floor_workgroups": wgs})
    at.close()
    return out_row


def bench_decode_c1(A, torch, steps, warmup):
    """Config 1: fp32 cache, one sequence of 1024 tokens, Hq4/Hkv1, one layer
    (2 MiB: a latency figure, the cache stays in L2)."""
    hq, hkv, ctx = 4, 1, 1024
    stream = torch.cuda.current_stream().cuda_stream
    at = A.Attn(1, hq, hkv, D, ctx, 1, A.F32, A.F32, stream=stream)
    fill_cache(at, torch, 1, [ctx], hkv, torch.float32, seed=0xC0FFEE)
    q = torch.randn((1, hq, D), device="cuda:0")
    out = torch.empty_like(q)
    lens = A._i32_array([ctx])

    def step(i):
        at.decode(0, lens, q, out, num_splits=0, batch=1)

    sec, timed = time_steps(torch, step, steps, warmup)
    kms, _ = kernel_ms(torch, at, step, 0, bursts=4, burst=16)
    at.close()
    nbytes = ctx * hkv * D * 2 * 4 + 2 * hq * D * 4
    return {"workload": "C1: 1 seq x 1024, Hq4/Hkv1, fp32, one layer, cache-resident (latency)",
            "ms_per_step": sec * 1e3, "timed_steps": timed, "kernel_ms": kms, "bytes": nbytes, "GBps": nbytes / sec / 1e9,
            "kernel_GBps": nbytes / (kms * 1e-3) / 1e9, "tokens_per_s": 1.0 / sec}


# ---------------------------------------------------------------------------------------------- prefill
def prefill_flops(n, hq, window):
    pairs = sum(min(i + 1, window) if window > 0 else i + 1 for i in range(n))
    return 4 * hq * D * pairs


def bench_prefill_c2(A, torch, steps, warmup, layers=26, n=1024, half=False, by_layer=False, rows16=-1, sustained=False):
    hq, hkv = 4, 1
    windows = [0 if (l + 1) % 6 == 0 else 512 for l in range(layers)]
    stream = torch.cuda.current_stream().cuda_stream
    dt, tdt = (A.F16, torch.float16) if half else (A.BF16, torch.bfloat16)
    at = A.Attn(layers, hq, hkv, D, n, 1, dt, dt, layer_window=windows, stream=stream)
    at.set_option("prefill_rows16", rows16)
    fill_cache(at, torch, layers, [n], hkv, tdt, seed=0xC0FFEE + 1)
    q = torch.randn((layers, n, hq, D), device="cuda:0").to(tdt)
    out = torch.empty_like(q)

    def step(i):
        at.prefill(0, 0, 0, n, q, out, n_layers=layers)

    sec, timed = time_steps(torch, step, steps, warmup)
    kms, burst_ms = kernel_ms(torch, at, step, 0)
    flops = sum(prefill_flops(n, hq, w) for w in windows)
    sec_long, timed_long = time_steps(torch, step, steps, 0, min_region_s=SUSTAINED_S) if sustained else (float("nan"), 0)

    def step1(i):
        at.prefill(5, 0, 0, n, q[5], out[5])  # one global layer
    lat1, _ = time_steps(torch, step1, 50, 5)

    def step_layers(i):  # the way an executor calls it: one launch per layer, in turn
        for layer in range(layers):
            at.prefill(layer, 0, 0, n, q[layer], out[layer])
    per_layer = lat1_whole = per_layer_whole = float("nan")
    if by_layer:
        per_layer, _ = time_steps(torch, step_layers, 10, 2)
        at.set_option("prefill_key_split", 0)
        lat1_whole, _ = time_steps(torch, step1, 50, 5)
        per_layer_whole, _ = time_steps(torch, step_layers, 10, 2)
    at.close()
    return {"workload": f"C2: 26 layers x 1024 tokens, Hq4/Hkv1, {'fp16' if half else 'bf16'}, "
                        "22 local(W=512)+4 global, one launch",
            "ms_per_step": sec * 1e3, "timed_steps": timed, "kernel_ms": kms, "burst_ms_per_step": burst_ms,
            "flops": flops, "TFLOPs": flops / sec / 1e12, "sustained_sec_per_step": sec_long, "sustained_steps": timed_long,
            "kernel_TFLOPs": flops / (kms * 1e-3) / 1e12,
            "frac_of_mfma_peak": flops / (kms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
            "tokens_per_s": n / sec, "single_global_layer_ms": lat1 * 1e3,
            "single_global_layer_unsplit_ms": lat1_whole * 1e3,
            "layer_by_layer_ms": per_layer * 1e3, "layer_by_layer_unsplit_ms": per_layer_whole * 1e3,
            "dense_counted_TFLOPs": layers * 4 * hq * D * n * n / sec / 1e12}


def bench_prefill_int8(A, torch, steps, warmup, layers, n, q_pos0, hq, hkv, windows=None):
    """Prefill over an int8 cache: the call as it runs by default (the planes it reads staged as half planes, then
    the matrix-core kernels of a half cache) beside the row-wise path (every query row a decode item, converted in
    registers). Whole calls, staging included; the FLOPs are those of the visible (query, key) pairs."""
    windows = windows or [0] * layers
    ctx = q_pos0 + n
    stream = torch.cuda.current_stream().cuda_stream
    at = A.Attn(layers, hq, hkv, D, ctx, 1, A.I8, A.F16, layer_window=windows, stream=stream)
    g = torch.Generator(device="cuda:0").manual_seed(0xC0FFEE + 9)
    for layer in range(layers):
        k = torch.randint(-127, 128, (ctx, hkv, D), generator=g, device="cuda:0", dtype=torch.int8)
        v = torch.randint(-127, 128, (ctx, hkv, D), generator=g, device="cuda:0", dtype=torch.int8)
        at.kv_append(layer, 0, 0, k, v)
        at.kv_set_scales(layer, 0, torch.rand((hkv, D), generator=g, device="cuda:0") * 0.02 + 0.005,
                         torch.rand((hkv, D), generator=g, device="cuda:0") * 0.02 + 0.005)
    q = torch.randn((layers, n, hq, D), device="cuda:0").half()
    out = torch.empty_like(q)

    def step(i):
        at.prefill(0, 0, q_pos0, n, q, out, n_layers=layers)

    flops = 0
    for w in windows:
        pairs = sum(min(q_pos0 + i + 1, w) if w > 0 else q_pos0 + i + 1 for i in range(n))
        flops += 4 * hq * D * pairs
    sec, timed = time_steps(torch, step, steps, warmup)
    kms, _ = kernel_ms(torch, at, step, 0)
    at.set_option("rowwise_prefill", 1)
    sec_row, _ = time_steps(torch, step, max(3, steps // 4), 2)
    kms_row, _ = kernel_ms(torch, at, step, 0, bursts=2, burst=8)
    at.close()
    return {"ms_per_step": sec * 1e3, "timed_steps": timed, "flops": flops, "TFLOPs": flops / sec / 1e12,
            "call_us_device": kms * 1e3, "device_TFLOPs": flops / (kms * 1e-3) / 1e12,
            "rowwise_ms_per_step": sec_row * 1e3, "rowwise_TFLOPs": flops / sec_row / 1e12,
            "rowwise_kernel_us": kms_row * 1e3, "rowwise_kernel_TFLOPs": flops / (kms_row * 1e-3) / 1e12}


def gemm_probe(torch, n=8192, reps=20):
    """Dense bf16 GEMM through the vendor library: what the matrix cores of this
    very card sustain next to the published peak the roofline is priced on."""
    a = torch.randn((n, n), device="cuda:0").bfloat16()
    b = torch.randn((n, n), device="cuda:0").bfloat16()
    for _ in range(3):
        torch.matmul(a, b)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        torch.matmul(a, b)
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / reps
    return 2 * n ** 3 / sec / 1e12


# ---------------------------------------------------------------------------------------------- the steps either side
def bench_sampler(S, torch, steps, warmup, batch=64, vocab=262144, k=64, p=0.95, rotation=8):
    """Token sampling right after the attention path: [batch, vocab] float32 logits in HBM ->
    one id per row (top-k 64, top-p 0.95). Rotates over `rotation` logits tensors (512 MiB)."""
    stream = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device="cuda:0").manual_seed(0xC0FFEE + 7)
    logits = [torch.randn((batch, vocab), generator=g, device="cuda:0") * 3.0 for _ in range(rotation)]
    ids = torch.zeros((batch,), dtype=torch.int32, device="cuda:0")
    with S.Sampler(k, p, 1.0, batch, 1, vocab, stream=stream) as s:
        def step(i):
            s.sample_to_id_and_score_buffer(logits[i % rotation], ids)
        sec, timed = time_steps(torch, step, steps, warmup)
        kms, _ = kernel_ms(torch, s, step, 0, bursts=4, burst=8)
    with S.Sampler(k, p, 1.0, 1, 1, vocab, stream=stream) as s1:
        one = logits[0][:1].contiguous()
        id1 = torch.zeros((1,), dtype=torch.int32, device="cuda:0")
        lat, _ = time_steps(torch, lambda i: s1.sample_to_id_and_score_buffer(one, id1), 200, 20)
    nbytes = batch * vocab * 4
    return {"workload": f"sampling: {batch} rows x {vocab} float32 logits, top-k {k}, top-p {p}, one launch",
            "ms_per_step": sec * 1e3, "timed_steps": timed, "kernel_ms": kms, "bytes": nbytes, "GBps": nbytes / sec / 1e9,
            "kernel_GBps": nbytes / (kms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (kms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "tokens_per_s": batch / sec, "single_row_latency_us": lat * 1e6}


def bench_pre_attention(A, torch, steps, warmup, layers=26, n=1024, hq=4, hkv=1):
    """The step before attention at config 2's shape: per layer one launch that RMS-normalises
    and rotates the chunk's q / k rows and writes k / v into the cache planes (bf16). Every
    step takes the next layer (its own inputs and planes), as a forward pass does."""
    dt = torch.bfloat16
    g = torch.Generator(device="cuda:0").manual_seed(0xC0FFEE + 8)
    mk = lambda heads: [torch.randn((n, heads, D), generator=g, device="cuda:0").to(dt) for _ in range(layers)]
    q, k, v = mk(hq), mk(hkv), mk(hkv)
    q_out = torch.zeros_like(q[0])
    rng = np.random.default_rng(0xC0FFEE + 8)
    d = np.arange(0, D, 2, dtype=np.float64) / D
    with A.Attn(layers, hq, hkv, D, n, 1, A.BF16, A.BF16, stream=torch.cuda.current_stream().cuda_stream) as at:
        for layer in range(layers):
            theta = 1000000.0 if (layer + 1) % 6 == 0 else 10000.0
            at.set_layer_transform(layer, norm_q=True, norm_k=True,
                                   q_weight=(rng.standard_normal(D) * 0.1).astype(np.float32),
                                   k_weight=(rng.standard_normal(D) * 0.1).astype(np.float32), eps=1e-6,
                                   weight_offset=1.0, rope_inv_freq=(theta ** -d).astype(np.float32))

        def step(i):
            layer = i % layers
            at.pre_attention(layer, 0, 0, q[layer], k[layer], v[layer], q_out)
        sec, timed = time_steps(torch, step, steps, warmup)
        kms, _ = kernel_ms(torch, at, step, 0, bursts=4, burst=26)
    with A.Attn(1, 8, 2, D, 4096, 1, A.F16, A.F16, stream=torch.cuda.current_stream().cuda_stream) as at1:
        at1.set_layer_transform(0, norm_q=True, norm_k=True, eps=1e-6, rope_inv_freq=(10000.0 ** -d).astype(np.float32))
        q1 = torch.randn((1, 8, D), generator=g, device="cuda:0").half()
        k1 = torch.randn((1, 2, D), generator=g, device="cuda:0").half()
        o1 = torch.zeros_like(q1)
        lat, _ = time_steps(torch, lambda i: at1.pre_attention(0, 0, i % 4000, q1, k1, k1, o1), 200, 20)
    nbytes = 2 * n * (hq + 2 * hkv) * D * 2  # every row read once and written once
    return {"workload": f"step before attention, config 2 shape: {n} tokens x (Hq{hq} + 2 x Hkv{hkv}) rows, bf16, "
                        f"RMS norm of q / k + rotary embedding + cache write, one launch per layer, {layers} layers in turn "
                        "(6 MiB per launch: L2 / Infinity Cache resident, launch-latency bound)",
            "ms_per_step": sec * 1e3, "timed_steps": timed, "kernel_ms": kms, "bytes": nbytes, "GBps": nbytes / sec / 1e9,
            "kernel_GBps": nbytes / (kms * 1e-3) / 1e9, "tokens_per_s": n / sec,
            "single_token_latency_us": lat * 1e6}


def pipeline_report(X, device_resident, two_call_decode_step=False):
    """The reference's benchmark protocol (1024 prefill ids, 256 decode steps, README.md:390-400 of the
    reference) through the C++ executor, reported by the reference's own BenchmarkInfo text. The layers
    around attention are synthetic stand-ins; the rates say how the protocol runs end to end, they are
    not kernel figures."""
    import re
    layers = 26
    windows = [0 if (l + 1) % 6 == 0 else 512 for l in range(layers)]
    kw = {"device_resident": bool(device_resident), "two_call_decode_step": bool(two_call_decode_step)}
    with X.HipLlmExecutor(layers, 4, 1, 64, 2048, runner_lengths=(1024,), layer_window=windows, fp16=True,
                          pre_attention=True, **kw) as ex:
        r = X.run_benchmark(ex, [3, 1, 4, 1, 5, 9, 2, 6], 1024, 256)
    pre = re.search(r"Prefill Speed: ([0-9.]+) tokens/sec", r["report"])
    dec = re.search(r"Decode Speed: ([0-9.]+) tokens/sec", r["report"])
    return r["report"], float(pre.group(1)), float(dec.group(1))


def protocol_layer_latency(A, torch, ctx=1152):
    """Latency of one decode attention call (attention + merge launches, queued back to back) at the shape of the
    benchmark protocol's decode turn: Hq4 / Hkv1, fp16, about the middle context of the 256 steps."""
    at = A.Attn(1, 4, 1, D, 2048, 1, A.F16, A.F16)
    fill_cache(at, torch, 1, [ctx], 1, torch.float16, seed=7)
    q = torch.randn((1, 4, D), device="cuda:0", dtype=torch.float32).half()
    out = torch.empty_like(q)
    lens = A._i32_array([ctx])
    sec, _ = time_steps(torch, lambda i: at.decode(0, lens, q, out, num_splits=0, batch=1), 500, 50)
    at.close()
    return sec


def decode_step_latency(A, torch, ctx=1152):
    """One decode step of one layer at the same shape from the raw projections of the new token (Gemma-3-like
    norms and rotary embedding): mi355_attn_pre_attention + mi355_attn_decode (two calls) against
    mi355_attn_decode_step (one call, the same bits). Seconds per step, (two calls, one call)."""
    at = A.Attn(1, 4, 1, D, 2048, 1, A.F16, A.F16)
    fill_cache(at, torch, 1, [ctx], 1, torch.float16, seed=7)
    ones = np.ones(D, np.float32)
    at.set_layer_transform(0, norm_q=True, norm_k=True, q_weight=ones, k_weight=ones, eps=1e-6,
                           rope_inv_freq=(10000.0 ** (-np.arange(0, D, 2, dtype=np.float64) / D)).astype(np.float32))
    q = torch.randn((1, 4, D), device="cuda:0").half()
    k = torch.randn((1, 1, D), device="cuda:0").half()
    v = torch.randn((1, 1, D), device="cuda:0").half()
    q_rot, out = torch.empty_like(q), torch.empty_like(q)
    lens = A._i32_array([ctx])

    def two_calls(i):
        at.pre_attention(0, 0, ctx - 1, q, k, v, q_rot)
        at.decode(0, lens, q_rot, out, num_splits=0, batch=1)

    two, _ = time_steps(torch, two_calls, 500, 50)
    one, _ = time_steps(torch, lambda i: at.decode_step(0, lens, q, k, v, out, num_splits=0, batch=1), 500, 50)
    at.close()
    return two, one


def cpu_baseline_c3(layers, ctx, budget_s=24.0):
    """C restatement of the reference CPU op order (fp32, OpenMP) on the same
    30-layer decode sweep, repeated until about `budget_s` seconds are spent:
    at 4 threads (the reference's CpuConfig default) and at all host cores."""
    from oracle import c_oracle
    hq, hkv = 8, 2
    rng = np.random.default_rng(0xC0FFEE + 2)
    ks = [rng.standard_normal((ctx, hkv, D), dtype=np.float32) for _ in range(layers)]
    vs = [rng.standard_normal((ctx, hkv, D), dtype=np.float32) for _ in range(layers)]
    q = rng.standard_normal((layers, hq, D), dtype=np.float32)
    res = []
    for threads in (4, 0):
        c_oracle.decode_batch_ref_f32(q, ks, vs, D ** -0.5, threads=threads)  # warm
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < budget_s / 2:
            c_oracle.decode_batch_ref_f32(q, ks, vs, D ** -0.5, threads=threads)
            reps += 1
        sec = (time.perf_counter() - t0) / reps
        res.append({"threads": threads if threads > 0 else c_oracle.num_threads(), "sec_per_step": sec, "reps": reps})
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="headline decode workload only")
    ap.add_argument("--no-pipeline", action="store_true",
                    help="skip the legs that call the way an executor does: the 1024 / 256 protocol run through the "
                         "C++ executor and prefill as one launch per layer (thousands of small launches: left out "
                         "of rocprofv3 runs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (reference point for rocprofv3 --pmc counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from __graft_entry__ import load_package
    A = load_package().attn
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    log(f"[bench] {A.version()} on {torch.cuda.get_device_name(0)}")

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").random_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    dec = bench_decode_c3(A, torch, args.steps, args.warmup)
    log(f"[bench] decode C3x{dec['layers']}: {dec['sec_per_step']*1e6:.1f} us/step over {dec['timed_steps']} steps, "
        f"kernel {dec['kernel_ms']*1e3:.1f} us; graphs: {json.dumps(dec['graph'].get('one_launch'))} "
        f"{json.dumps(dec['graph'].get('per_layer_chain'))} {dec['graph'].get('error', '')}")
    value = dec["step_bytes"] / dec["sec_per_step"] / 1e9
    achieved = dec["step_bytes"] / (dec["kernel_ms"] * 1e-3) / 1e9
    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "timed_steps": dec["timed_steps"],
        "timed_region_s": round(dec["timed_steps"] * dec["sec_per_step"], 4),
        "ms_per_step": round(dec["sec_per_step"] * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "C3 x 30 layers: Gemma3n-E2B-shaped decode attention, batch 1, Hq8/Hkv2, head_dim 256, "
                        "fp16 KV cache at 4096 context, 16 split-KV partitions + LSE merge, one multi-layer launch "
                        "per step, rotating over 4 cache sets (1 GiB) so reads come from HBM",
            "layers_per_step": dec["layers"], "context": 4096, "num_splits": 16,
            "algorithmic_bytes_per_step": dec["step_bytes"],
            "timing": f"every leg is timed over at least {MIN_TIMED_REGION_S} s of back-to-back steps (timed_steps >= --steps)",
        },
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "value_is": f"algorithmic bytes per step / wall time per step over the {MIN_TIMED_REGION_S} s region (ms_per_step x "
                    "timed_steps); `sustained` is the same step queued back to back for 2 s",
        "sustained": {"seconds": round(dec["sustained_sec_per_step"] * dec["sustained_steps"], 3),
                      "steps": dec["sustained_steps"], "ms_per_step": round(dec["sustained_sec_per_step"] * 1e3, 5),
                      "GBps": round(dec["step_bytes"] / dec["sustained_sec_per_step"] / 1e9, 1),
                      "frac_of_hbm_peak": round(dec["step_bytes"] / dec["sustained_sec_per_step"] / 1e9 / HBM_PEAK_GBS, 4)},
        "decode_steps_per_s": round(dec["tokens_per_s"], 1),
        "single_layer_latency_us": round(dec["single_layer_latency_us"], 2),
        "roofline": {
            "kernel": "decode_attn_kernel<f16,f16,256>",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": load_traffic("decode_c3x30"),
            "algorithmic_bytes_per_launch": dec["step_bytes"],
            "avg_kernel_us": round(dec["kernel_ms"] * 1e3, 2),
            "us_per_step_of_the_same_bursts": round(dec["burst_ms_per_step"] * 1e3, 2),
            "read_floor_us": round(dec["floor_ms"] * 1e3, 2),
            "frac_of_read_floor": round(dec["floor_ms"] / dec["kernel_ms"], 4),
            "read_floor_is": "a launch of the same shape (960 one-wave workgroups) that only streams the same number of "
                             "bytes with the kernel's load pattern (mi355_attn_stream_probe), same stamps",
        },
        "decode_graph": dec["graph"],
    }

    if not args.no_extras:
        few, fw = max(20, args.steps // 4), max(5, args.warmup // 4)
        pre = bench_prefill_c2(A, torch, few, fw, by_layer=not args.no_pipeline, sustained=True)
        log(f"[bench] prefill C2: {pre['ms_per_step']:.4f} ms/step over {pre['timed_steps']} steps, "
            f"{pre['kernel_TFLOPs']:.1f} TFLOP/s kernel")
        result["prefill"] = {
            "workload": pre["workload"], "value": round(pre["TFLOPs"], 2), "unit": "TFLOP/s", "dtype": "bf16",
            "ms_per_step": round(pre["ms_per_step"], 4), "timed_steps": pre["timed_steps"],
            "prefill_tokens_per_s": round(pre["tokens_per_s"], 1),
            "sustained": {"seconds": round(pre["sustained_sec_per_step"] * pre["sustained_steps"], 3),
                          "steps": pre["sustained_steps"], "ms_per_step": round(pre["sustained_sec_per_step"] * 1e3, 5),
                          "TFLOPs": round(pre["flops"] / pre["sustained_sec_per_step"] / 1e12, 2),
                          "frac_of_mfma_peak": round(pre["flops"] / pre["sustained_sec_per_step"] / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)},
            "single_global_layer_ms": round(pre["single_global_layer_ms"], 4),
            "layer_by_layer": None if args.no_pipeline else {
                "what": "the same 26 layers as 26 launches in turn (how an executor calls it); key ranges of a "
                        "launch this small are cut into parts that a second kernel merges (option "
                        "prefill_key_split, default by rule), *_unsplit: with that switched off",
                "ms": round(pre["layer_by_layer_ms"], 4), "TFLOPs": round(pre["flops"] / pre["layer_by_layer_ms"] / 1e9, 2),
                "unsplit_ms": round(pre["layer_by_layer_unsplit_ms"], 4),
                "single_global_layer_unsplit_ms": round(pre["single_global_layer_unsplit_ms"], 4)},
            "dense_counted_TFLOPs": round(pre["dense_counted_TFLOPs"], 2),
            "roofline": {"kernel": "prefill_attn16_kernel<bf16,256>", "bound": "mfma",
                         "achieved": round(pre["kernel_TFLOPs"], 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(pre["frac_of_mfma_peak"], 4), "traffic": load_traffic("prefill_c2_bf16"),
                         "algorithmic_flops_per_launch": pre["flops"], "avg_kernel_us": round(pre["kernel_ms"] * 1e3, 2),
                         "us_per_step_of_the_same_bursts": round(pre["burst_ms_per_step"] * 1e3, 2),
                         "note": "avg_kernel_us: begin / end stamps of the dispatch, read at the end of bursts of 32 "
                                 "back-to-back launches; us_per_step_of_the_same_bursts: stream events around those "
                                 "bursts / 32 (launch gaps and the read-out at the end of each burst included)"},
        }
        pre16 = bench_prefill_c2(A, torch, few, fw, half=True)
        log(f"[bench] prefill C2 in fp16: {pre16['ms_per_step']:.4f} ms/step, {pre16['kernel_TFLOPs']:.1f} TFLOP/s kernel")
        result["prefill_fp16"] = {"workload": pre16["workload"], "value": round(pre16["TFLOPs"], 2), "unit": "TFLOP/s",
                                  "ms_per_step": round(pre16["ms_per_step"], 4),
                                  "kernel_TFLOPs": round(pre16["kernel_TFLOPs"], 2),
                                  "frac_of_mfma_peak": round(pre16["frac_of_mfma_peak"], 4),
                                  "avg_kernel_us": round(pre16["kernel_ms"] * 1e3, 2),
                                  "us_per_step_of_the_same_bursts": round(pre16["burst_ms_per_step"] * 1e3, 2)}
        pre32 = bench_prefill_c2(A, torch, few, fw, rows16=0)
        log(f"[bench] prefill C2 with the 32x32x16-MFMA kernel: {pre32['ms_per_step']:.4f} ms/step, "
            f"{pre32['kernel_TFLOPs']:.1f} TFLOP/s kernel")
        result["prefill_mfma32_kernel"] = {
            "workload": pre32["workload"] + ", option prefill_rows16=0: the kernel with one workgroup per CU that "
                                            "small launches use (the default picks the 16x16x32 kernel here)",
            "value": round(pre32["TFLOPs"], 2), "unit": "TFLOP/s", "kernel_TFLOPs": round(pre32["kernel_TFLOPs"], 2),
            "frac_of_mfma_peak": round(pre32["frac_of_mfma_peak"], 4), "avg_kernel_us": round(pre32["kernel_ms"] * 1e3, 2)}
        i8_rows = []
        for name, kw in (("one layer, Hq8/Hkv2 (config 5's heads), rows 0..1023 of a sequence",
                          dict(layers=1, n=1024, q_pos0=0, hq=8, hkv=2)),
                         ("one layer, Hq8/Hkv2, rows 3072..4095 of a 4096-token sequence",
                          dict(layers=1, n=1024, q_pos0=3072, hq=8, hkv=2)),
                         ("26 layers x 1024 tokens, Hq4/Hkv1, 22 local(W=512)+4 global (config 2's shape on an int8 cache)",
                          dict(layers=26, n=1024, q_pos0=0, hq=4, hkv=1,
                               windows=[0 if (l + 1) % 6 == 0 else 512 for l in range(26)]))):
            r = bench_prefill_int8(A, torch, few, fw, **kw)
            log(f"[bench] prefill int8, {name}: {r['ms_per_step'] * 1e3:.1f} us/call = {r['TFLOPs']:.1f} TFLOP/s "
                f"(device time {r['call_us_device']:.1f} us = {r['device_TFLOPs']:.1f} TFLOP/s); row-wise path "
                f"{r['rowwise_ms_per_step'] * 1e3:.1f} us/call = {r['rowwise_TFLOPs']:.2f} TFLOP/s")
            i8_rows.append({"workload": name, "unit": "TFLOP/s", "value": round(r["TFLOPs"], 2),
                            "us_per_call": round(r["ms_per_step"] * 1e3, 2),
                            "device_us_per_call": round(r["call_us_device"], 2),
                            "device_TFLOPs": round(r["device_TFLOPs"], 2),
                            "frac_of_mfma_peak": round(r["device_TFLOPs"] / MFMA_BF16_PEAK_TFLOPS, 4),
                            "rowwise_path": {"value": round(r["rowwise_TFLOPs"], 3), "us_per_call": round(r["rowwise_ms_per_step"] * 1e3, 2),
                                             "kernel_us": round(r["rowwise_kernel_us"], 2),
                                             "kernel_TFLOPs": round(r["rowwise_kernel_TFLOPs"], 3)}})
        result["prefill_int8"] = {
            "what": "prefill over an int8 cache, fp16 activations. value: whole calls back to back (query staging, "
                    "the planes' conversion to half planes, attention); device_us_per_call: from the start of the first "
                    "of those launches to the end of the attention kernel; rowwise_path: the same call with option "
                    "rowwise_prefill=1 (every query row a decode item, int8 converted in registers)",
            "rows": i8_rows}
        probe = gemm_probe(torch)
        log(f"[bench] vendor bf16 GEMM 8192^3: {probe:.0f} TFLOP/s")
        result["mfma_peak_probe"] = {"what": "torch.matmul bf16 8192x8192x8192 (hipBLASLt)", "TFLOPs": round(probe, 1),
                                     "published_dense_peak_TFLOPs": MFMA_BF16_PEAK_TFLOPS}
        rng = np.random.default_rng(0xC0FFEE + 3)
        lens4 = [int(x) for x in rng.integers(256, 4097, size=64)]
        extras = []
        # (the 16-layer launches sweep 2 to 4.5 GB of cache each: nothing of it stays in L2 or the Infinity Cache)
        for name, kv, lens, rot, nl in (("C4: 64 seqs, L~U[256,4096], fp16, one layer", A.F16, lens4, 4, 1),
                                        ("C5: 32 seqs x 4096, int8 KV + fp32 scales, one layer", A.I8, [4096] * 32, 6, 1),
                                        ("C4 x 16 layers in one launch, split count by the library's rule (none)", A.F16, lens4, 1, 16),
                                        ("C5 x 16 layers in one launch, split count by the library's rule (none)", A.I8, [4096] * 32, 1, 16),
                                        ("32 seqs x 4096, fp16, 16 layers in one launch, split count by the library's rule (none)", A.F16, [4096] * 32, 1, 16)):
            # split count: 16 for one layer; the library's own rule (num_splits 0) for the 16-layer launches,
            # which have a workgroup per wave slot without any split
            r = bench_decode_batch(A, torch, name, kv, lens, few, fw, rot, 16 if nl == 1 else 0, layers=nl)
            log(f"[bench] {name}: {r['ms_per_step']*1e3:.1f} us/step, kernel {r['kernel_GBps']:.0f} GB/s")
            extras.append(rounded(r))
        c1 = bench_decode_c1(A, torch, args.steps, args.warmup)
        log(f"[bench] {c1['workload']}: {c1['ms_per_step']*1e3:.1f} us/step")
        extras.append(rounded(c1))
        result["other_decode_configs"] = extras
        smp = bench_sampler(load_package().sampler, torch, few, fw)
        log(f"[bench] {smp['workload']}: {smp['ms_per_step']*1e3:.1f} us/step, kernel {smp['kernel_GBps']:.0f} GB/s, "
            f"one row {smp['single_row_latency_us']:.1f} us")
        result["sampler"] = rounded(smp)
        pa = bench_pre_attention(A, torch, args.steps, args.warmup)
        log(f"[bench] {pa['workload']}: {pa['ms_per_step']*1e3:.1f} us/step, kernel {pa['kernel_ms']*1e3:.1f} us "
            f"({pa['kernel_GBps']:.0f} GB/s), one token {pa['single_token_latency_us']:.1f} us")
        result["pre_attention"] = rounded(pa)
        if not args.no_pipeline:
            X = load_package().executor
            proto = {"what": "1024 prefill ids + 256 decode steps through HipLlmExecutor (26 layers, 5 local : 1 global, fp16, "
                             "fused step before attention), in the reference's report format; the layers other than "
                             "attention are synthetic stand-ins, so these are protocol figures, not kernel figures. "
                             "device_resident: activations, cache, logits and sampling stay on the GPU and only the "
                             "token id returns, and a decode step makes one attention call per layer (mi355_attn_decode_step); "
                             "device_resident_two_calls_per_layer: the same with mi355_attn_pre_attention and "
                             "mi355_attn_decode as two calls; host_staged: float32 host tensors staged through the "
                             "boundary per call"}
            for mode, resident, two_calls in (("device_resident", True, False),
                                              ("device_resident_two_calls_per_layer", True, True),
                                              ("host_staged", False, False)):
                if resident and not getattr(X, "HAS_DEVICE_RESIDENT", False):
                    continue
                text, pre_tps, dec_tps = pipeline_report(X, resident, two_calls)
                log(f"[bench] the reference's benchmark protocol (1024 prefill / 256 decode ids), {mode}:\n" + text)
                proto[mode] = {"prefill_tokens_per_s": pre_tps, "decode_tokens_per_s": dec_tps}
            lat = protocol_layer_latency(A, torch)
            proto["one_layer_decode_attention_latency_us"] = round(lat * 1e6, 2)
            two, one = decode_step_latency(A, torch)
            proto["one_layer_decode_step_latency_us"] = {"pre_attention_then_decode": round(two * 1e6, 2),
                                                         "decode_step": round(one * 1e6, 2)}
            proto["decode_tokens_per_s_if_only_attention_ran"] = round(1.0 / (26 * lat), 1)
            if "device_resident" in proto:
                proto["device_resident_fraction_of_that"] = round(
                    proto["device_resident"]["decode_tokens_per_s"] * 26 * lat, 3)
            result["pipeline_protocol"] = proto

    if not args.no_cpu:
        cpu = cpu_baseline_c3(dec["layers"], 4096)
        ref, allc = cpu[0], cpu[1]
        result["cpu_baseline"] = {
            "value": round(dec["step_bytes"] / ref["sec_per_step"] / 1e9, 3),
            "unit": "GB/s",
            "cores": ref["threads"],
            "kind": "port",
            "sample": f"{ref['reps']} passes of the same 30-layer decode sweep (fp32 K/V copies, about 12 s), "
                      "C restatement of the reference CPU op order (oracle/attn_oracle.c, OpenMP); "
                      "4 threads = the reference's CpuConfig default; bytes counted as for the GPU (fp16 sizes)",
            "ms_per_step": round(ref["sec_per_step"] * 1e3, 3),
        }
        result["cpu_baseline_all_cores"] = {
            "value": round(dec["step_bytes"] / allc["sec_per_step"] / 1e9, 3), "unit": "GB/s", "cores": allc["threads"],
            "kind": "port", "ms_per_step": round(allc["sec_per_step"] * 1e3, 3),
            "note": "the same restatement with every host thread the process may use "
                    f"(OpenMP reports {allc['threads']}; equal to the 4-thread leg when the host grants 4)"}
    try:  # what is left behind at exit is stated, not guessed
        import psutil
        kids = psutil.Process().children(recursive=True)
        result["child_processes_at_exit"] = [f"{p.pid}:{p.name()}" for p in kids]
    except Exception:
        pass
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
