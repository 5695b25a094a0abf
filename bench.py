#!/usr/bin/env python3
"""Benchmark of the GGUF quantized decode hot path on one MI355X.

Headline workload (config.workload = "C3"): the seven projections of one Llama-7B decoder layer at
batch 1 -- q, k, o (4096x4096), gate, up (11008x4096) in Q4_K and v (4096x4096), down (4096x11008) in
Q6_K -- 129 785 856 weight bytes per layer.  One "step" is one pass over one layer: quantize the seven
activation vectors, then the seven dequant-fused GEMVs in one grouped launch.  Steps rotate through 32
distinct synthetic layers (4.15 GB), so weights come from HBM and not from the 256 MB Infinity Cache.
`value` is weight GB/s = weight bytes per step / wall time per step (inputs resident in HBM).

Also reported on the same JSON line:
  roofline      the GEMV kernel alone: algorithmic bytes per launch / mean launch duration (HIP events
                around back-to-back launches on the library's stream) against the 8 TB/s HBM peak
  decode        the 32-layer, 7B-shaped greedy decode loop (config C5): tokens/s after a 128-token prompt
  cpu_baseline  the oracle's restatement of the reference CPU path (dequantize the whole tensor to f32,
                then naive row-dot with sequential k accumulation) timed on this host for one layer
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK = 8.0e12
PARITY_BOUND = 1e-3     # max |y - y_f64| / (||w_row|| ||x||) a benchmarked launch may show
# HBM bytes one launch moves on the headline workload, per kernel, from the FETCH_SIZE and WRITE_SIZE hardware counters
# (each scaled by what the same counter reads for a plain x += y kernel of known size); measured offline with the
# profiler, since counters cannot be read from inside this process.  A kernel without a measurement reports null.
GEMV_TRAFFIC_BYTES = {"qgemv_kernel<512>": 131_800_000}
SEED = 20250127
H, F, V, NH, NL = 4096, 11008, 32000, 32, 32


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def timed_regions(ex, region, min_ms=10.0, max_regions=500):
    """Times `region()` -- a callable that enqueues a fixed number of launches -- between two events and a synchronisation on
    both sides, again and again until at least `min_ms` of device time have been measured (at least three regions).  Returns
    the median region: (milliseconds between the events, wall seconds, number of regions).  A region of 20 launches of
    30 us is 0.6 ms, too short to hang a headline on; the median over the repeats is what is reported."""
    ev, wall, total = [], [], 0.0
    while (total < min_ms or len(ev) < 3) and len(ev) < max_regions:
        e0, e1 = ex.event(), ex.event()
        ex.synchronize()
        t0 = time.perf_counter()
        e0.record()
        region()
        e1.record()
        ex.synchronize()
        wall.append(time.perf_counter() - t0)
        ev.append(e0.elapsed_ms(e1))
        total += ev[-1]
    return float(np.median(ev)), float(np.median(wall)), len(ev)


def layer_bytes_algorithmic(specs):
    """weights once + f32 x + f32 y per projection."""
    w = sum(t.row_bytes(c) * r for _, t, r, c in specs)
    io = sum(4 * c + 4 * r for _, _, r, c in specs)
    return w, w + io


def bench_layer_gemv(ex, steps, warmup, n_layers):
    from rustorch_amd import synth
    specs = synth.layer_tensor_specs(H, F)
    wbytes, abytes = layer_bytes_algorithmic(specs)
    layers = []
    t0 = time.time()
    for l in range(n_layers):
        ws = [ex.upload_qweight(t, r, c, synth.blocks(t, SEED, synth.layer_tid(l, slot), r, c)) for slot, t, r, c in specs]
        layers.append(ws)
    log("[bench] %d layers (%.2f GB) generated and uploaded in %.1f s" % (n_layers, n_layers * wbytes / 1e9, time.time() - t0))
    plan = ex.qgemv_describe(layers[0])       # the kernel the timed launch runs and how the planner cuts it
    log("[bench] headline launch:", plan)
    xs = [ex.to_device(synth.normal(SEED, 1000 + i, c)) for i, (_, _, _, c) in enumerate(specs)]
    xqs = [ex.buffer(ex.xq_bytes(c)) for _, _, _, c in specs]
    ys = [ex.buffer(4 * r) for _, _, r, _ in specs]
    ncols = [c for _, _, _, c in specs]

    def step(i):
        ex.quantize_act_dev(xs, ncols, xqs)
        ex.qgemv_xq_grouped_dev(layers[i % n_layers], xqs, ys)

    for i in range(warmup):
        step(i)
    ex.synchronize()
    # every region below is `steps` launches (or steps) back to back, timed as a whole and repeated (timed_regions)
    ev_ms, wall, n_regions = timed_regions(ex, lambda: [step(warmup + i) for i in range(steps)])
    # kernel-only region: the grouped GEMV launch alone, back to back
    ex.quantize_act_dev(xs, ncols, xqs)
    kern_ms = timed_regions(ex, lambda: [ex.qgemv_xq_grouped_dev(layers[(warmup + i) % n_layers], xqs, ys) for i in range(steps)])[0] / steps
    # the step with the quantization folded into the GEMV's staging (what the decode loop launches)
    fused_ms = timed_regions(ex, lambda: [ex.qgemv_grouped_dev(layers[(warmup + i) % n_layers], xs, ys) for i in range(steps)])[0] / steps
    # the same launch on one layer over and over: its 130 MB stay in the 256 MB Infinity Cache
    for i in range(8):
        ex.qgemv_xq_grouped_dev(layers[0], xqs, ys)
    hot_ms = timed_regions(ex, lambda: [ex.qgemv_xq_grouped_dev(layers[0], xqs, ys) for i in range(steps)])[0] / steps
    # what the benchmarked launch computes for layer 0, for the correctness gate (checked outside the timed regions)
    ex.qgemv_xq_grouped_dev(layers[0], xqs, ys)
    ex.synchronize()
    results = [y.download(np.float32) for y in ys]
    for ws in layers:
        for w in ws:
            w.free()
    return dict(wbytes=wbytes, abytes=abytes, wall_s=wall, event_ms=ev_ms, kernel_ms=kern_ms, hot_ms=hot_ms, fused_ms=fused_ms, regions=n_regions,
                results=results, plan=plan)


def bench_read_probe(ex, nbytes, steps):
    """What a plain read kernel reaches on launches of the headline's size: `steps` launches over rotating 130 MB pieces of a
    4 GB buffer (HBM) and over one piece again and again (Infinity Cache), in the GEMV's own access shape."""
    n_sets = 32
    buf = ex.buffer(n_sets * nbytes)
    buf.zero()
    for i in range(8):
        ex.stream_read_dev(buf, i * nbytes, nbytes)
    hbm_ms = timed_regions(ex, lambda: [ex.stream_read_dev(buf, ((i + 8) % n_sets) * nbytes, nbytes) for i in range(steps)])[0] / steps
    hot_ms = timed_regions(ex, lambda: [ex.stream_read_dev(buf, 0, nbytes) for i in range(steps)])[0] / steps
    buf.free()
    return {"bytes_per_launch": nbytes, "hbm_launch_ms": round(hbm_ms, 5), "hbm_gbps": round(nbytes / hbm_ms / 1e6, 1),
            "hbm_frac": round(nbytes / (hbm_ms * 1e-3) / HBM_PEAK, 4), "cache_resident_launch_ms": round(hot_ms, 5)}


def bench_single_gemv(ex, reps=200):
    """The single-matrix decode configurations: Q8_0 4096x4096 and Q4_0 at the two FFN shapes (and one Q5_K and one unquantized F16 matrix), batch 1, x resident
    in HBM as f32 (quantized in the kernel's staging).  Eight synthetic copies of each matrix are rotated so that
    the larger ones come from HBM rather than from the Infinity Cache."""
    from rustorch_amd import synth, GGMLType
    out = []
    for name, t, rows, cols in (("q8_0_4096x4096", GGMLType.Q8_0, 4096, 4096),
                                ("q4_0_11008x4096", GGMLType.Q4_0, 11008, 4096),
                                ("q4_0_4096x11008", GGMLType.Q4_0, 4096, 11008),
                                ("q5_k_11008x4096", GGMLType.Q5_K, 11008, 4096),      # not benchmark configurations: for the record
                                ("f16_4096x4096", GGMLType.F16, 4096, 4096)):
        ws = [ex.upload_qweight(t, rows, cols, synth.blocks(t, SEED, 8000 + i, rows, cols)) for i in range(8)]
        x = ex.to_device(synth.normal(SEED, 8100, cols))
        y = ex.buffer(4 * rows)
        for i in range(16):
            ex.qgemv_dev(ws[i % 8], x, y)
        ms = timed_regions(ex, lambda: [ex.qgemv_dev(ws[i % 8], x, y) for i in range(reps)])[0] / reps
        wbytes = t.row_bytes(cols) * rows
        out.append({"shape": name, "us": round(ms * 1e3, 2), "weight_gbps": round(wbytes / ms / 1e6, 1),
                    "hbm_frac": round(wbytes / (ms * 1e-3) / HBM_PEAK, 4)})
        for w in ws:
            w.free()
        x.free(); y.free()
    return out


# A 70B-class shape for the record (--decode-shape 70b): 43 GB of blocks resident on the one GPU, grouped-query attention.
SHAPES = {"7b": dict(NL=NL, H=H, NH=NH, NKV=NH, F=F, V=V), "70b": dict(NL=80, H=8192, NH=64, NKV=8, F=28672, V=32000)}


def bench_batch8(ex, reps=100):
    """Config C3 at M = 8: the layer shapes and the output head with eight activation rows per call.  From three rows on
    Q4_K / Q6_K weights take the integer matrix-core GEMV (one pass over the weights, preceded by a small launch that
    quantizes the rows); the time is the call's, both launches.  Weight GB/s counts the weights once."""
    from rustorch_amd import synth, GGMLType
    out = []
    for name, t, rows, cols in (("q4k_4096x4096", GGMLType.Q4_K, 4096, 4096), ("q4k_11008x4096", GGMLType.Q4_K, 11008, 4096),
                                ("q6k_4096x11008", GGMLType.Q6_K, 4096, 11008), ("q6k_32000x4096", GGMLType.Q6_K, 32000, 4096)):
        ws = [ex.upload_qweight(t, rows, cols, synth.blocks(t, SEED, 9000 + i, rows, cols)) for i in range(8)]
        x = ex.to_device(synth.normal(SEED, 9100, 8 * cols))
        y = ex.buffer(4 * 8 * rows)
        res = {}
        for batch in (1, 8):
            for i in range(8):
                ex.qgemv_dev(ws[i % 8], x, y, batch)
            res[batch] = timed_regions(ex, lambda: [ex.qgemv_dev(ws[i % 8], x, y, batch) for i in range(reps)])[0] / reps
        wbytes = t.row_bytes(cols) * rows
        out.append({"shape": name, "us_batch1": round(res[1] * 1e3, 2), "us_batch8": round(res[8] * 1e3, 2),
                    "weight_gbps_batch8": round(wbytes / res[8] / 1e6, 1), "rows_per_s_batch8": round(8 / (res[8] * 1e-3))})
        for w in ws:
            w.free()
        x.free(); y.free()
    return out


def bench_layer_batch8(ex, n_layers=4, reps=100):
    """Config C3 at M = 8 as one step: the seven projections of a Llama-7B layer with eight activation rows each, issued the
    way a layer would (q, k, v against the same rows; o; gate, up against the same rows; down), rotating through n_layers
    sets of weights (520 MB, beyond the 256 MB Infinity Cache).  Weight GB/s counts the weights once."""
    from rustorch_amd import synth
    specs = synth.layer_tensor_specs(H, F)
    wbytes, _ = layer_bytes_algorithmic(specs)
    layers = [[ex.upload_qweight(t, r, c, synth.blocks(t, SEED, synth.layer_tid(l, slot), r, c)) for slot, t, r, c in specs]
              for l in range(n_layers)]
    xh = ex.to_device(synth.normal(SEED, 9200, 8 * H))
    xf = ex.to_device(synth.normal(SEED, 9201, 8 * F))
    ys = [ex.buffer(4 * 8 * r) for _, _, r, _ in specs]

    def layer(ws):
        ex.qgemv_shared_x_dev(ws[0:3], xh, ys[0:3], 8)
        ex.qgemv_dev(ws[3], xh, ys[3], 8)
        ex.qgemv_shared_x_dev(ws[4:6], xh, ys[4:6], 8)
        ex.qgemv_dev(ws[6], xf, ys[6], 8)

    for i in range(8):
        layer(layers[i % n_layers])
    ms = timed_regions(ex, lambda: [layer(layers[i % n_layers]) for i in range(reps)])[0] / reps
    for ws in layers:
        for w in ws:
            w.free()
    for b in [xh, xf] + ys:
        b.free()
    return {"us_layer_batch8": round(ms * 1e3, 2), "weight_gbps": round(wbytes / ms / 1e6, 1), "rows_per_s": round(8 / (ms * 1e-3)),
            "launches_per_layer": 9}


def bench_decode_batch(gm, n_seq, n_prompt, n_gen, vocab):
    """Config C3's batch of eight as a loop: n_seq sequences decoded side by side against the model's weights (every matrix
    streamed once per step for all of them), prompts of n_prompt tokens through the prefill passes, then n_gen greedy steps timed.
    tokens/s counts the tokens of all sequences."""
    from rustorch_amd import llama, synth
    b = llama.HipLlamaBatch(gm, n_seq, n_prompt + n_gen)
    prompts = [synth.tokens(SEED, 9500 + i, n_prompt, vocab) for i in range(n_seq)]
    for i, pr in enumerate(prompts):                    # all but the last prompt token through the prefill passes
        b.prefill(i, pr[:-1], 0)
    picks = b.step([int(pr[-1]) for pr in prompts], [n_prompt - 1] * n_seq)
    t0 = time.perf_counter()
    for p in range(n_prompt, n_prompt + n_gen):
        picks = b.step([int(t) for t in picks], [p] * n_seq)
    dt = time.perf_counter() - t0
    b.close()
    return {"sequences": n_seq, "n_prompt": n_prompt, "n_generated": n_gen, "tokens_per_s": round(n_seq * n_gen / dt, 1),
            "ms_per_step": round(1e3 * dt / n_gen, 4), "note": "one host round trip per step (the picks come back to be fed)"}


def bench_decode(ex, n_prompt, n_gen, shape="7b", batch=0):
    from rustorch_amd import llama, synth
    sh = SHAPES[shape]
    NL, H, NH, NKV, F, V = sh["NL"], sh["H"], sh["NH"], sh["NKV"], sh["F"], sh["V"]
    t0 = time.time()
    gm = llama.HipLlama(ex, NL, H, NH, F, V, n_prompt + n_gen, n_kv_heads=NKV)
    wbytes = llama.load_synthetic(gm, SEED)
    log("[bench] %s-shaped model (%.2f GB of blocks) generated and uploaded in %.1f s" % (shape.upper(), wbytes / 1e9, time.time() - t0))
    prompt = synth.tokens(SEED, synth.TID_PROMPT, n_prompt, V)
    t0 = time.perf_counter()
    gm.prefill(prompt[:-1], 0)
    ex.synchronize()
    t_prefill = time.perf_counter() - t0
    # warm-up step, then rewind so the timed loop starts right after the prompt
    t0 = time.perf_counter()
    toks = gm.decode(int(prompt[-1]), n_prompt - 1, n_gen)
    t_dec = time.perf_counter() - t0
    side_by_side = bench_decode_batch(gm, batch, 16, 64, V) if batch else None
    gm.close()
    kv_dim = NKV * (H // NH)
    per_layer = sum(t.row_bytes(c) * r for _, t, r, c in synth.layer_tensor_specs(H, F, kv_dim))
    tok_bytes = NL * per_layer + 210 * (H // 256) * V       # weights streamed per token (output head is Q6_K)
    kv_avg = 2 * NL * kv_dim * 2 * (n_prompt + n_gen / 2)      # fp16 K and V rows read per token, averaged over the run
    return dict(shape=shape, tokens_per_s=n_gen / t_dec, ms_per_token=1e3 * t_dec / n_gen, prefill_tokens_per_s=(n_prompt - 1) / t_prefill,
                bytes_per_token=int(tok_bytes + kv_avg), hbm_frac=(tok_bytes + kv_avg) * n_gen / t_dec / HBM_PEAK,
                n_prompt=n_prompt, n_generated=n_gen, first_tokens=[int(t) for t in toks[:8]], **({"batch": side_by_side} if side_by_side else {}))


def bench_prefill(ex, reps=20):
    """Config C4: Y = X . dequant(W)^T on the matrix cores, X resident in HBM; 2MNK flops against the fp16 MFMA peak."""
    from rustorch_amd import synth, GGMLType
    MFMA_PEAK = 2.5e15
    out = []
    # the last two are not benchmark configurations: the fp16 contraction that serves the other formats, for the record
    for name, t, rows, cols in (("q4k_4096x4096", GGMLType.Q4_K, 4096, 4096), ("q4k_11008x4096", GGMLType.Q4_K, 11008, 4096),
                                ("q6k_4096x11008", GGMLType.Q6_K, 4096, 11008), ("q5k_4096x4096", GGMLType.Q5_K, 4096, 4096),
                                ("f16_4096x4096", GGMLType.F16, 4096, 4096)):
        w = ex.upload_qweight(t, rows, cols, synth.blocks(t, SEED, 7000 + rows + cols, rows, cols))
        for M in ((64, 512, 2048) if t in (GGMLType.Q4_K, GGMLType.Q6_K) else (512,)):
            x = ex.to_device(synth.normal(SEED, 7100 + M, M * cols))
            y = ex.buffer(4 * M * rows)
            for _ in range(3):
                ex.qgemm_dev(w, x, M, y)
            ms = timed_regions(ex, lambda: [ex.qgemm_dev(w, x, M, y) for _ in range(reps)])[0] / reps
            flops = 2.0 * M * rows * cols
            out.append({"shape": name, "M": M, "ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1),
                        "mfma_frac": round(flops / (ms * 1e-3) / MFMA_PEAK, 4)})
            x.free(); y.free()
        w.free()
    return out


def bench_dense_f32(ex, reps=5):
    """The dense f32 product on resident buffers (the executor the reference's unquantized callers use): 2 m n k flops against
    the f32 matrix-core peak.  Not a benchmark configuration; reported beside the others."""
    from rustorch_amd import synth
    F32_PEAK = 157.3e12
    out = []
    for m, n, k in ((4096, 4096, 4096), (512, 4096, 4096), (512, 11008, 4096)):
        a = ex.to_device(synth.normal(SEED, 7300 + m, m * k)); b = ex.to_device(synth.normal(SEED, 7301 + n, k * n))
        c = ex.buffer(4 * m * n)
        ex.matmul_f32_dev(a, b, c, m, n, k)
        ms = timed_regions(ex, lambda: [ex.matmul_f32_dev(a, b, c, m, n, k) for _ in range(reps)])[0] / reps
        flops = 2.0 * m * n * k
        out.append({"m": m, "n": n, "k": k, "ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1), "mfma_f32_frac": round(flops / (ms * 1e-3) / F32_PEAK, 4),
                    "kernel": "matmul_f32_mfma_kernel" if ex.get_option(ex.OPT_DENSE_MFMA) else "matmul_f32_kernel"})
        for buf in (a, b, c):
            buf.free()
    return out


def layer_inputs():
    """Blocks and activation vectors of layer 0 of the headline workload, as the GPU legs generate them."""
    from rustorch_amd import synth
    specs = synth.layer_tensor_specs(H, F)
    return [(t, r, c, synth.blocks(t, SEED, synth.layer_tid(0, slot), r, c), synth.normal(SEED, 1000 + i, c))
            for i, (slot, t, r, c) in enumerate(specs)]


def parity_of_launch(tensors, gpu_results):
    """The correctness gate of the timing: the worst |y_gpu - y_f64| / (||w_row|| ||x||) over the seven projections of the
    benchmarked launch, against the oracle's f64 products of the same blocks.  Computed outside the timed regions."""
    from oracle import oracle as orc
    worst = 0.0
    for (t, r, c, raw, x), got in zip(tensors, gpu_results):
        y64, wn = orc.qgemv_f64(t, raw, r, c, x)
        yard = wn * np.linalg.norm(x.astype(np.float64))
        if not np.isfinite(got).all():
            return float("inf")
        worst = max(worst, float((np.abs(got.astype(np.float64) - np.asarray(y64).reshape(-1)) / yard).max()))
    return worst


def cpu_baseline(tensors, reps):
    """Reference CPU path for one layer: dequantize each tensor to dense f32, then x . W^T with sequential k-sums."""
    from oracle import oracle as orc
    wbytes = sum(t.row_bytes(c) * r for t, r, c, _, _ in tensors)
    ncores = orc.num_threads()
    best = {}
    for threads in (1, ncores):
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            for t, r, c, raw, x in tensors:
                W = orc.dequant(t, raw, r, c, threads)
                orc.matmul_xwt(x, W, threads)
            ts.append(time.perf_counter() - t0)
        best[threads] = min(ts)
    return wbytes, best[1], best[ncores], ncores


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=320)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--layers", type=int, default=32, help="distinct synthetic layers rotated through (32 = 4.15 GB)")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--prefill-only", action="store_true", help="run only the prefill contraction shapes (for kernel traces)")
    ap.add_argument("--batch8-only", action="store_true", help="run only the eight-row GEMV shapes (for kernel traces)")
    ap.add_argument("--decode-prompt", type=int, default=128)
    ap.add_argument("--decode-gen", type=int, default=128)
    ap.add_argument("--decode-shape", choices=sorted(SHAPES), default="7b", help="model shape of the decode measurement (the benchmark's is 7b)")
    ap.add_argument("--decode-batch", type=int, default=0,
                    help="also decode this many sequences (1..8) side by side against the same model (rt_hip_llama_batch_*); off by default")
    ap.add_argument("--gemv-path", choices=("default", "general", "lean", "lean5"), default="default",
                    help="decode GEMV kernel of every leg: the library's default, the general kernel, the lean one, or the lean one with "
                         "five waves per SIMD where the launch allows it (rt_hip_set_option)")
    ap.add_argument("--dense-mfma", action="store_true", help="dense f32 leg on the f32 matrix-core kernel (rt_hip_set_option)")
    ap.add_argument("--calibrate", action="store_true",
                    help="run only a plain x += y kernel over 2 x 128 MiB (reads 256 MiB, writes 128 MiB per launch): "
                         "the known-size launch that hardware traffic counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported (use --gpus 1)" % args.gpus)

    from rustorch_amd.executor import HipKernelExecutor
    ex = HipKernelExecutor(0)
    info = ex.device_info()
    log("[bench] device:", info)

    if args.gemv_path != "default":
        ex.set_option(ex.OPT_GEMV_LEAN, {"general": 0, "lean": 1, "lean5": 2}[args.gemv_path])
    if args.dense_mfma:
        ex.set_option(ex.OPT_DENSE_MFMA, 1)

    if args.calibrate:
        n = 32 << 20
        a, b = ex.buffer(4 * n), ex.buffer(4 * n)
        a.zero(); b.zero()
        for _ in range(8):
            ex.add_dev(a, b, n)
        ex.synchronize()
        print(json.dumps({"calibrate": "add_kernel", "launches": 8, "read_bytes_per_launch": 8 * n, "write_bytes_per_launch": 4 * n}), flush=True)
        ex.close()
        return

    if args.prefill_only:
        print(json.dumps({"prefill": bench_prefill(ex)}), flush=True)
        ex.close()
        return
    if args.batch8_only:
        print(json.dumps({"batch8": bench_batch8(ex), "layer_batch8": bench_layer_batch8(ex)}), flush=True)
        ex.close()
        return

    g = bench_layer_gemv(ex, args.steps, args.warmup, args.layers)
    kernel = g["plan"].split(" ")[0]
    # the gate before anything is reported: a launch outside the bound has no rate
    tensors = None if args.no_cpu else layer_inputs()
    parity = None if args.no_cpu else parity_of_launch(tensors, g["results"])
    if parity is not None and not parity <= PARITY_BOUND:
        log("[bench] the benchmarked launch (%s) is outside the bound: worst |y - y_f64| / (||w_row|| ||x||) = %.3e > %.0e" % (g["plan"], parity, PARITY_BOUND))
        print(json.dumps({"metric": "Q4_K/Q6_K GEMV weight GB/s, one Llama-7B decoder layer at batch 1 (plus decode tokens/s), 1xMI355X", "value": None,
                          "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True,
                          "error": "parity gate failed", "config": {"workload": "C3", "parity_worst": parity, "kernel": g["plan"]}}), flush=True)
        ex.close()
        sys.exit(1)
    # wall_s, event_ms: the median region of `steps` steps (timed_regions)
    ms_per_step = 1e3 * g["wall_s"] / args.steps
    value = g["wbytes"] / (g["wall_s"] / args.steps) / 1e9
    achieved = g["abytes"] / (g["kernel_ms"] * 1e-3) / 1e9
    out = {
        "metric": "Q4_K/Q6_K GEMV weight GB/s, one Llama-7B decoder layer at batch 1 (plus decode tokens/s), 1xMI355X",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "q4_K/q6_K blocks x int16 block-scaled activations (int8 dot4, f32 accumulate)", "data": "synthetic",
        "config": {"workload": "C3: seven projections of one Llama-7B decoder layer, batch 1, q/k/o/gate/up Q4_K, v/down Q6_K",
                   "weight_bytes_per_step": g["wbytes"], "layers_rotated": args.layers, "hbm_frac_of_value": round(value * 1e9 / HBM_PEAK, 4),
                   "event_ms_per_step": round(g["event_ms"] / args.steps, 5),
                   "timing": "every figure is the median over %d repeats of a region of `steps` launches (repeated until 10 ms of device time are covered)" % g["regions"],
                   "tolerance": "max |y - y_f64| <= 1e-3 * ||w_row|| * ||x|| per element",
                   # of the benchmarked launch on one layer, in units of ||w_row|| ||x||; the run ends without a rate when it exceeds the bound
                   "parity_worst": parity},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK, 4), "traffic": GEMV_TRAFFIC_BYTES.get(kernel), "kernel": kernel, "launch": g["plan"],
                     "bytes_per_launch": g["abytes"], "avg_launch_ms": round(g["kernel_ms"], 5),
                     "cache_resident_launch_ms": round(g["hot_ms"], 5),
                     "fused_quantize_launch_ms": round(g["fused_ms"], 5)},
    }
    # the same number of bytes through a kernel that only reads: what the device grants a weight stream of this size
    out["roofline"]["read_probe"] = bench_read_probe(ex, g["wbytes"] // 2048 * 2048, args.steps)
    out["single_gemv"] = bench_single_gemv(ex)
    if not args.no_prefill:
        out["prefill"] = bench_prefill(ex)
        out["batch8"] = bench_batch8(ex)
        out["layer_batch8"] = bench_layer_batch8(ex)
        out["dense_f32"] = bench_dense_f32(ex)
    if not args.no_decode:
        out["decode"] = bench_decode(ex, args.decode_prompt, args.decode_gen, args.decode_shape, args.decode_batch)
    ex.close()
    if not args.no_cpu:
        wbytes, t1, tn, ncores = cpu_baseline(tensors, 3)
        out["cpu_baseline"] = {"value": round(wbytes / t1 / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": "one of the 32 layers (seven projections, batch 1): dequantize to dense f32, then naive x.W^T; best of 3",
                               "all_cores_value": round(wbytes / tn / 1e9, 4), "all_cores": ncores}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
