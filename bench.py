#!/usr/bin/env python3
"""Benchmark of the KV-cache attention path on one MI355X.

Workload (N = 1): GLM-4-9B-shaped long-context decode: 40 layers, 32 query heads, 2 KV groups,
head size 128, n_past = 32767, cache rows 32768, fp16 caches filled from N(0,1), one new token per
layer.  One "step" is one token: rope + K/V append + attention for all 40 layers, one
glm_attn_forward call (one kernel launch) per layer on one stream, each layer with its own 32 MiB cache (1.34 GB per
step, far beyond the 256 MB Infinity Cache).  The step is captured once in a HIP graph and replayed;
the eager (call-by-call) time is reported beside it.

Also measured and reported in the same JSON line: one 8192-token prefill chunk appended at
n_past = 24576 (TFLOP/s against the fp16 MFMA peak); the projections either side of the path ("linear"); the
whole decoder stack for one token ("layer": norms, projections, attention, gated MLP, residuals, 5 launches per
layer); the whole model through the C++ host classes with fp16 and with q4_0 weights ("model", "model_q4_0":
ids in, logits out, separate processes); and the CPU oracle on a bounded sample of the decode workload (the
reference's CPU path cannot be built here: ggml is not vendored).  --skip-* flags leave sections out.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
# HBM bytes one decode_kernel launch of this workload moves, from two rocprofv3 --pmc runs of this script
# (FETCH_SIZE 17,783 KiB x 2.000, WRITE_SIZE 2,073 KiB x 1.000; scales from a 256 MiB device copy in the same runs)
DECODE_TRAFFIC_PROFILE = os.path.join("profiles", "decode_kernel_glm4_32k_hbm_traffic_pmc.txt")


def decode_traffic_bytes_per_launch():
    """HBM bytes per decode launch from the committed counter summary (its line `traffic_bytes_per_launch: N`):
    the figure is refreshed with the profile, not kept as a constant here.  None when the file holds no such line."""
    import re

    try:
        text = open(os.path.join(os.path.dirname(os.path.abspath(__file__)), DECODE_TRAFFIC_PROFILE)).read()
    except OSError:
        return None
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9_,]+)", text, flags=re.M)
    return int(m.group(1).replace(",", "").replace("_", "")) if m else None
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16

H, KVH, D = 32, 2, 128
LAYERS = 40
MAX_LENGTH = 32768
N_PAST_DECODE = 32767
PREFILL_Q, PREFILL_N_PAST = 8192, 24576


def decode_bytes_per_layer(kvs):
    # K and V cache reads + the appended row/column + q, k, v in + out
    return 2 * KVH * kvs * D * 2 + 2 * KVH * D * 2 + H * D * 4 + 2 * KVH * D * 4 + H * D * 4


def prefill_flops_per_layer(qlen, n_past, causal):
    kvs = n_past + qlen
    pairs = qlen * (n_past) + qlen * (qlen + 1) // 2 if causal else qlen * kvs
    return 4 * H * D * pairs


def fill_cache_normal(torch, kv, seed):
    """fp16 N(0,1) into the whole slab, in chunks to bound temporary memory."""
    g = torch.Generator(device=kv.device)
    g.manual_seed(seed)
    n = kv.numel()
    chunk = 1 << 26
    view = kv.view(torch.float16)
    for o in range(0, n, chunk):
        m = min(chunk, n - o)
        view[o:o + m] = torch.randn(m, generator=g, device=kv.device, dtype=torch.float32).to(torch.float16)


def read_ceilings(torch, pkg, kv, layer_halfs, stream, warmup, steps):
    """Kernels that only load, launched like the decode step: LAYERS launches back to back on one stream, each
    over another layer's 32 MiB of cache, timed with events on that stream."""
    lib = pkg.bench_lib()
    sink = torch.zeros(1, dtype=torch.float32, device=kv.device)
    sh = stream.cuda_stream
    layer_bytes = layer_halfs * 2
    base = kv.data_ptr()

    def run(pattern, per_launch_bytes, launches, whole=False, sweep=None):
        def step():
            for l in range(launches):
                ptr = base if whole else base + l * layer_bytes
                if sweep is None:
                    st = lib.glm_bench_read(pattern, ptr, MAX_LENGTH, KVH, per_launch_bytes, sink.data_ptr(), sh)
                else:
                    st = lib.glm_bench_read_sweep(sweep[0], sweep[1], sweep[2], sweep[3], ptr, per_launch_bytes,
                                                  sink.data_ptr(), sh)
                if st != 0:
                    pkg.check(st, "glm_bench_read")

        with torch.cuda.stream(stream):
            for _ in range(warmup):
                step()
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(steps):
                step()
            e1.record(stream)
            torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (steps * launches)
        return {"us_per_launch": round(us, 3), "bytes_per_launch": per_launch_bytes,
                "gbs": round(per_launch_bytes / (us * 1e-6) / 1e9, 1) if per_launch_bytes else None,
                "frac_of_hbm_peak": round(per_launch_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
                if per_launch_bytes else None}

    out = {"workload": f"{LAYERS} launches back to back per step, one layer's caches (32 MiB) per launch, "
                       "256 workgroups of 8 waves, nothing but loads"}
    out["empty_launch"] = run(pkg.BENCH_EMPTY, 0, LAYERS)
    out["linear_read_per_launch"] = run(pkg.BENCH_READ_LINEAR, layer_bytes, LAYERS)
    out["decode_pattern_read_per_launch"] = run(pkg.BENCH_READ_DECODE_PATTERN, layer_bytes, LAYERS)
    out["one_long_streaming_launch"] = run(pkg.BENCH_READ_STREAM, layer_bytes * LAYERS, 1, whole=True)
    # The same 32 MiB per launch asked for in other ways: workgroups of 4, 8 or 16 waves, 8 to 32 loads of 16 bytes
    # per lane in flight, cache policy bits, straight into LDS.  The best of them is the ceiling.
    sweep = {}
    policies = (("plain", pkg.BENCH_POLICY_PLAIN), ("nt", pkg.BENCH_POLICY_NT), ("sc1", pkg.BENCH_POLICY_SC1),
                ("sc0_sc1_nt", pkg.BENCH_POLICY_SC0_SC1_NT))
    shapes = ((8, 16), (4, 16), (4, 32), (16, 8), (8, 8), (4, 8), (16, 16))
    for pname, pol in policies:
        for waves, loads in shapes:
            r = run(None, layer_bytes, LAYERS, sweep=(pol, waves, loads, 0))
            sweep[f"{pname}, {layer_bytes // (waves * loads * 1024)} workgroups x {waves} waves x {loads} loads"] = r
    for pname, pol in policies[:2]:
        for waves, loads in ((8, 16), (4, 16), (4, 32)):
            r = run(None, layer_bytes, LAYERS, sweep=(pol, waves, loads, 1))
            sweep[f"{pname} into LDS, {layer_bytes // (waves * loads * 1024)} workgroups x {waves} waves x {loads} "
                  "loads"] = r
    best = min(sweep, key=lambda k: sweep[k]["us_per_launch"])
    out["sweep"] = {k: {"us_per_launch": v["us_per_launch"], "frac_of_hbm_peak": v["frac_of_hbm_peak"]}
                    for k, v in sweep.items()}
    out["best_read_per_launch"] = dict(sweep[best], shape=best)
    return out


def mfma_ceilings(torch, pkg, stream):
    """Loops of matrix instructions (two waves per SIMD on every CU, operands with random bits), each long enough for
    the clock to settle: what the matrix pipes give any kernel here, beside the prefill kernel's rate."""
    import ctypes

    lib = pkg.bench_lib()
    dev = torch.device("cuda:0")
    operands = (torch.rand(1 << 16, device=dev, dtype=torch.float32) - 0.5).to(torch.float16)  # 128 KiB
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    sh = stream.cuda_stream
    out = {"workload": "2 workgroups of 4 waves per CU; per wave 2000 iterations of 32 32x32x16 (64 16x16x32) matrix "
                       "instructions; the 'mix' forms add one 16-byte-per-lane LDS read per 32x32x16 and 21 vector "
                       "instructions (4 v_exp_f32) per four, the prefill kernel's diet"}
    for name, pattern in (("mfma_32x32x16_f16", pkg.BENCH_MFMA_32X32X16), ("mfma_16x16x32_f16", pkg.BENCH_MFMA_16X16X32),
                          ("mfma_32x32x16_f16_mix", pkg.BENCH_MFMA_32X32X16_MIX),
                          ("mfma_16x16x32_f16_mix", pkg.BENCH_MFMA_16X16X32_MIX)):
        flops = ctypes.c_double(0.0)

        def launch():
            st = lib.glm_bench_mfma(pattern, operands.data_ptr(), operands.numel() * 2, 2000, sink.data_ptr(), sh,
                                    ctypes.byref(flops))
            if st != 0:
                pkg.check(st, "glm_bench_mfma")

        with torch.cuda.stream(stream):
            for _ in range(4):  # a few milliseconds each: the clock settles
                launch()
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(4):
                launch()
            e1.record(stream)
            torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 4
        tf = flops.value / (ms * 1e-3) / 1e12
        out[name] = {"ms_per_launch": round(ms, 3), "tflops": round(tf, 1),
                     "frac_of_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS, 4)}
    return out


def timelines(torch, pkg, capi):
    """In-kernel clock readings of the instrumented build: the decode launch of the headline workload and causal
    prompts of the ChatGLM3-6B shape.  Times are us since the first wave of the launch started; reading the clock
    costs about 0.1 us a time, so the instrumented kernels run a little longer than the plain ones."""
    import numpy as np

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(99)
    out = {}
    slot = np.arange(capi.TIMELINE_SLOTS)
    # decode, GLM-4-9B shape at 32k: 4 layers' caches, the last launch's readings
    layers = 4
    ctx = pkg.Context(num_layers=layers, num_attention_heads=H, num_key_value_heads=KVH, head_size=D,
                      max_length=MAX_LENGTH, max_qlen=1)
    width = (H + 2 * KVH) * D
    qkv = torch.randn(layers, width, generator=gen, device=dev, dtype=torch.float32)
    o = torch.zeros(layers, H * D, device=dev, dtype=torch.float32)
    for n_past in (N_PAST_DECODE, 4095):
        for _ in range(3):
            for l in range(layers):
                pkg.check(ctx.forward(l, qkv[l].data_ptr(), 1, n_past, o[l].data_ptr(), position_ids_host=[n_past]),
                          "glm_attn_forward")
        torch.cuda.synchronize()
        t = capi.read_timeline("decode")
        out[f"decode_kernel, n_past {n_past}"] = {
            "score waves": capi.summarise_timeline(t, capi.DECODE_STAMPS["score"], (slot % 8) < 4),
            "output waves": capi.summarise_timeline(t, capi.DECODE_STAMPS["output"], (slot % 8) >= 4)}
    ctx.close()
    # causal prompts at n_past 0, ChatGLM3-6B shape (32 heads, 2 KV groups, max_length 8192)
    ctx = pkg.Context(num_layers=1, num_attention_heads=32, num_key_value_heads=2, head_size=128, max_length=8192,
                      max_qlen=2048)
    for qlen in (2048, 512):
        qkv = torch.randn(qlen, width, generator=gen, device=dev, dtype=torch.float32)
        o = torch.zeros(qlen, 32 * 128, device=dev, dtype=torch.float32)
        pos = torch.arange(qlen, device=dev, dtype=torch.int32)
        for _ in range(3):
            pkg.check(ctx.forward(0, qkv.data_ptr(), qlen, 0, o.data_ptr(), position_ids_ptr=pos.data_ptr()),
                      "glm_attn_forward")
        torch.cuda.synchronize()
        t = capi.read_timeline("prefill")
        out[f"prefill_kernel, {qlen} causal tokens"] = capi.summarise_timeline(t, capi.PREFILL_STAMPS, slot >= 0)
    ctx.close()
    return out


class optional_section:
    """The sections beyond the contract's line (projections, whole layers, whole model) must not take the line with
    them: an exception inside one is recorded as that section's "error" and the run goes on."""

    def __init__(self, result, name):
        self.result, self.name = result, name

    def __enter__(self):
        return self

    def __exit__(self, etype, evalue, tb):
        if etype is not None and issubclass(etype, Exception):
            self.result[self.name] = {"error": f"{etype.__name__}: {evalue}"[:500]}
            return True
        return False


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="do not time the CPU oracle")
    ap.add_argument("--skip-prefill", action="store_true", help="do not time the prefill chunk")
    ap.add_argument("--prefill-only", action="store_true", help="time only the prefill chunk (for profiling)")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only")
    ap.add_argument("--skip-linear", action="store_true", help="do not time the two projections around the path")
    ap.add_argument("--skip-layer", action="store_true", help="do not time whole decoder layers")
    ap.add_argument("--skip-model", action="store_true", help="do not time the whole model (C++ host classes)")
    ap.add_argument("--ceiling", action="store_true",
                    help="also time kernels that only read (one layer's caches per launch in address order and in "
                         "the decode kernel's order, an empty launch, one long streaming launch): what this GPU "
                         "gives a launch shaped like the decode kernel's")
    ap.add_argument("--ceiling-only", action="store_true", help="time only those read kernels (for profiling)")
    ap.add_argument("--decode-only", action="store_true", help="time only the decode step (for profiling)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (known size) so that FETCH_SIZE / WRITE_SIZE "
                         "counters of a profiled run can be scaled")
    ap.add_argument("--timeline", action="store_true",
                    help="not a timing run: load the instrumented library (libglm_attn_timeline.so), run the decode "
                         "step and a causal prompt once and print where the waves' time went (in-kernel clock)")
    args = ap.parse_args()
    if args.ceiling_only:
        args.ceiling = True
    if args.decode_only or args.ceiling_only:
        args.skip_cpu = args.skip_prefill = args.skip_linear = args.skip_layer = args.skip_model = True
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)

    import torch

    from __graft_entry__ import load_package

    pkg = load_package()
    if args.timeline:
        import chatglm_cpp_amd.capi as capi

        capi.use_timeline_build()
    pkg.lib()  # fails loudly if libglm_attn.so is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.timeline:
        print(json.dumps({"timeline": timelines(torch, pkg, capi)}))
        return
    dev = torch.device("cuda:0")
    torch.cuda.set_device(0)

    L = MAX_LENGTH
    layer_halfs = 2 * KVH * L * D
    kv = torch.empty(LAYERS * layer_halfs, dtype=torch.int16, device=dev)
    fill_cache_normal(torch, kv, 0xC0FFEE)
    ctx = pkg.Context(num_layers=LAYERS, num_attention_heads=H, num_key_value_heads=KVH, head_size=D, max_length=L,
                      max_qlen=PREFILL_Q, kv_buffer=kv.data_ptr())
    width = (H + 2 * KVH) * D
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    result = {}

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    stream = torch.cuda.Stream()
    sh = stream.cuda_stream

    # ------------------------------------------------------------------ read ceilings
    if args.ceiling:
        with optional_section(result, "ceiling"):
            result["ceiling"] = read_ceilings(torch, pkg, kv, layer_halfs, stream, args.warmup, args.steps)
            result["ceiling"]["mfma"] = mfma_ceilings(torch, pkg, stream)

    # ------------------------------------------------------------------ decode
    if not args.prefill_only and not args.ceiling_only:
        qkv = torch.randn(LAYERS, width, generator=gen, device=dev, dtype=torch.float32)
        out = torch.zeros(LAYERS, H * D, device=dev, dtype=torch.float32)
        pos_host = [N_PAST_DECODE]
        qkv_ptrs = [qkv[l].data_ptr() for l in range(LAYERS)]
        out_ptrs = [out[l].data_ptr() for l in range(LAYERS)]

        def step():
            for l in range(LAYERS):
                st = ctx.forward(l, qkv_ptrs[l], 1, N_PAST_DECODE, out_ptrs[l], position_ids_host=pos_host,
                                 stream=sh)
                if st != 0:
                    pkg.check(st, "glm_attn_forward")

        def timed(fn, warmup, steps):
            with torch.cuda.stream(stream):
                for _ in range(warmup):
                    fn()
                torch.cuda.synchronize()
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(steps):
                    fn()
                e1.record(stream)
                torch.cuda.synchronize()
            return e0.elapsed_time(e1) / steps  # ms per step

        eager_ms = timed(step, args.warmup, args.steps)
        graph_ms = None
        if not args.no_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(stream):
                step()
                torch.cuda.synchronize()
                with torch.cuda.graph(graph, stream=stream):
                    step()
            graph_ms = timed(graph.replay, args.warmup, args.steps)
        assert bool(torch.isfinite(out).all()), "decode produced non-finite output"
        ms = eager_ms if graph_ms is None else min(graph_ms, eager_ms)
        mode = "eager" if (graph_ms is None or eager_ms <= graph_ms) else "hip graph replay"
        bytes_layer = decode_bytes_per_layer(N_PAST_DECODE + 1)
        bytes_token = bytes_layer * LAYERS
        gbs = bytes_token / (ms * 1e-3) / 1e9
        result.update({
            "metric": "decode attn+append HBM GB/s (GLM-4-9B, 32k ctx)",
            "value": round(gbs, 1),
            "unit": "GB/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(ms, 5),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "f16",
            "data": "synthetic",
            "config": {"workload": "GLM-4-9B decode, 40 layers, h32/kvh2/d128, n_past=32767, max_length=32768, "
                                   "one token per step, one launch per layer",
                       "launch_mode": mode},
            "us_per_token": round(ms * 1e3, 2),
            "us_per_layer": round(ms * 1e3 / LAYERS, 3),
            "eager_us_per_token": round(eager_ms * 1e3, 2),
            "graph_us_per_token": None if graph_ms is None else round(graph_ms * 1e3, 2),
            "roofline": {
                "bound": "hbm",
                "kernel": "decode_kernel",
                "achieved": round(bytes_layer / (ms * 1e-3 / LAYERS) / 1e9, 1),
                "peak": HBM_PEAK_GBS,
                "unit": "GB/s",
                "frac": round(bytes_layer / (ms * 1e-3 / LAYERS) / 1e9 / HBM_PEAK_GBS, 4),
                "bytes_per_launch": bytes_layer,
                "traffic": decode_traffic_bytes_per_launch(),
                "traffic_source": DECODE_TRAFFIC_PROFILE,
            },
        })

    # ------------------------------------------------------------------ prefill chunk
    if not args.skip_prefill:
        qlen, n_past = PREFILL_Q, PREFILL_N_PAST
        n_layers_pf = 2
        qkv_pf = torch.randn(qlen, width, generator=gen, device=dev, dtype=torch.float32)
        out_pf = torch.zeros(qlen, H * D, device=dev, dtype=torch.float32)
        pos_pf = torch.arange(n_past, n_past + qlen, device=dev, dtype=torch.int32)

        def pf_step():
            for l in range(n_layers_pf):
                st = ctx.forward(l, qkv_pf.data_ptr(), qlen, n_past, out_pf.data_ptr(),
                                 position_ids_ptr=pos_pf.data_ptr(), stream=sh)
                if st != 0:
                    pkg.check(st, "glm_attn_forward")

        with torch.cuda.stream(stream):
            pf_warmup = 3  # the shader clock takes a few of these 5 ms dispatches to settle
            for _ in range(pf_warmup):
                pf_step()
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            reps = 5
            e0.record(stream)
            for _ in range(reps):
                pf_step()
            e1.record(stream)
            torch.cuda.synchronize()
        pf_ms = e0.elapsed_time(e1) / (reps * n_layers_pf)
        assert bool(torch.isfinite(out_pf).all()), "prefill produced non-finite output"
        flops = prefill_flops_per_layer(qlen, n_past, causal=False)  # the reference leaves a continuation unmasked
        tflops = flops / (pf_ms * 1e-3) / 1e12
        result["prefill"] = {
            "workload": "one 8192-token chunk at n_past=24576 (unmasked, as the reference computes it), per layer",
            "ms_per_layer": round(pf_ms, 4),
            "tokens_per_s": round(qlen / (pf_ms * 1e-3), 1),
            "tflops": round(tflops, 1),
            "roofline": {"bound": "mfma", "kernel": "prefill_kernel", "achieved": round(tflops, 1),
                         "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tflops / MFMA_FP16_PEAK_TFLOPS, 4), "flops_per_launch": flops},
        }
        if args.prefill_only:
            result.update({"metric": "prefill attention TFLOP/s (GLM-4-9B, 8192-token chunk at 24576)",
                           "value": round(tflops, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": reps, "warmup": pf_warmup,
                           "ms_per_step": round(pf_ms, 4), "higher_is_better": True, "scaling": "weak",
                           "vs_baseline": None, "dtype": "f16", "data": "synthetic",
                           "config": {"workload": result["prefill"]["workload"]},
                           "roofline": result["prefill"]["roofline"]})

    # ------------------------------------------------------------------ causal prompt (BASELINE config 2)
    if not args.skip_prefill and not args.prefill_only:
        with optional_section(result, "prefill_causal_2048"):
            c_layers, c_h, c_kvh, c_len, c_q = 4, 32, 2, 8192, 2048
            ctx2 = pkg.Context(num_layers=c_layers, num_attention_heads=c_h, num_key_value_heads=c_kvh, head_size=D,
                               max_length=c_len, max_qlen=c_q)
            c_width = (c_h + 2 * c_kvh) * D
            qkv_c = torch.randn(c_layers, c_q, c_width, generator=gen, device=dev, dtype=torch.float32)
            out_c = torch.zeros(c_layers, c_q, c_h * D, device=dev, dtype=torch.float32)
            pos_c = torch.arange(c_q, device=dev, dtype=torch.int32)

            def c_forward():
                for l in range(c_layers):
                    st = ctx2.forward(l, qkv_c[l].data_ptr(), c_q, 0, out_c[l].data_ptr(),
                                      position_ids_ptr=pos_c.data_ptr(), stream=sh)
                    if st != 0:
                        pkg.check(st, "glm_attn_forward")

            def c_rope():
                for l in range(c_layers):
                    st = ctx2.rope_append(l, qkv_c[l].data_ptr(), pos_c.data_ptr(), c_q, 0, stream=sh)
                    if st != 0:
                        pkg.check(st, "glm_attn_rope_append")

            def c_time(fn):
                with torch.cuda.stream(stream):
                    for _ in range(3):
                        fn()
                    torch.cuda.synchronize()
                    e0 = torch.cuda.Event(enable_timing=True)
                    e1 = torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for _ in range(10):
                        fn()
                    e1.record(stream)
                    torch.cuda.synchronize()
                return e0.elapsed_time(e1) * 1e3 / (10 * c_layers)  # us per layer

            def c_attend():
                for l in range(c_layers):
                    st = ctx2.attend(l, c_q, 0, out_c[l].data_ptr(), stream=sh)
                    if st != 0:
                        pkg.check(st, "glm_attn_attend")

            us_call, us_rope = c_time(c_forward), c_time(c_rope)
            us_attend = c_time(c_attend)  # the queries of the last rope_append are still in the context's scratch
            assert bool(torch.isfinite(out_c).all()), "causal prompt produced non-finite output"
            c_flops = 4 * c_h * D * (c_q * (c_q + 1) // 2)
            us_kernel = us_attend
            result["prefill_causal_2048"] = {
                "workload": "ChatGLM3-6B shape (32 heads, 2 KV groups, max_length 8192): one 2048-token chunk at "
                            "n_past=0, causal, per layer",
                "us_per_layer": round(us_call, 2),
                "rope_append_us": round(us_rope, 2),
                "tokens_per_s": round(c_q / (us_call * 1e-6), 1),
                "tflops_whole_call": round(c_flops / us_call / 1e6, 1),
                "roofline": {"bound": "mfma", "kernel": "prefill_kernel",
                             "duration": "glm_attn_attend alone (the second launch of the call), events around "
                                         "back-to-back launches over 4 layers",
                             "us_per_launch": round(us_attend, 2),
                             "achieved": round(c_flops / us_kernel / 1e6, 1), "peak": MFMA_FP16_PEAK_TFLOPS,
                             "unit": "TFLOP/s", "frac": round(c_flops / us_kernel / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4),
                             "flops_per_launch": c_flops},
            }
            ctx2.close()

    # ------------------------------------------------------------------ the projections either side of the path
    if not args.skip_linear and not args.prefill_only:
        with optional_section(result, "linear"):
            hidden = H * D
            n_lin = 8  # distinct layers' weights, cycled: 8 x 71 MB is beyond the 256 MB Infinity Cache
            w_qkv = (torch.randn(n_lin, width, hidden, generator=gen, device=dev) * 0.02).to(torch.float16)
            w_dense = (torch.randn(n_lin, hidden, hidden, generator=gen, device=dev) * 0.02).to(torch.float16)
            b_qkv = torch.randn(width, generator=gen, device=dev)
            lin_qkv = [pkg.Linear(hidden, width, weight_dtype=pkg.LINEAR_F16, use_bias=True, max_rows=PREFILL_Q,
                                  weight=w_qkv[i].data_ptr(), bias=b_qkv.data_ptr()) for i in range(n_lin)]
            lin_dense = [pkg.Linear(hidden, hidden, weight_dtype=pkg.LINEAR_F16, use_bias=False, max_rows=PREFILL_Q,
                                    weight=w_dense[i].data_ptr()) for i in range(n_lin)]
            x = torch.randn(PREFILL_Q, hidden, generator=gen, device=dev)
            y_qkv = torch.zeros(PREFILL_Q, width, device=dev)
            y_dense = torch.zeros(PREFILL_Q, hidden, device=dev)
            torch.cuda.synchronize()  # made on torch's default stream; the steps run on `stream`

            def lin_step(rows):
                for i in range(n_lin):
                    for lin, y in ((lin_qkv[i], y_qkv), (lin_dense[i], y_dense)):
                        st = lin.forward(x.data_ptr(), rows, y.data_ptr(), stream=sh)
                        if st != 0:
                            pkg.check(st, "glm_linear_forward")

            def lin_time(rows, warm, reps):
                with torch.cuda.stream(stream):
                    for _ in range(warm):
                        lin_step(rows)
                    torch.cuda.synchronize()
                    e0 = torch.cuda.Event(enable_timing=True)
                    e1 = torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for _ in range(reps):
                        lin_step(rows)
                    e1.record(stream)
                    torch.cuda.synchronize()
                return e0.elapsed_time(e1) / (reps * n_lin)  # ms per layer (both projections)

            ms1 = lin_time(1, 3, 10)
            bytes1 = (width + hidden) * hidden * 2 + (2 * hidden + width + hidden) * 4 + width * 4
            msp = lin_time(PREFILL_Q, 2, 3)
            flop_p = 2.0 * PREFILL_Q * hidden * (width + hidden)
            assert bool(torch.isfinite(y_qkv).all()) and bool(torch.isfinite(y_dense).all())
            result["linear"] = {
                "workload": "query_key_value (4096 -> 4608, bias) + dense (4096 -> 4096) of one GLM-4-9B layer, fp16 "
                            "weights, fp32 activations, 8 layers' weights cycled",
                "decode_us_per_layer": round(ms1 * 1e3, 2),
                "decode_roofline": {"bound": "hbm", "kernel": "gemv_f16_kernel", "achieved": round(bytes1 / ms1 / 1e6, 1),
                                    "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                    "frac": round(bytes1 / ms1 / 1e6 / HBM_PEAK_GBS, 4), "bytes_per_layer": bytes1},
                "prefill_ms_per_layer": round(msp, 4),
                "prefill_roofline": {"bound": "mfma", "kernel": "gemm_f16_kernel after round_rows_kernel", "achieved": round(flop_p / msp / 1e9, 1),
                                     "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                     "frac": round(flop_p / msp / 1e9 / MFMA_FP16_PEAK_TFLOPS, 4),
                                     "rows": PREFILL_Q, "flops_per_layer": flop_p},
            }
            for lin in lin_qkv + lin_dense:
                lin.close()

    # ------------------------------------------------------------------ whole decoder layers, one token
    if not args.skip_layer and not args.prefill_only:
        with optional_section(result, "layer"):
            # BasicBlock<RMSNorm, BasicGLU>::forward (chatglm.h:488-503) of GLM-4-9B for one token at n_past = 32767,
            # 40 layers with 8 layers' fp16 weights cycled (8 x 408 MB, beyond the Infinity Cache) and 40 distinct caches
            hidden, inter, n_w = H * D, 13696, 8
            lib = pkg.lib()

            def rand_w(n_out, n_in):
                return (torch.randn(n_w, n_out, n_in, generator=gen, device=dev) * 0.02).to(torch.float16)

            w_qkv, w_dense = rand_w(width, hidden), rand_w(hidden, hidden)
            w_gate, w_up, w_down = rand_w(inter, hidden), rand_w(inter, hidden), rand_w(hidden, inter)
            b_qkv = torch.randn(width, generator=gen, device=dev) * 0.02
            ln_w = torch.ones(hidden, device=dev)

            def mk(w, i, n_in, n_out, bias=None):
                return pkg.Linear(n_in, n_out, weight_dtype=pkg.LINEAR_F16, use_bias=bias is not None, max_rows=1,
                                  weight=w[i].data_ptr(), bias=bias.data_ptr() if bias is not None else None)

            lins = [dict(qkv=mk(w_qkv, i, hidden, width, b_qkv), dense=mk(w_dense, i, hidden, hidden),
                         gate=mk(w_gate, i, hidden, inter), up=mk(w_up, i, hidden, inter),
                         down=mk(w_down, i, inter, hidden)) for i in range(n_w)]
            t = {k: torch.zeros(n, device=dev) for k, n in
                 dict(h=hidden, x=hidden, qkv=width, ctx=hidden, a=hidden, h2=hidden, g=inter, u=inter, m=hidden).items()}
            t["h"].copy_(torch.randn(hidden, generator=gen, device=dev))
            h0 = t["h"].clone()
            torch.cuda.synchronize()  # these tensors were made on torch's default stream; the steps run on `stream`
            p = {k: v.data_ptr() for k, v in t.items()}
            pos_host = [N_PAST_DECODE]

            def ok(st, what):
                if st != 0:
                    pkg.check(st, what)

            def layer_step(n_layers=LAYERS):
                for l in range(n_layers):
                    m = lins[l % n_w]
                    ok(lib.glm_block_rms_norm(p["h"], ln_w.data_ptr(), 1e-5, 1, hidden, p["x"], sh), "rms_norm")
                    ok(m["qkv"].forward(p["x"], 1, p["qkv"], stream=sh), "qkv")
                    ok(ctx.forward(l, p["qkv"], 1, N_PAST_DECODE, p["ctx"], position_ids_host=pos_host, stream=sh), "attn")
                    ok(m["dense"].forward(p["ctx"], 1, p["a"], stream=sh), "dense")
                    ok(lib.glm_attn_scale_add(p["h2"], p["a"], 1.0, p["h"], hidden, sh), "add")
                    ok(lib.glm_block_rms_norm(p["h2"], ln_w.data_ptr(), 1e-5, 1, hidden, p["x"], sh), "rms_norm")
                    ok(m["gate"].forward(p["x"], 1, p["g"], stream=sh), "gate")
                    ok(m["up"].forward(p["x"], 1, p["u"], stream=sh), "up")
                    ok(lib.glm_block_gated_activation(p["g"], p["u"], inter, pkg.ACT_SILU, p["u"], sh), "silu_mul")
                    ok(m["down"].forward(p["u"], 1, p["m"], stream=sh), "down")
                    ok(lib.glm_attn_scale_add(p["h"], p["m"], 1.0, p["h2"], hidden, sh), "add")

            f_norm = pkg.make_fusion(prologue=pkg.PRO_RMS_NORM, norm_weight=ln_w.data_ptr(), norm_eps=1e-5)
            f_res_h = pkg.make_fusion(residual=p["h"], residual_scale=1.0)
            f_glu = pkg.make_fusion(prologue=pkg.PRO_RMS_NORM, norm_weight=ln_w.data_ptr(), norm_eps=1e-5,
                                    activation=pkg.ACT_SILU)
            f_res_h2 = pkg.make_fusion(residual=p["h2"], residual_scale=1.0)

            def fused_layer_step(n_layers=LAYERS):
                # the same arithmetic in 5 launches: the norms run inside the projections that consume them, the gate and
                # up projections share a launch that also applies the activation, the residual sums run inside the
                # projections that produce their other operand
                for l in range(n_layers):
                    m = lins[l % n_w]
                    ok(m["qkv"].forward_fused(f_norm, p["h"], 1, p["qkv"], stream=sh), "norm+qkv")
                    ok(ctx.forward(l, p["qkv"], 1, N_PAST_DECODE, p["ctx"], position_ids_host=pos_host, stream=sh), "attn")
                    ok(m["dense"].forward_fused(f_res_h, p["ctx"], 1, p["h2"], stream=sh), "dense+residual")
                    ok(m["gate"].forward_glu(m["up"], f_glu, p["h2"], 1, p["u"], stream=sh), "norm+gate/up+silu_mul")
                    ok(m["down"].forward_fused(f_res_h2, p["u"], 1, p["h"], stream=sh), "down+residual")

            def layer_time(warm, reps, graph, step):
                with torch.cuda.stream(stream):
                    run = step
                    t["h"].copy_(h0)
                    if graph:
                        step()
                        torch.cuda.synchronize()
                        t["h"].copy_(h0)
                        g = torch.cuda.CUDAGraph()
                        with torch.cuda.graph(g, stream=stream):
                            step()
                        run = g.replay
                    for _ in range(warm):
                        run()
                    torch.cuda.synchronize()
                    e0 = torch.cuda.Event(enable_timing=True)
                    e1 = torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for _ in range(reps):
                        run()
                    e1.record(stream)
                    torch.cuda.synchronize()
                return e0.elapsed_time(e1) / reps

            # the two forms give the same hidden state (same operations, same order within each sum); compared after
            # two layers: through 40 layers of random weights a last-bit difference of a norm's sum can grow at will
            with torch.cuda.stream(stream):
                t["h"].copy_(h0)
                layer_step(2)
                h_sep = t["h"].clone()
                t["h"].copy_(h0)
                fused_layer_step(2)
                torch.cuda.synchronize()
            assert bool(torch.isfinite(h_sep).all())
            err, top = float((t["h"] - h_sep).abs().max()), float(h_sep.abs().max())
            assert err <= 1e-3 * top, (err, top)
            ms_separate = layer_time(2, 10, False, layer_step)
            ms_eager = layer_time(2, 10, False, fused_layer_step)
            ms_graph = None if args.no_graph else layer_time(2, 10, True, fused_layer_step)
            ms_tok = min(ms_eager, ms_graph) if ms_graph is not None else ms_eager
            assert bool(torch.isfinite(t["h"]).all())
            w_bytes = (width + hidden + 3 * inter) * hidden * 2
            result["layer"] = {
                "workload": "GLM-4-9B decoder stack, one token at n_past=32767: 40 x (RMSNorm, QKV, attention, dense, "
                            "residual, RMSNorm, gate/up, SiLU-gate, down, residual), fp16 weights (8 layers' cycled), "
                            "fp32 activations; no embedding, LM head or sampling; 5 launches per layer (norms, gate and "
                            "residuals inside the projections)",
                "ms_per_token": round(ms_tok, 4),
                "separate_launches_eager_ms_per_token": round(ms_separate, 4),
                "eager_ms_per_token": round(ms_eager, 4),
                "graph_ms_per_token": None if ms_graph is None else round(ms_graph, 4),
                "us_per_layer": round(ms_tok * 1e3 / LAYERS, 2),
                "bytes_per_layer": w_bytes + bytes_layer,
                "hbm_gbs": round((w_bytes + bytes_layer) * LAYERS / ms_tok / 1e6, 1),
                "frac_of_hbm_peak": round((w_bytes + bytes_layer) * LAYERS / ms_tok / 1e6 / HBM_PEAK_GBS, 4),
            }
            for m in lins:
                for lin in m.values():
                    lin.close()

    # ------------------------------------------------------------------ whole model through the C++ host classes
    if not args.skip_model and not args.prefill_only:
        with optional_section(result, "model"):
            # embedding, 40 blocks, final norm, LM head; ids in, logits out, per token at n_past = 32767, and a
            # 2048-token prompt: a separate process (chatglm.cpp_amd/host/bench_model.cpp), run after this one's tensors
            # are released so that the 19 GB of weights fit beside nothing else
            import subprocess

            exe = os.path.join(ROOT, "chatglm.cpp_amd", "bench_model")
            if not os.path.exists(exe):
                raise RuntimeError("chatglm.cpp_amd/bench_model is not built (run __graft_entry__.build())")
            # (--followup 20: also one forward of 20 new tokens on top of the 32767 cached ones)
            r = subprocess.run([exe, "--n-past", str(N_PAST_DECODE), "--tokens", "20", "--warmup", "3", "--prompt", "2048",
                                "--followup", "20"], capture_output=True, text=True, timeout=600)
            if r.returncode != 0:
                raise RuntimeError("bench_model failed: " + r.stderr[-1000:])
            result["model"] = json.loads(r.stdout.strip().splitlines()[-1])
            assert result["model"]["finite"]
            # the same model with the converter's default weight type (ggml's q4_0 blocks), one token only
            r = subprocess.run([exe, "--dtype", "q4_0", "--n-past", str(N_PAST_DECODE), "--tokens", "20", "--warmup", "3",
                                "--prompt", "0"], capture_output=True, text=True, timeout=600)
            if r.returncode != 0:
                raise RuntimeError("bench_model --dtype q4_0 failed: " + r.stderr[-1000:])
            result["model_q4_0"] = json.loads(r.stdout.strip().splitlines()[-1])
            assert result["model_q4_0"]["finite"]

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    if not args.skip_cpu and not args.prefill_only:
        import numpy as np

        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import glm_oracle as orc

        threads = orc.reference_threads(1)  # the reference's decode policy: min(physical cores, 16)
        ocfg = orc.make_cfg(num_attention_heads=H, num_key_value_heads=KVH, head_size=D, max_length=L,
                            n_threads=threads)
        k_ref, v_ref = orc.new_caches(ocfg)
        k_ref[:, :N_PAST_DECODE, :] = orc.randn_f16_bits(1, 1, KVH * N_PAST_DECODE * D).reshape(KVH, N_PAST_DECODE, D)
        v_ref[:, :, :N_PAST_DECODE] = orc.randn_f16_bits(1, 2, KVH * D * N_PAST_DECODE).reshape(KVH, D, N_PAST_DECODE)
        q_cpu = orc.randn_f32(1, 0, width).reshape(1, width)
        pos = orc.position_ids_glm2(1, N_PAST_DECODE)
        # 8 layers' caches (270 MB) taken in turn, so that the CPU streams them from memory as a 40-layer model would
        caches = [(k_ref, v_ref)] + [(k_ref.copy(), v_ref.copy()) for _ in range(7)]
        orc.attention_forward(ocfg, q_cpu.copy(), pos, N_PAST_DECODE, k_ref, v_ref)  # warm-up 1
        t0 = time.perf_counter()
        reps = 0
        while reps < 3 or (time.perf_counter() - t0 < 12.0 and reps < 100000):
            k_c, v_c = caches[reps % len(caches)]
            orc.attention_forward(ocfg, q_cpu.copy(), pos, N_PAST_DECODE, k_c, v_c)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        result["cpu_baseline"] = {
            "value": round(decode_bytes_per_layer(N_PAST_DECODE + 1) / cpu_s / 1e9, 2),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "us_per_token": round(cpu_s * LAYERS * 1e6, 1),
            "sample": f"single layers of the decode workload for 12 s: {reps} timed passes after 1 warm-up over 8 "
                      f"layers' caches in turn (CPU restatement of the reference graph, {threads} threads of "
                      f"{os.cpu_count()} logical CPUs); us_per_token = 40 x the per-layer time",
        }

    # ------------------------------------------------------------------ CPU beside the prefill chunk (bounded sample)
    if not args.skip_cpu and not args.skip_prefill and "prefill" in result:
        import numpy as np

        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import glm_oracle as orc

        qlen, n_past = PREFILL_Q, PREFILL_N_PAST
        threads = orc.reference_threads(qlen)  # the reference's prompt policy: the physical cores (chatglm.cpp:476-499)
        ocfg = orc.make_cfg(num_attention_heads=H, num_key_value_heads=KVH, head_size=D, max_length=L,
                            n_threads=threads)
        k_ref, v_ref = orc.new_caches(ocfg)
        k_ref[:, :n_past, :] = orc.randn_f16_bits(3, 1, KVH * n_past * D).reshape(KVH, n_past, D)
        v_ref[:, :, :n_past] = orc.randn_f16_bits(3, 2, KVH * D * n_past).reshape(KVH, D, n_past)
        qkv_cpu = orc.randn_f32(3, 0, qlen * width).reshape(qlen, width)
        pos = orc.position_ids_glm2(qlen, n_past)
        t0 = time.perf_counter()
        orc.rope_inplace(ocfg, qkv_cpu, pos)          # rope and append of the whole chunk: timed in full
        orc.append(ocfg, qkv_cpu, n_past, k_ref, v_ref)
        t_head = time.perf_counter() - t0
        block, rows_done = 64, 0
        out_cpu = np.zeros((qlen, H * D), dtype=np.float32)
        orc.attend(ocfg, qkv_cpu, n_past, k_ref, v_ref, rows=(qlen - 8, qlen), out=out_cpu)  # warm-up
        t0 = time.perf_counter()
        while rows_done < qlen and (rows_done < block or time.perf_counter() - t0 < 12.0):
            orc.attend(ocfg, qkv_cpu, n_past, k_ref, v_ref, rows=(rows_done, rows_done + block), out=out_cpu)
            rows_done += block
        t_rows = time.perf_counter() - t0
        cpu_layer_s = t_head + t_rows * qlen / rows_done
        pf_flops = prefill_flops_per_layer(qlen, n_past, causal=False)
        result["prefill"]["cpu_baseline"] = {
            "value": round(pf_flops / cpu_layer_s / 1e12, 4),
            "unit": "TFLOP/s",
            "tokens_per_s": round(qlen / cpu_layer_s, 1),
            "s_per_layer": round(cpu_layer_s, 2),
            "cores": threads,
            "kind": "port",
            "sample": f"rope and append of the whole 8192-token chunk ({t_head * 1e3:.0f} ms) plus the attention of "
                      f"its first {rows_done} token rows against all {n_past + qlen} keys ({t_rows:.1f} s), "
                      f"extrapolated to 8192 rows (every row costs the same: the chunk is unmasked); CPU restatement "
                      f"of the reference graph, {threads} threads of {os.cpu_count()} logical CPUs",
        }

    ctx.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
