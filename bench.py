#!/usr/bin/env python3
"""Benchmark of the HQMQ KV-cache hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--context 32768] [--n-splits 0]

A step is one fused decode-attention pass of one layer over the compressed cache of benchmark config 2
(Llama-3-8B shape: 32 query / 8 KV heads, d_h = 128, batch 1, s96_r4, fp16, context 32768, one query
token, causal=False).  Inputs (packed cache, query) are resident in HBM before the timed region.  The K
timed steps are captured in one HIP graph and replayed once, bracketed by torch.cuda.synchronize().

One JSON line is printed:
  value      = algorithmic compressed bytes per step / step time (GB/s), whole job on the one GPU
  roofline   = same bytes / the attention kernel's own average launch duration (HIP events on the launch
               stream around back-to-back launches of that kernel alone), against 8 TB/s
  cpu_baseline = the CPU restatement of the reference's torch path (decode to dense + SDPA) timed on this
               host over a token slice of the same cache
Extra keys report the quantize throughput (GTok/s, K and V of one layer) and the other contexts.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the attention kernel from the FETCH_SIZE / WRITE_SIZE passes (scaled by a plain
# 256 MiB copy), recorded in profiles/attn_fast_kernel_config2_32k_hbm_traffic.txt; known for these contexts only.
MEASURED_TRAFFIC_BYTES = {32768: 37.73e6}


def build_cache(q, T, dt, dev, seed):
    import torch
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(1, 8, T, 128, generator=g).to(dt).to(dev)
    v = torch.randn(1, 8, T, 128, generator=g).to(dt).to(dev)
    cache = q.new_cache(1, T, 128, dt, layer_idx=0)
    q.append(cache, k, v, 0)
    return cache, k, v


def event_time_us(fn, iters, stream):
    """Average duration of fn() over `iters` back-to-back calls, HIP events on the launch stream."""
    import torch
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(iters):
        fn()
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def kernel_time_us(launch, iters):
    """Average GPU duration of the attention kernel itself over `iters` back-to-back launches: every launch
    carries its own pair of HIP events, which the runtime stamps at the begin and at the end of that dispatch (the
    same interval a kernel trace reports; the gap between two dependent dispatches is not part of it)."""
    import ctypes as C
    import torch
    hip = C.CDLL("libamdhip64.so")
    ev = [(C.c_void_p(), C.c_void_p()) for _ in range(iters)]
    for a, b in ev:
        for e in (a, b):
            if hip.hipEventCreate(C.byref(e)) != 0:
                raise RuntimeError("hipEventCreate failed")
    for _ in range(3):
        launch(None)
    torch.cuda.synchronize()
    for a, b in ev:
        launch((a.value, b.value))
    torch.cuda.synchronize()
    total, ms = 0.0, C.c_float()
    for a, b in ev:
        if hip.hipEventElapsedTime(C.byref(ms), a, b) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        total += ms.value
        hip.hipEventDestroy(a)
        hip.hipEventDestroy(b)
    return total * 1e3 / iters


def cpu_baseline(T, slice_tokens, repeats=5):
    """Reference torch path on the host: dense decode of K and V, GQA broadcast, SDPA; slice of the context."""
    import torch
    from oracle import torch_oracle as TO
    dt = torch.float16
    g = torch.Generator().manual_seed(7)
    S, qmax, Hkv, n = 96, 15, 8, 32
    Jk = TO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, 0], dt)
    Jv = TO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, 1], dt)
    idx = torch.randint(0, 24 * S, (1, Hkv, slice_tokens, n), generator=g, dtype=torch.int32)
    rq = torch.randint(0, qmax + 1, (1, Hkv, slice_tokens, n), generator=g, dtype=torch.int32)
    rs = (torch.rand(1, Hkv, slice_tokens, generator=g) + 0.5).to(dt)
    Q = torch.randn(1, 32, 1, 128, generator=g).to(dt)
    times = []
    for i in range(2 + repeats):
        t0 = time.perf_counter()
        TO.attention(Q, idx, rq, rs, Jk, idx, rq, rs, Jv, qmax, causal=False)
        dtm = time.perf_counter() - t0
        if i >= 2:
            times.append(dtm)
    times.sort()
    return times[len(times) // 2]


def cpu_quantize_baseline(slice_tokens, repeats=3):
    import torch
    from oracle import torch_oracle as TO
    dt = torch.float16
    x = torch.randn(1, 8, slice_tokens, 128, generator=torch.Generator().manual_seed(8)).to(dt)
    J = TO.joint_table(TO.secondary_raw(1, 8, 96, 42)[0, :, 0], dt)
    times = []
    for i in range(1 + repeats):
        t0 = time.perf_counter()
        TO.quantize(x, J, 4)
        dtm = time.perf_counter() - t0
        if i >= 1:
            times.append(dtm)
    times.sort()
    return times[len(times) // 2]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--context", type=int, default=32768)
    ap.add_argument("--n-splits", type=int, default=0)
    ap.add_argument("--no-graph", action="store_true", help="launch every step from Python instead of one HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--all-contexts", action="store_true", help="also report 4k / 8k / 16k")
    ap.add_argument("--counters", action="store_true",
                    help="for rocprofv3 --pmc runs: only 20 eager attention steps and 5 plain 256 MiB copies (the "
                         "calibration kernel for FETCH_SIZE / WRITE_SIZE), no JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: every box of this build has one, and the path needs no second "
              f"(got --gpus {args.gpus}); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import hqmq
    from hqmq_amd import ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the HQMQ kernels have no CPU path", file=sys.stderr)
        sys.exit(1)
    dev, dt = "cuda:0", torch.float16
    torch.cuda.set_device(0)
    T = args.context
    q = hqmq.HQMQ(n_layers=1, n_heads=8, secondary_size=96, radius_bits=4, device=dev)
    cache, k, v = build_cache(q, T, dt, dev, seed=0)
    Q = torch.randn(1, 32, 1, 128, generator=torch.Generator().manual_seed(1)).to(dt).to(dev)
    out = torch.empty_like(Q)
    n_splits = args.n_splits or ops.pick_splits(1, 32, 8, 1, T)
    cache_bytes = cache.nbytes(T)
    step_bytes = cache_bytes + 2 * Q.numel() * Q.element_size()      # + Q read and O written

    def step():
        hqmq.fused_attention_packed(Q, cache, n_splits=n_splits, out=out)

    # correctness of what is being timed: dense SDPA over the dequantized cache
    step()
    Kd, Vd = ops.dequant_packed(cache.K, T, 0), ops.dequant_packed(cache.V, T, 0)
    ref = torch.nn.functional.scaled_dot_product_attention(Q, Kd.repeat_interleave(4, 1), Vd.repeat_interleave(4, 1))
    max_err = (out.float() - ref.float()).abs().max().item()
    del Kd, Vd
    if not max_err < 2e-3:
        print(f"attention output differs from dense SDPA by {max_err}", file=sys.stderr)
        sys.exit(1)

    stream = torch.cuda.current_stream()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if args.counters:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(20):
            step()
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(f"counters mode: 20 attention steps of {cache_bytes} compressed bytes, 5 copies of {src.numel()} bytes")
        return
    used_graph = False
    if not args.no_graph:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(stream)
            with torch.cuda.stream(side):
                step()
            stream.wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(args.steps):
                    step()
            graph.replay()                      # one untimed replay
            torch.cuda.synchronize()
            used_graph = True
        except Exception as e:                  # noqa: BLE001
            print(f"graph capture unavailable ({e}); timing eager launches", file=sys.stderr)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if used_graph:
        graph.replay()
    else:
        for _ in range(args.steps):
            step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    us_step = wall / args.steps * 1e6
    value = step_bytes / (us_step * 1e-6) / 1e9

    # the attention kernel alone (split partials left in the workspace), HIP events on its stream
    us_main = kernel_time_us(lambda ev: ops.attn_fwd(Q, cache.K, cache.V, T, n_splits=n_splits, out=out, skip_combine=True,
                                                     kernel_events=ev), 200)
    us_back_to_back = event_time_us(lambda: ops.attn_fwd(Q, cache.K, cache.V, T, n_splits=n_splits, out=out,
                                                         skip_combine=True), 200, stream)
    us_both = event_time_us(step, 200, stream)
    achieved = cache_bytes / (us_main * 1e-6) / 1e9

    # quantize throughput: K and V of one layer, bulk (prefill) call, packed output
    def quant():
        c = q.new_cache(1, T, 128, dt, 0)
        q.append(c, k, v, 0)
    c2 = q.new_cache(1, T, 128, dt, 0)

    def quant_only():
        c2.K.length = c2.V.length = 0
        q.append(c2, k, v, 0)
    us_quant = event_time_us(quant_only, 10, stream)
    gtok_s = T / (us_quant * 1e-6) / 1e9

    result = {
        "metric": "decode-attn HBM GB/s on compressed bytes (us/step and % of 8 TB/s alongside); quantize GTok/s",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_step / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"BASELINE config 2: fused decode attention, Llama-3-8B shape (32 q / 8 kv heads, d_h 128, "
                               f"batch 1), s96_r4 fp16 cache, context {T}, one query token, one layer per step",
                   "context": T, "n_splits": n_splits, "hip_graph": used_graph,
                   "compressed_bytes_per_step": cache_bytes},
        "us_per_step": round(us_step, 2),
        "pct_of_hbm_roofline": round(100 * value / HBM_PEAK_GBPS, 2),
        "max_abs_err_vs_dense_sdpa": max_err,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(T),
                     "kernel": "attn_fast_kernel<8,16,0,f16>", "kernel_us": round(us_main, 2),
                     "kernel_launch_interval_us": round(us_back_to_back, 2),
                     "kernel_plus_combine_us": round(us_both, 2), "algorithmic_bytes_per_launch": cache_bytes},
        "quantize": {"GTok_per_s": round(gtok_s, 5), "us_per_call": round(us_quant, 1), "tokens": T,
                     "what": "K and V of one layer, 8 kv heads x d_h 128, s96_r4 fp16, quantize + pack"},
    }
    if args.all_contexts:
        other = {}
        for Tc in (4096, 8192, 16384):
            cc, _, _ = build_cache(q, Tc, dt, dev, seed=Tc)
            ns = ops.pick_splits(1, 32, 8, 1, Tc)
            us = event_time_us(lambda: hqmq.fused_attention_packed(Q, cc, n_splits=ns, out=out), 200, stream)
            other[str(Tc)] = {"us_per_step": round(us, 2), "GBps": round(cc.nbytes(Tc) / us / 1e3, 1), "n_splits": ns}
        result["other_contexts"] = other
    if not args.no_cpu_baseline:
        threads = torch.get_num_threads()
        slice_tokens = 4096
        sec = cpu_baseline(T, slice_tokens)
        slice_bytes = cache_bytes * slice_tokens / T
        qsec = cpu_quantize_baseline(128)
        result["cpu_baseline"] = {
            "value": round(slice_bytes / sec / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"torch restatement of the reference path (dense decode + SDPA), fp16, {slice_tokens} of {T} tokens, "
                      f"median of 5 after 2 warm-ups; os.cpu_count()={os.cpu_count()}",
            "us_per_step_scaled_to_full_context": round(sec * T / slice_tokens * 1e6, 1),
            "quantize_GTok_per_s": round(128 / (2 * qsec) / 1e9, 8),
            "quantize_sample": "one tensor of 128 tokens x 8 heads s96_r4 fp16, median of 3, time doubled for K and V",
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
