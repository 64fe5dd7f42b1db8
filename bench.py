#!/usr/bin/env python3
"""Benchmark of the HQMQ KV-cache hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--context 32768] [--layers 16] [--quick]

A step is one fused decode-attention pass of one layer over the compressed cache of benchmark config 2
(Llama-3-8B shape: 32 query / 8 KV heads, d_h = 128, batch 1, s96_r4, fp16, context 32768, one query token,
causal=False).  A decode step of a model walks a different layer's cache every time, so the timed steps rotate
over `--layers` distinct caches (16 x 34.6 MB = 554 MB, more than the 256 MB Infinity Cache and the L2s hold):
every step reads its cache from HBM.  Inputs (packed caches, queries) are resident in HBM before the timed
region; the K timed steps are captured in one HIP graph and replayed once between two torch.cuda.synchronize()
(host clock from the replay call to the completion of an event recorded behind the graph, see host_time_s).
Warm-up: the first 32 of the W warm-up steps are launched one by one, the rest as whole untimed replays of that same
graph ((W - 32) // K of them, at least one); the default W is 32 + 10 K, about 30 ms of the workload, because the
first replays after a start run 5 - 10 % slower than every later one (clocks still settling).

One JSON line is printed:
  value        = algorithmic compressed bytes per step / step time (GB/s), whole job on the one GPU, caches
                 rotating (read from HBM)
  roofline     = same bytes / the attention kernel's own average launch duration (a pair of HIP events per
                 launch, stamped by the runtime at the begin and the end of that dispatch), against 8 TB/s
  cpu_baseline = the CPU restatement of the reference's torch path (decode to dense + SDPA) timed on this host
                 over a token slice of the same cache, and its quantizer on benchmark config 1 in full
Extra keys: the same step replayed over one cache (resident in the Infinity Cache: an upper bound, labelled),
the contexts 4k / 8k / 16k, the batch-8 streaming rate, the quantize throughput, configs 3-5 at full size with and
without Med3x (hqmq_amd/bench_configs.py), and the one prefill shape the reference publishes a number for.
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
# HBM bytes per launch of the attention kernel as the FETCH_SIZE / WRITE_SIZE counters read them, recorded offline
# (rocprofv3 --pmc does not run inside this script); known for these contexts only.
TRAFFIC_FILE = "profiles/attn_lds_kernel_config2_32k_hbm_traffic.txt"
RECORDED_TRAFFIC_BYTES = {32768: 35.59e6}
Hq, Hkv, D_H, S, B_R = 32, 8, 128, 96, 4


def kv_pair(T, dt, dev, seed, B=1):
    import torch
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, Hkv, T, D_H, generator=g).to(dt).to(dev)
    v = torch.randn(B, Hkv, T, D_H, generator=g).to(dt).to(dev)
    return k, v


def build_layers(q, T, dt, dev, n_layers, B=1):
    """One packed cache and one query per layer (CPU-seeded inputs)."""
    import torch
    caches, queries = [], []
    for layer in range(n_layers):
        k, v = kv_pair(T, dt, dev, 1000 * layer + T % 997, B)
        cache = q.new_cache(B, T, D_H, dt, layer_idx=layer)
        q.append(cache, k, v, layer)
        caches.append(cache)
        queries.append(torch.randn(B, Hq, 1, D_H, generator=torch.Generator().manual_seed(7 + layer)).to(dt).to(dev))
    return caches, queries


def graph_us(fn, steps, stream, replays=1, warm_replays=1):
    """Time per step of `steps` calls fn(i) captured in one HIP graph (`warm_replays` untimed replays first); falls
    back to eager launches when capture is unavailable.  replays > 1: the graph is replayed that many times, each replay
    timed on its own, and the median is returned (the figures beside the headline: the first replays of a workload run
    before the clocks have settled, by up to 20 % for the long launches).  Returns (us per step, used_graph)."""
    import torch
    graph = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            fn(0)
        stream.wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(steps):
                fn(i)
        for _ in range(max(1, warm_replays)):
            graph.replay()
        torch.cuda.synchronize()
    except Exception as e:                  # noqa: BLE001
        print(f"graph capture unavailable ({e}); timing eager launches", file=sys.stderr)
        graph = None
    def run():
        if graph is not None:
            graph.replay()
        else:
            for i in range(steps):
                fn(i)
    times = sorted(host_time_s(run) / steps * 1e6 for _ in range(max(1, replays)))
    return times[len(times) // 2], graph is not None


def host_time_s(run):
    """Host wall time of the GPU work that run() enqueues, between two torch.cuda.synchronize().  The clock stops
    when an event recorded behind the work reports completion to a polling host: a blocking synchronize returns
    20 - 40 us after the work has ended (the time the host needs to wake up), which is 1 - 2 us per step when only 20
    steps are timed."""
    import torch
    done = torch.cuda.Event()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run()
    done.record()
    while not done.query():
        pass
    t1 = time.perf_counter()
    torch.cuda.synchronize()
    return t1 - t0


def event_time_us(fn, iters, stream):
    """Average duration of fn(i) over `iters` back-to-back calls, HIP events on the launch stream."""
    import torch
    for i in range(3):
        fn(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for i in range(iters):
        fn(i)
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


LAST_KERNEL_STATS = {}


def kernel_time_us(launch, iters):
    """Median GPU duration of the attention kernel itself over `iters` launches launch(i, events): every launch
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
    for i in range(3):
        launch(i, None)
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(ev):
        launch(i, (a.value, b.value))
    torch.cuda.synchronize()
    durs, ms = [], C.c_float()
    for a, b in ev:
        if hip.hipEventElapsedTime(C.byref(ms), a, b) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        durs.append(ms.value * 1e3)
        hip.hipEventDestroy(a)
        hip.hipEventDestroy(b)
    # The median of all launches is what is reported (eager launches are paced by the host, and now and then one is
    # stretched by whatever else the device did between them); the plain mean, the maximum and the mean without the
    # launches beyond 1.5 x the median go into LAST_KERNEL_STATS, nothing is left out of the figure itself.
    med = sorted(durs)[len(durs) // 2]
    kept = [d for d in durs if d <= 1.5 * med]
    LAST_KERNEL_STATS.update(mean_all=sum(durs) / len(durs), median=med, max=max(durs), min=min(durs),
                             mean_without_stretched=sum(kept) / len(kept), stretched=len(durs) - len(kept), launches=len(durs))
    return med


def cpu_attention_baseline(slice_tokens, repeats=5):
    """Reference torch path on the host: dense decode of K and V, GQA broadcast, SDPA; slice of the context."""
    import torch
    from oracle import torch_oracle as TO
    dt = torch.float16
    g = torch.Generator().manual_seed(7)
    qmax, n = (1 << B_R) - 1, D_H // 4
    Jk = TO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, 0], dt)
    Jv = TO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, 1], dt)
    idx = torch.randint(0, 24 * S, (1, Hkv, slice_tokens, n), generator=g, dtype=torch.int32)
    rq = torch.randint(0, qmax + 1, (1, Hkv, slice_tokens, n), generator=g, dtype=torch.int32)
    rs = (torch.rand(1, Hkv, slice_tokens, generator=g) + 0.5).to(dt)
    Q = torch.randn(1, Hq, 1, D_H, generator=g).to(dt)
    times = []
    for i in range(2 + repeats):
        t0 = time.perf_counter()
        TO.attention(Q, idx, rq, rs, Jk, idx, rq, rs, Jv, qmax, causal=False)
        dtm = time.perf_counter() - t0
        if i >= 2:
            times.append(dtm)
    times.sort()
    return times[len(times) // 2]


def config1_inputs():
    """Benchmark config 1: K and V of one layer, Mistral-7B shape (8 KV heads, d_h 128, batch 1, 2048 tokens), fp16
    ~N(0,1) with lognormal(0, 0.5) channel scales; CPU-seeded, the same tensors for the GPU and the CPU leg."""
    import torch
    from tests.helpers import kv_input
    return kv_input((1, 8, 2048, 128), torch.float16, 1), kv_input((1, 8, 2048, 128), torch.float16, 2)


def cpu_quantize_baseline_config1(repeats=3):
    """Benchmark config 1 in full on the host: s24_r3 with Med3x (C = 3), the restated reference quantizer
    (reference: src/quantizers/hqmq.py:145-216, outlier_aware.py:56-87), median of `repeats` after one warm-up.
    Returns (seconds for K and V, tokens, MSE of the dequantized K and V against the input)."""
    import torch
    from oracle import torch_oracle as TO
    k, v = config1_inputs()
    T = k.shape[2]
    raw = TO.secondary_raw(1, 8, 24, 42)
    Jk, Jv = TO.joint_table(raw[0, :, 0], k.dtype), TO.joint_table(raw[0, :, 1], k.dtype)
    times, mse = [], None
    for i in range(1 + repeats):
        t0 = time.perf_counter()
        rk = TO.outlier_quantize(k, Jk, 3, 3.0)
        rv = TO.outlier_quantize(v, Jv, 3, 3.0)
        dtm = time.perf_counter() - t0
        if i >= 1:
            times.append(dtm)
        mse = (float(((rk["out"].float() - k.float()) ** 2).mean()), float(((rv["out"].float() - v.float()) ** 2).mean()))
    times.sort()
    return times[len(times) // 2], T, mse


def gpu_config1(dev, calls=10):
    """Benchmark config 1 on the GPU: quantize + Med3x (C = 3) + pack of K and V of one layer into a packed cache
    (one bulk append), then the dequantized KV and its MSE against the input, outlier rate and bits per value."""
    import torch
    import hqmq
    from hqmq_amd import ops
    k, v = config1_inputs()
    k, v = k.to(dev), v.to(dev)
    T, d = k.shape[2], k.shape[3]
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=8, secondary_size=24, radius_bits=3, device=dev), C=3.0)
    fresh = [w.new_cache(1, T, d, k.dtype, 0) for _ in range(calls + 3)]
    for c in fresh[:3]:
        w.append(c, k, v, 0)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for c in fresh[3:]:
        w.append(c, k, v, 0)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / calls
    cache = fresh[-1]
    cache.K.check_overflow()
    cache.V.check_overflow()
    Kd, Vd = ops.dequant_packed(cache.K, T, 1), ops.dequant_packed(cache.V, T, 1)       # the quantizer's own rounding: the reference's output tensor
    chunks = 8 * T * d // 4
    return {"what": "BASELINE config 1 on the GPU: one bulk append = quantize (s24_r3) + Med3x (C = 3) + bit-packing + sideband of K and V, "
                    "8 heads x 2048 tokens x d_h 128 fp16; MSE of the cache dequantized again (packed codes + verbatim outlier chunks) "
                    "against the input",
            "us_per_call_K_and_V": round(us, 1), "GTok_per_s": round(T / us / 1e3, 6),
            "mse_K": float(((Kd.float() - k.float()) ** 2).mean()), "mse_V": float(((Vd.float() - v.float()) ** 2).mean()),
            "outlier_rate_K": round(float(cache.K.sb_count.sum()) / chunks, 5), "outlier_rate_V": round(float(cache.V.sb_count.sum()) / chunks, 5),
            "bits_per_value": round(w.bits_per_value(), 4), "packed_bytes_K_and_V": cache.nbytes(T)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=192)
    ap.add_argument("--warmup", type=int, default=-1, help="untimed warm-up steps (default 32 + 10 x steps)")
    ap.add_argument("--context", type=int, default=32768)
    ap.add_argument("--layers", type=int, default=16, help="distinct caches the timed steps rotate over")
    ap.add_argument("--n-splits", type=int, default=0)
    ap.add_argument("--no-graph", action="store_true", help="launch every step from Python instead of one HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--quick", action="store_true", help="only the headline step, its kernel and the CPU baseline")
    ap.add_argument("--counters", action="store_true",
                    help="for rocprofv3 --pmc runs: only 32 eager attention steps (rotating caches) and 5 plain 256 MiB "
                         "copies (the calibration kernel for FETCH_SIZE / WRITE_SIZE), no JSON line")
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
    T, NL = args.context, max(1, args.layers)
    q = hqmq.HQMQ(n_layers=max(NL, 64), n_heads=Hkv, secondary_size=S, radius_bits=B_R, device=dev)
    caches, queries = build_layers(q, T, dt, dev, NL)
    outs = [torch.empty_like(queries[0]) for _ in range(NL)]
    n_splits = args.n_splits or ops.pick_splits(1, Hq, Hkv, 1, T)
    cache_bytes = caches[0].nbytes(T)
    step_bytes = cache_bytes + 2 * queries[0].numel() * queries[0].element_size()      # + Q read and O written

    def step(i):
        j = i % NL
        hqmq.fused_attention_packed(queries[j], caches[j], n_splits=n_splits, out=outs[j])

    def step_same(i):
        hqmq.fused_attention_packed(queries[0], caches[0], n_splits=n_splits, out=outs[0])

    # correctness of what is being timed: dense SDPA over the dequantized cache
    step(0)
    Kd, Vd = ops.dequant_packed(caches[0].K, T, 0), ops.dequant_packed(caches[0].V, T, 0)
    ref = torch.nn.functional.scaled_dot_product_attention(queries[0], Kd.repeat_interleave(Hq // Hkv, 1),
                                                           Vd.repeat_interleave(Hq // Hkv, 1))
    max_err = (outs[0].float() - ref.float()).abs().max().item()
    del Kd, Vd
    if not max_err < 2e-3:
        print(f"attention output differs from dense SDPA by {max_err}", file=sys.stderr)
        sys.exit(1)

    stream = torch.cuda.current_stream()
    if args.warmup < 0:
        args.warmup = 32 + 10 * args.steps
    eager_warmup = args.warmup if args.no_graph else min(args.warmup, 32)
    warm_replays = max(1, (args.warmup - eager_warmup) // max(1, args.steps))
    for i in range(eager_warmup):
        step(i)
    torch.cuda.synchronize()
    if args.counters:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for i in range(32):
            step(i)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(f"counters mode: 32 attention steps of {cache_bytes} compressed bytes, 5 copies of {src.numel()} bytes")
        return

    if args.no_graph:
        def eager():
            for i in range(args.steps):
                step(i)
        us_step, used_graph = host_time_s(eager) / args.steps * 1e6, False
        warm_replays = 0
    else:
        us_step, used_graph = graph_us(step, args.steps, stream, warm_replays=warm_replays)
    value = step_bytes / (us_step * 1e-6) / 1e9

    # the attention kernel alone (split partials left in the workspace), a pair of HIP events per launch
    partials = torch.empty(max(16, int(ops.L.lib().hqmq_attn_workspace_bytes(1, Hq, 1, D_H, n_splits))), dtype=torch.uint8, device=dev)

    def main_kernel(i, ev, rotate=True):
        j = i % NL if rotate else 0
        ops.attn_fwd(queries[j], caches[j].K, caches[j].V, T, n_splits=n_splits, out=outs[j], skip_combine=True, kernel_events=ev,
                     workspace=partials)
    us_main = kernel_time_us(main_kernel, 192)
    main_stats = {k: round(v, 2) for k, v in LAST_KERNEL_STATS.items()}
    us_main_same = kernel_time_us(lambda i, ev: main_kernel(i, ev, False), 192)
    us_launch_interval, _ = graph_us(lambda i: main_kernel(i, None), args.steps, stream)
    us_step_same, _ = graph_us(step_same, args.steps, stream)
    us_step_settled, _ = graph_us(step, args.steps, stream, replays=9)
    achieved = cache_bytes / (us_main * 1e-6) / 1e9
    # what the memory system allows a launch of this shape: the kernel that only reads the same planes with the same
    # grid, per-wavefront ranges and loads (libhqmq_bench.so: hqmq_bench_read_planes), caches rotating / one cache
    from hqmq_amd import bench_ceiling
    sink = torch.empty(1 << 22, dtype=torch.uint8, device=dev)
    us_read = kernel_time_us(lambda i, ev: bench_ceiling.read_planes(caches[i % NL], n_splits, 3, 8, ev, sink), 192)
    us_read_same = kernel_time_us(lambda i, ev: bench_ceiling.read_planes(caches[0], n_splits, 3, 8, ev, sink), 192)

    result = {
        "metric": "decode-attn HBM GB/s on compressed bytes (us/step and % of 8 TB/s alongside); quantize GTok/s",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "warmup_steps_run": eager_warmup + warm_replays * args.steps,
        "ms_per_step": round(us_step / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"BASELINE config 2: fused decode attention, Llama-3-8B shape (32 q / 8 kv heads, d_h 128, "
                               f"batch 1), s96_r4 fp16 cache, context {T}, one query token, one layer per step, the steps "
                               f"rotating over {NL} layers' caches ({NL * cache_bytes / 1e6:.0f} MB: read from HBM every step)",
                   "context": T, "n_splits": n_splits, "hip_graph": used_graph, "layers": NL,
                   "compressed_bytes_per_step": cache_bytes},
        "us_per_step": round(us_step, 2),
        "us_per_step_median_of_9_replays": round(us_step_settled, 2),
        "pct_of_hbm_roofline": round(100 * value / HBM_PEAK_GBPS, 2),
        "max_abs_err_vs_dense_sdpa": max_err,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": RECORDED_TRAFFIC_BYTES.get(T),
                     "traffic_source": f"{TRAFFIC_FILE} (FETCH_SIZE + WRITE_SIZE of an earlier rocprofv3 --pmc run; not "
                                       f"measured by this run)" if T in RECORDED_TRAFFIC_BYTES else None,
                     "kernel": "hqmq::attn_lds_kernel<1, 12, 8>", "kernel_us": round(us_main, 2), "kernel_us_is": "median of 192 launches, each with its own pair of HIP events", "kernel_us_stats": main_stats,
                     "kernel_launch_interval_us": round(us_launch_interval, 2),
                     "algorithmic_bytes_per_launch": cache_bytes,
                     "read_only_kernel_same_grid_us": round(us_read, 2),
                     "read_only_kernel_GBps": round(cache_bytes / us_read / 1e3, 1),
                     "frac_of_read_only_kernel": round(us_read / us_main, 4)},
        "same_cache_replay": {
            "what": "the same step over ONE cache replayed back to back: its 34.6 MB stay in the L2s and the 256 MB "
                    "Infinity Cache, so this is not an HBM figure; reported as the cache-resident upper bound",
            "us_per_step": round(us_step_same, 2), "GBps": round(step_bytes / us_step_same / 1e3, 1),
            "kernel_us": round(us_main_same, 2), "kernel_GBps": round(cache_bytes / us_main_same / 1e3, 1),
            "read_only_kernel_same_grid_us": round(us_read_same, 2)},
    }
    if not args.quick:
        # quantize throughput: K and V of one layer, bulk (prefill) call, packed output
        k, v = kv_pair(T, dt, dev, 5)
        c2 = q.new_cache(1, T, D_H, dt, 0)

        def quant_only(i):
            c2.K.length = c2.V.length = 0
            q.append(c2, k, v, 0)
        us_quant = event_time_us(quant_only, 10, stream)
        # algorithmic bytes of the call: K and V, 8 heads: the input row (d_h x 2 B) read, the packed row (66 B) written
        q_bytes = 2 * Hkv * T * (D_H * 2 + cache_bytes // (2 * Hkv * T))
        valu_per_wave, waves = 1885, 2 * Hkv * T * (D_H // 4) // 64       # instructions per wavefront of 64 chunks: recorded by rocprofv3
        result["quantize"] = {"GTok_per_s": round(T / (us_quant * 1e-6) / 1e9, 5), "us_per_call": round(us_quant, 1), "tokens": T,
                              "what": "K and V of one layer, 8 kv heads x d_h 128, s96_r4 fp16, quantize + pack (no Med3x); "
                                      "the config-1 workload (s24_r3 + Med3x) is in the config1 block, GPU and CPU on the same input",
                              "algorithmic_bytes_per_call": q_bytes, "GBps": round(q_bytes / us_quant / 1e3, 1),
                              "bytes_roofline_frac": round(q_bytes / us_quant / 1e3 / HBM_PEAK_GBPS, 4),
                              "valu_issue_frac": round(valu_per_wave * 4 * waves / (1024 * 2.4e3 * us_quant), 3),
                              "valu_issue_frac_is": "1,885 vector-ALU instructions per wavefront (profiles/quantize_kernel_s96r4_fp16_32k.txt, "
                                                    "recorded offline) x 4 cycles x wavefronts / (1024 SIMDs x 2.4 GHz x the measured time): "
                                                    "the kernel is bound by vector-ALU issue, not by bytes"}
        k1, v1 = k[:, :, :1].contiguous(), v[:, :, :1].contiguous()

        def append_one(i):
            c2.K.length = c2.V.length = 0
            q.append(c2, k1, v1, 0)
        result["quantize"]["append_one_token_us"] = round(event_time_us(append_one, 50, stream), 2)
        del k, v, c2
        # the other contexts of config 2, rotating over enough layers to exceed the Infinity Cache
        other = {}
        for Tc in (4096, 8192, 16384):
            nl = min(64, max(NL, -(-600_000_000 // (cache_bytes * Tc // T))))
            cs, qs = build_layers(q, Tc, dt, dev, nl)
            ns = ops.pick_splits(1, Hq, Hkv, 1, Tc)
            us, _ = graph_us(lambda i: hqmq.fused_attention_packed(qs[i % nl], cs[i % nl], n_splits=ns, out=outs[0]), args.steps, stream, replays=5)
            us1, _ = graph_us(lambda i: hqmq.fused_attention_packed(qs[0], cs[0], n_splits=ns, out=outs[0]), args.steps, stream, replays=5)
            other[str(Tc)] = {"us_per_step": round(us, 2), "GBps": round(cs[0].nbytes(Tc) / us / 1e3, 1), "n_splits": ns,
                              "layers": nl, "same_cache_us_per_step": round(us1, 2)}
            del cs, qs
        result["other_contexts"] = other
        # steady state: batch 8 of the same shape (277 MB per step, 8192 tokens per block), two caches alternating
        cs, qs = build_layers(q, T, dt, dev, 2, B=8)
        o8 = torch.empty_like(qs[0])
        ns8 = ops.pick_splits(8, Hq, Hkv, 1, T)
        us8, _ = graph_us(lambda i: hqmq.fused_attention_packed(qs[i % 2], cs[i % 2], n_splits=ns8, out=o8), 48, stream, replays=7)
        result["batch8_steady_state"] = {"us_per_step": round(us8, 2), "GBps": round(cs[0].nbytes(T) / us8 / 1e3, 1),
                                         "pct_of_hbm_roofline": round(100 * cs[0].nbytes(T) / us8 / 1e3 / HBM_PEAK_GBPS, 2),
                                         "n_splits": ns8, "what": "config 2 shape at batch 8, two caches alternating; median of 7 replays of 48 steps"}
        del cs, qs
        # the one prefill shape the reference publishes (paper App. F: 1.568 ms on an RTX 4090): B = 1, 32 / 8 heads,
        # T = 2048 square causal, d_h 128, s192 with r_qmax = 15, fp16
        qp = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=192, radius_bits=4, device=dev)
        kp, vp = kv_pair(2048, dt, dev, 9)
        cp = qp.new_cache(1, 2048, D_H, dt, 0)
        qp.append(cp, kp, vp, 0)
        Qp = torch.randn(1, Hq, 2048, D_H, generator=torch.Generator().manual_seed(10)).to(dt).to(dev)
        Op = torch.empty_like(Qp)
        usp = event_time_us(lambda i: hqmq.fused_attention_packed(Qp, cp, causal=True, out=Op), 20, stream)
        Kd, Vd = ops.dequant_packed(cp.K, 2048, 0), ops.dequant_packed(cp.V, 2048, 0)
        refp = torch.nn.functional.scaled_dot_product_attention(Qp, Kd.repeat_interleave(4, 1), Vd.repeat_interleave(4, 1), is_causal=True)
        result["prefill_T2048_s192_fp16"] = {"ms": round(usp / 1e3, 4), "max_abs_err_vs_dense_sdpa": (Op.float() - refp.float()).abs().max().item(),
                                             "reference_published_ms_rtx4090": 1.568,
                                             "what": "B 1, 32/8 heads, T_q = T_kv = 2048 causal, d_h 128, s192 r_qmax 15, fp16"}
        del kp, vp, cp, Qp, Op, Kd, Vd, refp
        torch.cuda.empty_cache()
        # configs 3-5 at full size (one layer each): decode step, error against dense fp32 attention, bulk quantize
        from hqmq_amd import bench_configs
        result["configs_3_4_5"] = {}
        for cfg in (3, 4, 5):
            r = bench_configs.run(cfg, 30, emit=False)
            torch.cuda.empty_cache()
            # the same shape and inputs without Med3x: what the outlier handling costs on this shape
            plain = bench_configs.run(cfg, 30, emit=False, med3x=False)
            r["us_per_step_without_med3x"] = plain["us_per_step"]
            r["med3x_over_plain"] = round(r["us_per_step"] / plain["us_per_step"], 3)
            result["configs_3_4_5"][str(cfg)] = r
            del plain
            torch.cuda.empty_cache()
    if not args.quick:
        result["config1"] = gpu_config1(dev)
    if not args.no_cpu_baseline:
        threads = torch.get_num_threads()
        slice_tokens = 4096
        sec = cpu_attention_baseline(slice_tokens)
        slice_bytes = cache_bytes * slice_tokens / T
        qsec, qtok, qmse = cpu_quantize_baseline_config1()
        if "config1" in result:
            result["config1"]["mse_equal_to_cpu"] = bool(result["config1"]["mse_K"] == qmse[0] and result["config1"]["mse_V"] == qmse[1])
            result["config1"].update(cpu_us_per_call_K_and_V=round(qsec * 1e6, 1), cpu_GTok_per_s=round(qtok / qsec / 1e9, 8),
                                     cpu_mse_K=qmse[0], cpu_mse_V=qmse[1], cpu_cores=threads,
                                     cpu_what="the restated reference quantizer (oracle, torch on the host) on the same tensors")
        result["cpu_baseline"] = {
            "value": round(slice_bytes / sec / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"torch restatement of the reference path (dense decode + SDPA), fp16, {slice_tokens} of {T} tokens, "
                      f"median of 5 after 2 warm-ups; os.cpu_count()={os.cpu_count()}",
            "us_per_step_scaled_to_full_context": round(sec * T / slice_tokens * 1e6, 1),
            "quantize_GTok_per_s": round(qtok / qsec / 1e9, 8),
            "quantize_sample": "benchmark config 1 in full: K and V of one layer, 8 heads x 2048 tokens x d_h 128 fp16, s24_r3 + "
                               "Med3x (C = 3), restated reference quantizer, median of 3 after 1 warm-up",
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
