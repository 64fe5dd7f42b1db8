#!/usr/bin/env python3
"""Full-size runs of benchmark configs 3, 4 and 5 on one GPU (config 2 is bench.py's default workload).

    python -m hqmq_amd.bench_configs [--configs 3 4 5] [--steps 50] [--plain]

--plain builds the same caches without Med3x (no flags, no sideband): what the outlier handling costs on each shape.

For each config: build the packed cache with the HIP quantize path (bulk, Med3x where the config has it), run
one layer's fused decode-attention step over it, check the output against dense fp32 attention on the
dequantized cache (computed on the GPU in slices), and print one JSON line with us/step, GB/s on the
algorithmic compressed bytes, the fraction of 8 TB/s and the quantize throughput.
  3: Qwen2.5-7B shape, 28 q / 4 kv heads, d_h 128, batch 8, context 32768, s192_r6 + Med3x, fp16,
     2 % of K chunks scaled x50-200
  4: Qwen3-8B shape, 32 / 8, d_h 128, batch 64, per-sequence contexts U{1024..16384}, s24_r3 + Med3x, bf16,
     lognormal channel scales; a step = quantize-and-append one token per sequence, then attend
  5: gpt-oss-20b shape, 64 / 8, d_h 64, batch 4, context 131072, s96_r4 + Med3x, bf16, 1 % of chunks x100
"""
import argparse
import json
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

import hqmq  # noqa: E402
from hqmq_amd import ops  # noqa: E402

HBM_PEAK_GBPS = 8000.0
DEV = "cuda:0"


def event_us(fn, iters):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def synth(shape, dt, seed, lognormal=False, outlier_p=0.0, gain=(50.0, 200.0)):
    """Synthetic K or V (B, H, T, d): N(0, 1), optional per-channel lognormal(0, 0.5) scale, optional outlier chunks
    (a Bernoulli(outlier_p) choice of whole chunks scaled by U(gain)).  Seeded with a CPU generator, drawn one
    sequence at a time on the host and then moved, so that a CPU restatement can see the same inputs."""
    g = torch.Generator().manual_seed(seed)
    B, H, T, d = shape
    out = torch.empty(B, H, T, d, dtype=dt, device=DEV)
    chan = torch.exp(0.5 * torch.randn(H, 1, d, generator=g)) if lognormal else None
    n = d // 4
    for b in range(B):
        x = torch.randn(H, T, d, generator=g)
        if chan is not None:
            x *= chan
        if outlier_p > 0:
            hit = torch.rand(H, T, n, 1, generator=g) < outlier_p
            f = gain[0] + (gain[1] - gain[0]) * torch.rand(H, T, n, 1, generator=g)
            x = torch.where(hit, x.view(H, T, n, 4) * f, x.view(H, T, n, 4)).reshape(H, T, d)
        out[b] = x.to(dt).to(DEV, non_blocking=True)
    return out


def dense_check(Q, cache, lens, T):
    """max |O - dense fp32 attention over the dequantized cache|, one sequence at a time."""
    B, Hq, _, d = Q.shape
    Hkv = cache.K.H
    g = Hq // Hkv
    O = hqmq.fused_attention_packed(Q, cache, kv_lens=lens, T_kv=T)
    worst, ref_max = 0.0, 0.0
    Kd_all, Vd_all = ops.dequant_packed(cache.K, T, 0), ops.dequant_packed(cache.V, T, 0)
    for b in range(B):
        L = int(lens[b]) if lens is not None else T
        Kd, Vd = Kd_all[b, :, :L].float(), Vd_all[b, :, :L].float()
        s = torch.einsum("hgd,hkd->hgk", Q[b, :, 0].float().view(Hkv, g, d), Kd) * d ** -0.5
        ref = torch.einsum("hgk,hkd->hgd", torch.softmax(s, dim=-1), Vd).reshape(Hq, d)
        worst = max(worst, float((O[b, :, 0].float() - ref).abs().max()))
        ref_max = max(ref_max, float(ref.abs().max()))
    return worst, ref_max


def setup(cfg, med3x=True):
    """Inputs, quantizer and filled cache of one config: a dict with B, Hq, Hkv, d, dt, T, lens (CPU int32 or None), lens_dev,
    k, v, w (the quantizer), cache, name, med (Med3x on), quant_ms (the bulk append)."""
    if cfg == 3:
        B, Hq, Hkv, d, S, b_r, dt, med = 8, 28, 4, 128, 192, 6, torch.float16, True
        lens, T = None, 32768
        k = synth((B, Hkv, T, d), dt, 31, outlier_p=0.02)
        v = synth((B, Hkv, T, d), dt, 32)
        name = "config 3: Qwen2.5-7B shape, 28/4 heads, d_h 128, batch 8, context 32768, s192_r6 + Med3x, fp16"
    elif cfg == 4:
        B, Hq, Hkv, d, S, b_r, dt, med = 64, 32, 8, 128, 24, 3, torch.bfloat16, True
        lens = torch.randint(1024, 16385, (B,), generator=torch.Generator().manual_seed(4)).to(torch.int32)
        T = 16384 + 1024          # room for the tokens the timed decode steps append
        k = synth((B, Hkv, T, d), dt, 41, lognormal=True)
        v = synth((B, Hkv, T, d), dt, 42, lognormal=True)
        name = "config 4: Qwen3-8B shape, 32/8 heads, d_h 128, batch 64, contexts U{1024..16384}, s24_r3 + Med3x, bf16"
    elif cfg == 5:
        B, Hq, Hkv, d, S, b_r, dt, med = 4, 64, 8, 64, 96, 4, torch.bfloat16, True
        lens, T = None, 131072
        k = synth((B, Hkv, T, d), dt, 51, outlier_p=0.01, gain=(100.0, 100.0))
        v = synth((B, Hkv, T, d), dt, 52, outlier_p=0.01, gain=(100.0, 100.0))
        name = "config 5: gpt-oss-20b shape, 64/8 heads, d_h 64, batch 4, context 131072, s96_r4 + Med3x, bf16"
    else:
        raise SystemExit(f"unknown config {cfg}")
    q = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV)
    med = med and med3x
    if not med:
        name = name.replace(" + Med3x", " (Med3x off)")
    w = hqmq.with_outlier_extraction(q, C=3.0) if med else q
    cache = w.new_cache(B, T, d, dt, 0, sideband_frac=0.125)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    w.append(cache, k, v, 0)                     # bulk (prefill) quantize of the whole cache, K and V
    e1.record()
    torch.cuda.synchronize()
    quant_ms = e0.elapsed_time(e1)
    if med:
        cache.K.check_overflow()
        cache.V.check_overflow()
    lens_dev = lens.to(DEV) if lens is not None else None
    if lens is not None:
        cache.crop_(lens_dev)                    # every sequence keeps its own context; the rows behind it are free
    return dict(B=B, Hq=Hq, Hkv=Hkv, d=d, dt=dt, T=T, lens=lens, lens_dev=lens_dev, k=k, v=v, w=w, cache=cache, name=name, med=med,
                quant_ms=quant_ms, cfg=cfg)


def run(cfg, steps, emit=True, med3x=True):
    c = setup(cfg, med3x)
    B, Hq, Hkv, d, dt, T, lens, lens_dev = c["B"], c["Hq"], c["Hkv"], c["d"], c["dt"], c["T"], c["lens"], c["lens_dev"]
    k, v, w, cache, name, med, quant_ms = c["k"], c["v"], c["w"], c["cache"], c["name"], c["med"], c["quant_ms"]
    Q = torch.randn(B, Hq, 1, d, generator=torch.Generator().manual_seed(7)).to(dt).to(DEV)
    out = torch.empty_like(Q)
    err, ref_max = dense_check(Q, cache, lens, T)
    # algorithmic bytes of one step: the valid rows of every plane + 8 B per flagged chunk in them
    tokens = int(lens.sum()) if lens is not None else B * T
    row = cache.K.row_bytes()
    if not med:
        flagged = 0
    elif lens is None:
        flagged = int(cache.K.sb_count.sum()) + int(cache.V.sb_count.sum())
    else:
        flagged = 0
        for pt in (cache.K, cache.V):               # popcount of the flag bits of the valid rows
            bits = torch.stack([(pt.flags >> i) & 1 for i in range(8)], -1).sum(-1).sum(-1).to(torch.int64)   # (B, H, t_cap)
            valid = torch.arange(pt.t_cap, device=DEV).view(1, 1, -1) < lens_dev.view(B, 1, 1)
            flagged += int((bits * valid).sum())
    step_bytes = 2 * Hkv * tokens * row + flagged * 4 * cache.K.scale.element_size()
    n_splits = ops.pick_splits(B, Hq, Hkv, 1, T if lens is None else int(lens.max()), lens is not None)

    # ragged batch: the longest sequences start first (the order holds while all contexts grow in step)
    order = ops.longest_first(lens_dev) if lens is not None else None

    # a working set below the 256 MB Infinity Cache (config 3: 182 MB) would be served from it on every replay: such a
    # config alternates between two caches, so that every step reads its cache from HBM as a decode step over many
    # layers does
    rot = [cache]
    if step_bytes < 300e6 and lens is None:
        k2 = synth(k.shape, dt, 1000 + cfg, outlier_p=0.02 if cfg == 3 else 0.01, gain=(50.0, 200.0) if cfg == 3 else (100.0, 100.0))
        other = w.new_cache(B, T, d, dt, 0, sideband_frac=0.125)
        w.append(other, k2, v, 0)
        rot.append(other)
        del k2
    turn = [0]

    def attend():
        turn[0] += 1
        hqmq.fused_attention_packed(Q, rot[turn[0] % len(rot)], kv_lens=lens_dev, T_kv=T, n_splits=n_splits, out=out, batch_order=order)
    # the median of three measurements: the first one after the setup above runs before the clocks have settled (config 4:
    # 288 us against 248 - 265 us for every later one)
    us = sorted(event_us(attend, steps) for _ in range(3))[1]
    res = {"config": name, "us_per_step": round(us, 2), "compressed_bytes_per_step": step_bytes,
           "GBps": round(step_bytes / us / 1e3, 1), "pct_of_hbm_roofline": round(100 * step_bytes / us / 1e3 / HBM_PEAK_GBPS, 2),
           "n_splits": n_splits, "max_abs_err_vs_dense_fp32": err, "max_abs_ref": ref_max,
           "outlier_rate_K": round(float(cache.K.sb_count.sum()) / (Hkv * tokens * d / 4), 5) if med else 0.0,      # over the rows kept
           "bulk_quantize_ms_K_and_V": round(quant_ms, 2), "bulk_quantize_GTok_per_s": round(B * T / quant_ms / 1e6, 5),
           "bits_per_value": round(w.bits_per_value(), 3)}
    if cfg == 4:      # the step of config 4 also quantizes and appends one token per sequence (every context grows by 1)
        pos = lens_dev.clone()
        k1, v1 = k[:, :, :1].contiguous(), v[:, :, :1].contiguous()
        assert 7 * (steps + 3) + 3 <= T - int(lens.max()), "more timed appends than spare rows"

        def append():
            w.append(cache, k1, v1, 0, pos=pos)
            pos.add_(1)

        def step():
            append()
            hqmq.fused_attention_packed(Q, cache, kv_lens=pos, T_kv=T, n_splits=n_splits, out=out, batch_order=order)
        res["us_per_step_with_append"] = round(sorted(event_us(step, steps) for _ in range(3))[1], 2)
        res["us_append_only"] = round(sorted(event_us(append, steps) for _ in range(3))[1], 2)
        # the same step replayed from a HIP graph: what the GPU needs once the ten small launches of an append are
        # not paced by the host (every kernel of the path is capturable: no allocation, no memset, no sync)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        res["us_per_step_with_append_graph"] = round(event_us(graph.replay, steps), 2)
        if med:
            cache.K.check_overflow()
            cache.V.check_overflow()
    res["caches_rotated"] = len(rot)
    if emit:
        print(json.dumps(res), flush=True)
    return res


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--configs", type=int, nargs="+", default=[3, 4, 5])
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--plain", action="store_true", help="the same shapes and inputs without Med3x")
    a = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("needs a GPU: the HQMQ kernels have no CPU path")
    for c in a.configs:
        run(c, a.steps, med3x=not a.plain)
        torch.cuda.empty_cache()
