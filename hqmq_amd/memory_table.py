#!/usr/bin/env python3
"""KV-cache memory table with the bytes the packed cache really stores.

    python -m hqmq_amd.memory_table [--batch 1] [--med3x 0.015] [--json]

Same models, sequence lengths and codebook configs as the reference's analytic table
(experiments/18_memory.py of the reference, which counts log2(24 S) fractional bits per chunk); here every figure
comes from the packed layout itself: whole bits per code (main + aux planes), the per-token scale, and with
--med3x P the flag plane (1 bit per chunk) plus 8 bytes (4 elements of fp16) for a fraction P of the chunks.
Runs on the CPU: it only asks the library for the layout's bit widths.
"""
import argparse
import json
import math

from . import _lib as L

MODELS = {
    "Pythia-1B": {"n_layers": 16, "n_kv_heads": 8, "d_head": 256},
    "Pythia-2.8B": {"n_layers": 32, "n_kv_heads": 16, "d_head": 160},
    "Mistral-7B": {"n_layers": 32, "n_kv_heads": 8, "d_head": 128},
    "Qwen2.5-7B": {"n_layers": 28, "n_kv_heads": 4, "d_head": 128},
    "Llama-3-8B": {"n_layers": 32, "n_kv_heads": 8, "d_head": 128},
    "Llama-3-70B": {"n_layers": 80, "n_kv_heads": 8, "d_head": 128},
}
CONFIGS = [(24, 3), (24, 4), (48, 4), (96, 4), (192, 4), (192, 6)]
SEQ_LENS = [2048, 4096, 8192, 32768, 131072]


def fp16_kv_bytes(n_layers, n_kv_heads, d_head, seq_len, batch=1):
    return 2 * batch * n_layers * n_kv_heads * seq_len * d_head * 2


def analytic_kv_bytes(n_layers, n_kv_heads, d_head, seq_len, secondary_size, radius_bits, batch=1):
    """The reference's formula: (log2(24 S) + b_r) / 4 + 16 / d_head bits per element."""
    bits = (math.log2(24 * secondary_size) + radius_bits) / 4 + 16 / d_head
    return 2 * batch * n_layers * n_kv_heads * seq_len * d_head * bits / 8


def row_bytes(d_head, secondary_size, radius_bits, med3x=None, scale_bytes=2):
    """Bytes one (token, KV head, K or V) occupies in the packed planes; med3x = flagged fraction or None."""
    n = d_head // 4
    _, main_bits, aux_bits = L.layout_bits(secondary_size, radius_bits)
    b = (n * main_bits + 7) // 8 + (n * aux_bits + 7) // 8 + scale_bytes
    if med3x is not None:
        b += (n + 7) // 8 + med3x * n * 4 * scale_bytes
    return b


def packed_kv_bytes(n_layers, n_kv_heads, d_head, seq_len, secondary_size, radius_bits, batch=1, med3x=None):
    return 2 * batch * n_layers * n_kv_heads * seq_len * row_bytes(d_head, secondary_size, radius_bits, med3x)


def table(batch=1, med3x=None):
    rows = []
    for name, arch in MODELS.items():
        for T in SEQ_LENS:
            fp16 = fp16_kv_bytes(seq_len=T, batch=batch, **arch)
            r = {"model": name, "seq_len": T, "fp16_MB": fp16 / 1e6}
            for S, b_r in CONFIGS:
                key = f"hqmq_s{S}_r{b_r}"
                packed = packed_kv_bytes(seq_len=T, batch=batch, secondary_size=S, radius_bits=b_r, med3x=med3x, **arch)
                r[key + "_MB"] = packed / 1e6
                r[key + "_ratio"] = fp16 / packed
                r[key + "_analytic_MB"] = analytic_kv_bytes(seq_len=T, batch=batch, secondary_size=S, radius_bits=b_r, **arch) / 1e6
            rows.append(r)
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--med3x", type=float, default=None, help="fraction of chunks kept verbatim (adds the flag plane too)")
    ap.add_argument("--json", action="store_true")
    a = ap.parse_args()
    rows = table(a.batch, a.med3x)
    if a.json:
        print(json.dumps(rows))
        return
    keys = [f"hqmq_s{S}_r{b}" for S, b in CONFIGS]
    print(f"{'model':<12s} {'seq_len':>8s} {'fp16 MB':>10s} " + " ".join(f"{k[5:]:>16s}" for k in keys))
    for r in rows:
        print(f"{r['model']:<12s} {r['seq_len']:>8d} {r['fp16_MB']:>10.1f} " +
              " ".join(f"{r[k + '_MB']:>9.1f} ({r[k + '_ratio']:.2f}x)" for k in keys))
    print("\npacked bytes per (token, head, tensor) at d_head 128: " +
          ", ".join(f"s{S}_r{b}: {row_bytes(128, S, b, a.med3x):g}" for S, b in CONFIGS))


if __name__ == "__main__":
    main()
