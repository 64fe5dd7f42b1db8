"""Writes tests/golden/*.npz: inputs and outputs of the reference implementation.

Run once, in the build container only (the reference checkout does not exist on
the GPU box):  python tests/golden/make_golden.py [/root/reference]

The reference returns only dense tensors, so each fixture holds seeded inputs
and the dense result of the reference call; 16-bit tensors are stored as their
raw bit patterns (int16) so that comparisons are bit-exact and NaN-safe.
Functions covered: HQMQQuantizer._get_codebook / quantize_K / quantize_V,
OutlierAwareHQMQQuantizer.quantize_K / quantize_V (median_mult mode),
_decode_kv_torch, fused_hqmq_attention_torch.
"""
import sys
from pathlib import Path

import numpy as np
import torch

REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
OUT = Path(__file__).resolve().parent
sys.path.insert(0, str(REF))

from src.quantizers.hqmq import HQMQQuantizer  # noqa: E402
from src.quantizers.outlier_aware import OutlierAwareHQMQQuantizer  # noqa: E402
from src.quantizers.hqmq_attention import _decode_kv_torch, fused_hqmq_attention_torch  # noqa: E402

DT = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


def bits(t: torch.Tensor) -> np.ndarray:
    t = t.detach().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().copy()
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy().copy()
    return t.numpy().copy()


def make_input(gen, shape, dtype, lognormal=True):
    x = torch.randn(*shape, generator=gen)
    if lognormal:
        x = x * torch.exp(0.5 * torch.randn(shape[0], shape[1], 1, shape[3], generator=gen))
    return x.to(dtype)


def quantizer_cases():
    out = {}
    cfgs = [  # name, S, b_r, shape(B,H,T,d_h), seed
        ("s24r3", 24, 3, (2, 2, 12, 32), 42),
        ("s96r4", 96, 4, (1, 2, 10, 128), 42),
        ("s192r6", 192, 6, (1, 2, 6, 64), 7),
    ]
    for name, S, b_r, shape, seed in cfgs:
        B, H, T, d_h = shape
        with torch.no_grad():
            q = HQMQQuantizer(n_layers=2, n_heads=H, secondary_size=S, radius_bits=b_r,
                              device="cpu", seed=seed)
            for dn, dt in DT.items():
                gen = torch.Generator().manual_seed(1000 + seed + S)
                for kv, tag in ((0, "K"), (1, "V")):
                    x = make_input(gen, shape, dt)
                    # one all-zero chunk, one all-zero token, one token with a huge chunk
                    x[0, 0, 1, 4:8] = 0
                    x[0, 1, 2, :] = 0
                    x[0, 0, 3, 8:12] *= 64
                    layer = 1
                    y = q.quantize_K(x, layer) if kv == 0 else q.quantize_V(x, layer)
                    j = q._get_codebook(layer, kv, x)
                    key = f"{name}_{dn}_{tag}"
                    out[key + "_x"] = bits(x)
                    out[key + "_out"] = bits(y)
                    out[key + "_joint"] = bits(j)
            out[name + "_raw"] = q.secondary_raw.detach().numpy().copy()
            out[name + "_meta"] = np.array([S, b_r, seed, 2, H], dtype=np.int64)
    np.savez_compressed(OUT / "quantizer.npz", **out)
    return len(out)


def outlier_cases():
    out = {}
    cfgs = [("s24r3", 24, 3, (2, 2, 16, 32), 42), ("s96r4", 96, 4, (1, 2, 9, 64), 11)]
    for name, S, b_r, shape, seed in cfgs:
        B, H, T, d_h = shape
        n = d_h // 4
        with torch.no_grad():
            inner = HQMQQuantizer(n_layers=1, n_heads=H, secondary_size=S, radius_bits=b_r,
                                  device="cpu", seed=seed)
            for dn, dt in DT.items():
                w = OutlierAwareHQMQQuantizer(inner, threshold_mode="median_mult", median_mult=3.0)
                gen = torch.Generator().manual_seed(2000 + seed)
                for kv, tag in ((0, "K"), (1, "V")):
                    x = torch.randn(*shape, generator=gen)
                    hit = torch.rand(B, H, T, n, generator=gen) < 0.06
                    gain = 50 + 150 * torch.rand(B, H, T, n, generator=gen)
                    xc = x.view(B, H, T, n, 4)
                    xc = torch.where(hit.unsqueeze(-1), xc * gain.unsqueeze(-1), xc)
                    x = xc.reshape(shape).to(dt)
                    y = w.quantize_K(x, 0) if kv == 0 else w.quantize_V(x, 0)
                    key = f"{name}_{dn}_{tag}"
                    out[key + "_x"] = bits(x)
                    out[key + "_out"] = bits(y)
                out[f"{name}_{dn}_rate"] = np.array([w._observed_outlier_rate, w._n_observations, w.bits_per_value()])
            out[name + "_raw"] = inner.secondary_raw.detach().numpy().copy()
            out[name + "_meta"] = np.array([S, b_r, seed, 1, H], dtype=np.int64)
    np.savez_compressed(OUT / "outlier.npz", **out)
    return len(out)


def attention_cases():
    out = {}
    cfgs = [  # name, B, H_q, H_kv, T_q, T_kv, d_h, S, qmax, causal, dtype
        ("sq_fp32", 1, 4, 1, 24, 24, 32, 24, 7, True, "fp32"),
        ("gqa_dec_fp16", 2, 8, 2, 1, 40, 64, 96, 15, False, "fp16"),
        ("gqa_dec_bf16", 2, 6, 2, 1, 33, 64, 24, 7, False, "bf16"),
        ("rect_causal_fp16", 1, 4, 2, 5, 19, 32, 24, 7, True, "fp16"),
        ("rect_full_fp32", 1, 2, 2, 3, 17, 16, 24, 63, False, "fp32"),
    ]
    for i, (name, B, Hq, Hkv, Tq, Tkv, d_h, S, qmax, causal, dn) in enumerate(cfgs):
        dt = DT[dn]
        gen = torch.Generator().manual_seed(3000 + i)
        K = 24 * S
        n = d_h // 4
        Q = (torch.randn(B, Hq, Tq, d_h, generator=gen) * 0.7).to(dt)
        d = {}
        for tag in ("K", "V"):
            d[tag + "_idx"] = torch.randint(0, K, (B, Hkv, Tkv, n), generator=gen, dtype=torch.int32)
            d[tag + "_rq"] = torch.randint(0, qmax + 1, (B, Hkv, Tkv, n), generator=gen, dtype=torch.int32)
            d[tag + "_rs"] = (torch.rand(B, Hkv, Tkv, generator=gen) + 0.5).to(dt)
            j = torch.randn(Hkv, K, 4, generator=gen)
            d[tag + "_joint"] = (j / j.norm(dim=-1, keepdim=True).clamp(min=1e-6)).to(dt)
        with torch.no_grad():
            O = fused_hqmq_attention_torch(Q, d["K_idx"], d["K_rq"], d["K_rs"], d["K_joint"],
                                           d["V_idx"], d["V_rq"], d["V_rs"], d["V_joint"],
                                           r_qmax=qmax, causal=causal)
            Kd = _decode_kv_torch(d["K_idx"], d["K_rq"], d["K_rs"], d["K_joint"], qmax)
        out[name + "_Q"] = bits(Q)
        for k, v in d.items():
            out[f"{name}_{k}"] = bits(v)
        out[name + "_O"] = bits(O)
        out[name + "_Kdense"] = bits(Kd)
        out[name + "_meta"] = np.array([B, Hq, Hkv, Tq, Tkv, d_h, S, qmax, int(causal)], dtype=np.int64)
        out[name + "_dtype"] = np.array(dn)
    np.savez_compressed(OUT / "attention.npz", **out)
    return len(out)


if __name__ == "__main__":
    torch.manual_seed(0)
    print("quantizer arrays:", quantizer_cases())
    print("outlier arrays:", outlier_cases())
    print("attention arrays:", attention_cases())
    print("torch", torch.__version__, "threads", torch.get_num_threads())
