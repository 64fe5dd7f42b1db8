"""CPU oracle (torch ops) for the HQMQ KV-cache path.  TEST INFRASTRUCTURE ONLY.

This module restates, op for op and in the same order, the torch arithmetic of
the reference so that the integer intermediates the reference never returns
(codeword index, radius code, per-token scale, Med3x mask) can be compared with
the HIP kernels.  Only tests, the smoke check and the CPU-baseline leg of the
benchmark may import it; the product package never does.

Reference lines followed (paths relative to the reference checkout):
  cell24            src/quantizers/spherical.py:22-43
  quat_mul          src/quantizers/hqmq.py:33-41
  secondary_raw     src/quantizers/hqmq.py:90-92,105
  joint_table       src/quantizers/hqmq.py:119-143
  quantize          src/quantizers/hqmq.py:145-158,164-169,208-216
  med3x             src/quantizers/outlier_aware.py:56-72
  outlier_quantize  src/quantizers/outlier_aware.py:79-87
  decode_kv         src/quantizers/hqmq_attention.py:39-65
  attention         src/quantizers/hqmq_attention.py:68-101

Pinning status.  cell24/quat_mul: the reference's own known-answer tests
(unit norms, 60 degree minimum angle, group closure).  joint_table, quantize,
med3x, outlier_quantize, decode_kv, attention: golden fixtures written once
from the reference itself (tests/golden/), plus brute-force/invariant checks
and an independent scalar C restatement (oracle/hqmq_oracle.c).

bf16 contractions are run with oneDNN disabled so that the einsum is the plain
fp32-accumulate kernel on every host (AMX/oneDNN results are host dependent).
"""
from __future__ import annotations

import contextlib
import itertools
import math
from typing import Optional

import torch
import torch.nn.functional as F


def cell24(dtype=torch.float32) -> torch.Tensor:
    """The 24 Hurwitz units: 8 signed axes, then 16 half-integer sign patterns."""
    rows = []
    for axis in range(4):
        for sign in (1.0, -1.0):
            rows.append([sign if j == axis else 0.0 for j in range(4)])
    for signs in itertools.product((1.0, -1.0), repeat=4):
        rows.append([0.5 * s for s in signs])
    return torch.tensor(rows, dtype=dtype)


def quat_mul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Hamilton product on (..., 4) tensors, (w, x, y, z), terms combined left to right."""
    aw, ax, ay, az = a.unbind(-1)
    bw, bx, by, bz = b.unbind(-1)
    return torch.stack([
        aw * bw - ax * bx - ay * by - az * bz,
        aw * bx + ax * bw + ay * bz - az * by,
        aw * by - ax * bz + ay * bw + az * bx,
        aw * bz + ax * by - ay * bx + az * bw,
    ], dim=-1)


def secondary_raw(n_layers: int, n_heads: int, secondary_size: int, seed: int = 42) -> torch.Tensor:
    """Seeded, unnormalised secondary codebooks, (L, H, 2, S, 4) fp32."""
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n_layers, n_heads, 2, secondary_size, 4, generator=g)


def joint_table(raw_hs4: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """(H, S, 4) fp32 raw secondaries -> (H, 24*S, 4) joint table in `dtype`, k = p*S + s."""
    H, S, _ = raw_hs4.shape
    sec = raw_hs4 / raw_hs4.norm(dim=-1, keepdim=True).clamp(min=1e-8)
    sec = sec.to(dtype)
    prim = cell24().to(dtype)
    p = prim.view(1, 24, 1, 4).expand(H, 24, S, 4)
    s = sec.view(H, 1, S, 4).expand(H, 24, S, 4)
    return quat_mul(p, s).reshape(H, 24 * S, 4)


@contextlib.contextmanager
def _plain_cpu_matmul():
    with torch.backends.mkldnn.flags(enabled=False):
        yield


def quantize(x: torch.Tensor, joint: torch.Tensor, radius_bits: int,
             t_block: Optional[int] = None) -> dict:
    """Unit-magnitude / linear-radius HQMQ quantize of x (B, H, T, d_h).

    Returns idx (int32), rq (int32, NaN code -> 0), rq_f (the rounded/clamped
    radius code as the reference holds it, dtype of x, may be NaN), r_max
    (dtype of x, (B,H,T)), out (fake-quant tensor, dtype of x).
    T is processed in blocks so that the similarity tensor stays bounded; every
    op is per token, so blocking does not change any value.
    """
    B, H, T, d_h = x.shape
    if d_h % 4 != 0:
        raise ValueError(f"d_head={d_h} not divisible by 4")
    n = d_h // 4
    K = joint.shape[1]
    qmax = (1 << radius_bits) - 1
    if t_block is None:
        t_block = max(1, (1 << 27) // max(1, B * H * n * K))
    idx_out = torch.empty(B, H, T, n, dtype=torch.int32)
    rq_out = torch.empty(B, H, T, n, dtype=torch.int32)
    rqf_out = torch.empty(B, H, T, n, dtype=x.dtype)
    rmax_out = torch.empty(B, H, T, dtype=x.dtype)
    out = torch.empty(B, H, T, d_h, dtype=x.dtype)
    joint_b = joint.view(1, H, 1, 1, K, 4)
    with _plain_cpu_matmul():
        for t0 in range(0, T, t_block):
            t1 = min(T, t0 + t_block)
            xc = x[:, :, t0:t1].reshape(B, H, t1 - t0, n, 4)
            radius = xc.norm(dim=-1, keepdim=True).clamp(min=1e-8)
            direction = xc / radius
            sims = torch.einsum("bhtnc,hkc->bhtnk", direction, joint)
            idx = sims.argmax(dim=-1)
            del sims
            gather_idx = idx.view(B, H, t1 - t0, n, 1, 1).expand(-1, -1, -1, -1, 1, 4)
            cw = joint_b.expand(B, H, t1 - t0, n, K, 4).gather(-2, gather_idx).squeeze(-2)
            r_max = radius.amax(dim=-2, keepdim=True).clamp(min=1e-8)
            scale = r_max / qmax
            rq_f = (radius / scale).round().clamp(0, qmax)
            radius_q = rq_f * scale
            o = radius_q * cw
            idx_out[:, :, t0:t1] = idx.to(torch.int32)
            rqf_out[:, :, t0:t1] = rq_f.squeeze(-1)
            rq_out[:, :, t0:t1] = torch.nan_to_num(rq_f.squeeze(-1).float(), nan=0.0).to(torch.int32)
            rmax_out[:, :, t0:t1] = r_max.view(B, H, t1 - t0)
            out[:, :, t0:t1] = o.reshape(B, H, t1 - t0, d_h)
    return {"idx": idx_out, "rq": rq_out, "rq_f": rqf_out, "r_max": rmax_out, "out": out}


def med3x(x: torch.Tensor, median_mult: float = 3.0) -> dict:
    """Per-head median of chunk norms over the whole call, threshold and strict mask."""
    B, H, T, d_h = x.shape
    n = d_h // 4
    norms = x.reshape(B, H, T, n, 4).norm(dim=-1)
    flat = norms.permute(1, 0, 2, 3).reshape(H, -1).float()
    med = torch.quantile(flat, 0.5, dim=-1)
    thr32 = med * median_mult
    thr = thr32.view(1, H, 1, 1).to(norms.dtype)
    mask = norms > thr
    return {"norms": norms, "median": med, "threshold": thr.view(H), "mask": mask}


def outlier_quantize(x: torch.Tensor, joint: torch.Tensor, radius_bits: int,
                     median_mult: float = 3.0, t_block: Optional[int] = None) -> dict:
    """Med3x wrapper: quantize everything, then restore the flagged chunks verbatim."""
    B, H, T, d_h = x.shape
    n = d_h // 4
    m = med3x(x, median_mult)
    q = quantize(x, joint, radius_bits, t_block=t_block)
    res = torch.where(m["mask"].unsqueeze(-1), x.reshape(B, H, T, n, 4), q["out"].view(B, H, T, n, 4))
    q.update(m)
    q["inner_out"] = q["out"]
    q["out"] = res.reshape(B, H, T, d_h)
    return q


def decode_kv(idx, radius_q, radius_scale, joint, r_qmax: int) -> torch.Tensor:
    """Codes -> dense (B, H, T, 4n): joint[h, idx] * ((rq * rs) / qmax), all in joint.dtype."""
    B, H, T, n = idx.shape
    K = joint.shape[1]
    table = joint.view(1, H, 1, 1, K, 4).expand(B, H, T, n, K, 4)
    gi = idx.long().view(B, H, T, n, 1, 1).expand(B, H, T, n, 1, 4)
    cw = table.gather(-2, gi).squeeze(-2)
    radius = (radius_q.to(joint.dtype) * radius_scale.unsqueeze(-1)) / r_qmax
    return (cw * radius.unsqueeze(-1)).view(B, H, T, 4 * n)


def sdpa(Q, K, V, causal: bool, softmax_scale: Optional[float] = None) -> torch.Tensor:
    """GQA broadcast + torch SDPA (top-left aligned causal mask when T_q != T_kv)."""
    H_q, H_kv = Q.shape[1], K.shape[1]
    assert H_q % H_kv == 0
    g = H_q // H_kv
    if g > 1:
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(Q.shape[-1])
    return F.scaled_dot_product_attention(Q, K, V, attn_mask=None, is_causal=causal, scale=softmax_scale)


def attention(Q, K_idx, K_rq, K_rs, joint_K, V_idx, V_rq, V_rs, joint_V, r_qmax: int,
              causal: bool = True, softmax_scale: Optional[float] = None) -> torch.Tensor:
    """Decode K and V densely, then SDPA."""
    K = decode_kv(K_idx, K_rq, K_rs, joint_K, r_qmax)
    V = decode_kv(V_idx, V_rq, V_rs, joint_V, r_qmax)
    return sdpa(Q, K, V, causal, softmax_scale)


def sdpa_masked_f32(Q, K, V, kv_lens=None, causal: bool = False, causal_offset: int = 0,
                    softmax_scale: Optional[float] = None) -> torch.Tensor:
    """fp32 attention with per-sequence KV lengths and an optional causal diagonal offset.

    Query row i may see key j iff j < kv_len[b] and (not causal or j <= i + causal_offset).
    Used for the ragged-length and bottom-right-aligned cases SDPA's flag cannot express.
    """
    B, H_q, T_q, d = Q.shape
    H_kv, T_kv = K.shape[1], K.shape[2]
    g = H_q // H_kv
    Kf = K.float().repeat_interleave(g, dim=1)
    Vf = V.float().repeat_interleave(g, dim=1)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float(), Kf) * softmax_scale
    j = torch.arange(T_kv).view(1, 1, 1, T_kv)
    allow = torch.ones(B, 1, T_q, T_kv, dtype=torch.bool)
    if kv_lens is not None:
        allow = allow & (j < torch.as_tensor(kv_lens).view(B, 1, 1, 1))
    if causal:
        i = torch.arange(T_q).view(1, 1, T_q, 1)
        allow = allow & (j <= i + causal_offset)
    s = s.masked_fill(~allow, float("-inf"))
    p = torch.softmax(s, dim=-1)
    p = torch.nan_to_num(p, nan=0.0)
    return torch.einsum("bhqk,bhkd->bhqd", p, Vf)
