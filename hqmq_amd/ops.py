"""Tensor-level wrappers over the C ABI: allocate outputs with torch, pass raw pointers.

Everything here runs on the GPU through libhqmq_amd.so; there is no CPU path.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib as L


def _dt(t: torch.Tensor) -> int:
    try:
        return L.DT_CODE[t.dtype]
    except KeyError:
        raise L.HqmqError(f"unsupported dtype {t.dtype}; expected float32, float16 or bfloat16") from None


def build_joint(raw_hs4: torch.Tensor, dtype: torch.dtype):
    """(H, S, 4) fp32 raw secondaries on the GPU -> (joint (H, 24S, 4) in dtype, slack (H,) fp32)."""
    L.require_gpu(raw_hs4, "raw")
    raw = raw_hs4.detach().to(torch.float32).contiguous()
    H, S, _ = raw.shape
    joint = torch.empty(H, 24 * S, 4, dtype=dtype, device=raw.device)
    slack = torch.empty(H, dtype=torch.float32, device=raw.device)
    with torch.cuda.device(raw.device):
        L.check(L.lib().hqmq_build_joint(L.ptr(raw), C.c_int(H), C.c_int(S), C.c_int(L.DT_CODE[dtype]), L.ptr(joint),
                                         L.ptr(slack), L.stream_ptr(raw.device)), "hqmq_build_joint")
    return joint, slack


def _strided_x(x: torch.Tensor):
    if x.dim() != 4:
        raise ValueError(f"expected (B, H, T, d_head), got {tuple(x.shape)}")
    if x.shape[-1] > 1 and x.stride(-1) != 1:
        x = x.contiguous()
    return x


def quantize(x: torch.Tensor, joint: torch.Tensor, slack: Optional[torch.Tensor], radius_bits: int, *,
             want_codes: bool = True, want_dense: bool = False, thr: Optional[torch.Tensor] = None,
             want_mask: bool = False, cache=None, t_off: int = 0, pos: Optional[torch.Tensor] = None,
             algo: int = 0, stats: Optional[torch.Tensor] = None) -> dict:
    """Run the quantize kernel on x (B, H, T, d_h).

    Returns a dict with the requested outputs: idx/rq (int32), r_max (dtype of x),
    out (fake-quant tensor), mask (bool).  `cache` is a PackedTensor whose rows
    [t_off, t_off + T) (shifted by pos[b] per sequence) receive the packed codes.
    """
    L.require_gpu(x, "x")
    x = _strided_x(x)
    B, H, T, d_h = x.shape
    if d_h % 4 != 0:
        raise ValueError(f"d_head={d_h} not divisible by 4")
    n = d_h // 4
    S = joint.shape[1] // 24
    if joint.dtype != x.dtype or joint.shape[0] != H or not joint.is_contiguous():
        raise ValueError("joint must be a contiguous (H, 24S, 4) table in the dtype of x")
    dev = x.device
    a = L.QuantizeArgs()
    a.x = L.ptr(x)
    a.x_stride_b, a.x_stride_h, a.x_stride_t = x.stride(0), x.stride(1), x.stride(2)
    a.dtype = _dt(x)
    a.B, a.H, a.T, a.n_chunks = B, H, T, n
    a.joint = L.ptr(joint)
    a.slack = L.ptr(slack)
    a.secondary_size, a.radius_bits, a.algo = S, radius_bits, algo
    out = {}
    keep = [x, joint, slack]
    if want_codes:
        out["idx"] = torch.empty(B, H, T, n, dtype=torch.int32, device=dev)
        out["rq"] = torch.empty(B, H, T, n, dtype=torch.int32, device=dev)
        out["r_max"] = torch.empty(B, H, T, dtype=x.dtype, device=dev)
        a.idx_out, a.rq_out, a.rmax_out = L.ptr(out["idx"]), L.ptr(out["rq"]), L.ptr(out["r_max"])
    if want_dense:
        out["out"] = torch.empty(B, H, T, d_h, dtype=x.dtype, device=dev)
        a.dense_out = L.ptr(out["out"])
    if thr is not None:
        thr = thr.to(x.dtype).contiguous()
        keep.append(thr)
        a.thr = L.ptr(thr)
        if want_mask:
            out["mask8"] = torch.empty(B, H, T, n, dtype=torch.uint8, device=dev)
            a.mask_out = L.ptr(out["mask8"])
    if cache is not None:
        a.main_plane, a.aux_plane = L.ptr(cache.main), L.ptr(cache.aux)
        a.scale_plane = L.ptr(cache.scale)
        a.flag_plane = L.ptr(cache.flags) if thr is not None else None
        a.t_cap, a.t_off = cache.t_cap, t_off
        a.main_bits, a.aux_bits = cache.main_bits, cache.aux_bits
        if pos is not None:
            pos = pos.to(device=dev, dtype=torch.int32).contiguous()
            keep.append(pos)
            a.pos = L.ptr(pos)
    a.stats = L.ptr(stats)
    if T > 0:
        with torch.cuda.device(dev):
            L.check(L.lib().hqmq_quantize(C.byref(a), L.stream_ptr(dev)), "hqmq_quantize")
    if "mask8" in out:
        out["mask"] = out.pop("mask8").bool()
    return out
