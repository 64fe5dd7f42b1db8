"""ctypes binding of oracle/liborc.so (scalar C oracle).  TEST INFRASTRUCTURE ONLY.

All functions take and return CPU torch tensors; 16-bit tensors cross the
boundary as raw bit patterns.  Build the library with `make -C oracle`.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
_LIB = None
DT_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def build(force: bool = False) -> Path:
    so = _HERE / "liborc.so"
    if force or not so.exists():
        subprocess.run(["make", "-C", str(_HERE), "-B" if force else "-s"], check=True)
    return so


def lib():
    global _LIB
    if _LIB is None:
        _LIB = C.CDLL(str(build()))
    return _LIB


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def cell24() -> torch.Tensor:
    out = torch.empty(24, 4, dtype=torch.float32)
    lib().orc_cell24(_p(out))
    return out


def quat_mul(a: torch.Tensor, b: torch.Tensor, dtype) -> torch.Tensor:
    a32, b32 = a.float().contiguous(), b.float().contiguous()
    out = torch.empty(4, dtype=torch.float32)
    lib().orc_quat_mul(C.c_int(DT_CODE[dtype]), _p(a32), _p(b32), _p(out))
    return out


def round_array(x: torch.Tensor, dtype) -> torch.Tensor:
    x = x.float().contiguous()
    out = torch.empty_like(x)
    lib().orc_round_array(C.c_int(DT_CODE[dtype]), _p(x), _p(out), C.c_long(x.numel()))
    return out


def joint_table(raw_hs4: torch.Tensor, dtype) -> torch.Tensor:
    raw = raw_hs4.float().contiguous()
    H, S, _ = raw.shape
    out = torch.empty(H, 24 * S, 4, dtype=dtype)
    lib().orc_joint_table(_p(raw), C.c_int(H), C.c_int(S), C.c_int(DT_CODE[dtype]), _p(out))
    return out


def quantize(x: torch.Tensor, joint: torch.Tensor, radius_bits: int, dense: bool = True) -> dict:
    B, H, T, d_h = x.shape
    n = d_h // 4
    assert n <= 256 and joint.dtype == x.dtype
    x = x.contiguous()
    joint = joint.contiguous()
    S = joint.shape[1] // 24
    idx = torch.empty(B, H, T, n, dtype=torch.int32)
    rq = torch.empty(B, H, T, n, dtype=torch.int32)
    rqf = torch.empty(B, H, T, n, dtype=x.dtype)
    rmax = torch.empty(B, H, T, dtype=x.dtype)
    out = torch.empty_like(x) if dense else None
    lib().orc_quantize(_p(x), C.c_int(DT_CODE[x.dtype]), C.c_long(B), C.c_int(H), C.c_long(T), C.c_int(n),
                       _p(joint), C.c_int(S), C.c_int(radius_bits), _p(idx), _p(rq), _p(rqf), _p(rmax), _p(out))
    return {"idx": idx, "rq": rq, "rq_f": rqf, "r_max": rmax, "out": out}


def med3x(x: torch.Tensor, mult: float = 3.0) -> dict:
    B, H, T, d_h = x.shape
    n = d_h // 4
    x = x.contiguous()
    norms = torch.empty(B, H, T, n, dtype=x.dtype)
    med = torch.empty(H, dtype=torch.float32)
    thr = torch.empty(H, dtype=x.dtype)
    mask = torch.empty(B, H, T, n, dtype=torch.uint8)
    lib().orc_med3x(_p(x), C.c_int(DT_CODE[x.dtype]), C.c_long(B), C.c_int(H), C.c_long(T), C.c_int(n),
                    C.c_float(mult), _p(norms), _p(med), _p(thr), _p(mask))
    return {"norms": norms, "median": med, "threshold": thr, "mask": mask.bool()}


def outlier_quantize(x, joint, radius_bits: int, mult: float = 3.0) -> dict:
    q = quantize(x, joint, radius_bits)
    m = med3x(x, mult)
    merged = torch.empty_like(x)
    mask8 = m["mask"].to(torch.uint8).contiguous()
    x = x.contiguous()
    lib().orc_outlier_merge(_p(x), _p(q["out"]), _p(mask8), C.c_int(DT_CODE[x.dtype]),
                            C.c_long(mask8.numel()), _p(merged))
    q.update(m)
    q["inner_out"] = q["out"]
    q["out"] = merged
    return q


def dequant(idx, rq, rs, joint, qmax: int) -> torch.Tensor:
    B, H, T, n = idx.shape
    idx = idx.to(torch.int32).contiguous()
    rq = rq.to(torch.int32).contiguous()
    rs = rs.contiguous()
    joint = joint.contiguous()
    out = torch.empty(B, H, T, 4 * n, dtype=joint.dtype)
    lib().orc_dequant(_p(idx), _p(rq), _p(rs), _p(joint), C.c_int(DT_CODE[joint.dtype]), C.c_long(B), C.c_int(H),
                      C.c_long(T), C.c_int(n), C.c_int(joint.shape[1]), C.c_int(qmax), _p(out))
    return out


def attention_dense(Q, Kd, Vd, kv_lens=None, causal=False, causal_offset=0, softmax_scale=None) -> torch.Tensor:
    """softmax(Q K^T * scale) V over dense K/V with double accumulation; fp32 result."""
    B, Hq, Tq, d = Q.shape
    Hkv, Tkv = Kd.shape[1], Kd.shape[2]
    assert Q.dtype == Kd.dtype == Vd.dtype
    Q, Kd, Vd = Q.contiguous(), Kd.contiguous(), Vd.contiguous()
    lens = None if kv_lens is None else torch.as_tensor(kv_lens, dtype=torch.int32).contiguous()
    scale = softmax_scale if softmax_scale is not None else d ** -0.5
    out = torch.empty(B, Hq, Tq, d, dtype=torch.float32)
    lib().orc_attention(_p(Q), _p(Kd), _p(Vd), C.c_int(DT_CODE[Q.dtype]), C.c_long(B), C.c_int(Hq), C.c_int(Hkv),
                        C.c_long(Tq), C.c_long(Tkv), C.c_int(d), _p(lens), C.c_int(int(causal)),
                        C.c_long(causal_offset), C.c_double(scale), _p(out))
    return out


def pack_rows(idx, rq, idx_bits: int, main_bits: int, aux_bits: int):
    """(..., n) int32 codes -> (main uint8 (..., ceil(n*main_bits/8)), aux uint8 or None)."""
    lead, n = idx.shape[:-1], idx.shape[-1]
    rows = idx.numel() // n
    ms = (n * main_bits + 7) // 8
    as_ = (n * aux_bits + 7) // 8
    main = torch.empty(rows, ms, dtype=torch.uint8)
    aux = torch.empty(rows, as_, dtype=torch.uint8) if aux_bits else None
    idx32, rq32 = idx.to(torch.int32).contiguous(), rq.to(torch.int32).contiguous()  # keep alive across the call
    lib().orc_pack_rows(_p(idx32), _p(rq32), C.c_long(rows),
                        C.c_int(n), C.c_int(idx_bits), C.c_int(main_bits), C.c_int(aux_bits), _p(main),
                        C.c_long(ms), _p(aux), C.c_long(as_))
    return main.view(*lead, ms), (aux.view(*lead, as_) if aux is not None else None)


def pack_flags(mask: torch.Tensor) -> torch.Tensor:
    lead, n = mask.shape[:-1], mask.shape[-1]
    rows = mask.numel() // n
    st = (n + 7) // 8
    flags = torch.empty(rows, st, dtype=torch.uint8)
    mask8 = mask.to(torch.uint8).contiguous()  # keep alive across the call
    lib().orc_pack_flags(_p(mask8), C.c_long(rows), C.c_int(n), _p(flags), C.c_long(st))
    return flags.view(*lead, st)


def pack_coords(mask_bh: torch.Tensor) -> torch.Tensor:
    """One (b, h) stream: mask (T, n) -> int16 coordinates (t & 15) << 8 | c of the sideband entries."""
    T, n = mask_bh.shape
    m8 = mask_bh.to(torch.uint8).contiguous()
    out = torch.zeros(max(int(m8.sum()), 1), dtype=torch.int16)
    lib().orc_pack_coords.restype = C.c_long
    cnt = lib().orc_pack_coords(_p(m8), C.c_long(T), C.c_int(n), _p(out))
    return out[:cnt]


def pack_sideband(x_bh: torch.Tensor, mask_bh: torch.Tensor):
    """One (b, h) stream: x (T, 4n), mask (T, n) -> (sideband (count, 4), tile_off (ceil(T/16),), count)."""
    T, n = mask_bh.shape
    x_bh = x_bh.contiguous()
    m8 = mask_bh.to(torch.uint8).contiguous()
    cap = int(m8.sum())
    sb = torch.zeros(max(cap, 1), 4, dtype=x_bh.dtype)
    toff = torch.zeros((T + 15) // 16, dtype=torch.int32)
    lib().orc_pack_sideband.restype = C.c_long
    cnt = lib().orc_pack_sideband(_p(x_bh), _p(m8), C.c_int(DT_CODE[x_bh.dtype]), C.c_long(T), C.c_int(n), _p(sb), _p(toff))
    return sb[:cnt], toff, cnt
