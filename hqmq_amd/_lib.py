"""ctypes binding of libhqmq_amd.so (declared in include/hqmq_amd.h).

There is no CPU fallback: if the library is missing or a call fails, this
module raises.  torch owns every buffer; kernels run on torch's current stream.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
_SO = _HERE / "libhqmq_amd.so"
_lib = None

F32, F16, BF16 = 0, 1, 2
DT_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

vp = C.c_void_p
i64 = C.c_int64


class HqmqError(RuntimeError):
    pass


class QuantizeArgs(C.Structure):
    _fields_ = [
        ("x", vp), ("x_stride_b", i64), ("x_stride_h", i64), ("x_stride_t", i64),
        ("dtype", C.c_int), ("B", C.c_int), ("H", C.c_int), ("T", C.c_int), ("n_chunks", C.c_int),
        ("joint", vp), ("slack", vp), ("secondary_size", C.c_int), ("radius_bits", C.c_int), ("algo", C.c_int),
        ("idx_out", vp), ("rq_out", vp), ("rmax_out", vp), ("dense_out", vp),
        ("thr", vp), ("mask_out", vp),
        ("main_plane", vp), ("aux_plane", vp), ("flag_plane", vp), ("scale_plane", vp),
        ("t_cap", i64), ("t_off", C.c_int), ("pos", vp), ("main_bits", C.c_int), ("aux_bits", C.c_int),
        ("stats", vp), ("scale_max_bits", vp),
    ]


class AppendArgs(C.Structure):
    _fields_ = [
        ("q", QuantizeArgs), ("median_mult", C.c_float),
        ("med_workspace", vp), ("med_workspace_bytes", i64),
        ("median", vp), ("thr", vp), ("n_out", vp),
        ("sideband", vp), ("sb_cap", i64), ("sb_tile_off", vp), ("sb_count", vp), ("overflow", vp), ("sb_coord", vp),
    ]


class Packed(C.Structure):
    _fields_ = [
        ("main_plane", vp), ("aux_plane", vp), ("flag_plane", vp), ("scale_plane", vp),
        ("scale_sb", i64), ("scale_sh", i64), ("scale_st", i64),
        ("sideband", vp), ("sb_tile_off", vp), ("sb_cap", i64), ("sb_coord", vp), ("sb_count", vp),
        ("joint", vp), ("joint_sh", i64), ("K", C.c_int), ("scale_max_bits", vp),
    ]


class AttnArgs(C.Structure):
    _fields_ = [
        ("Q", vp), ("O", vp),
        ("q_sb", i64), ("q_sh", i64), ("q_st", i64), ("o_sb", i64), ("o_sh", i64), ("o_st", i64),
        ("K", Packed), ("V", Packed),
        ("dtype", C.c_int), ("B", C.c_int), ("H_q", C.c_int), ("H_kv", C.c_int), ("T_q", C.c_int),
        ("T_kv", C.c_int), ("n_chunks", C.c_int), ("t_cap", i64),
        ("idx_bits", C.c_int), ("main_bits", C.c_int), ("aux_bits", C.c_int), ("qmax", C.c_int),
        ("kv_len", vp), ("causal", C.c_int), ("causal_offset", i64), ("softmax_scale", C.c_float),
        ("n_splits", C.c_int), ("workspace", vp), ("workspace_bytes", i64), ("skip_combine", C.c_int), ("force_generic", C.c_int),
        ("kv_start", vp), ("batch_order", vp), ("start_event", vp), ("stop_event", vp),
        ("fp8_table_storage", C.c_int), ("wide_range", C.c_int),
    ]


class PackedRows(C.Structure):
    """hqmq_packed_rows: the packed planes of the rows a compaction call covers."""
    _fields_ = [("main_plane", vp), ("aux_plane", vp), ("scale_plane", vp),
                ("idx_bits", C.c_int), ("main_bits", C.c_int), ("aux_bits", C.c_int), ("qmax", C.c_int)]


EXPORTS = [
    "hqmq_version", "hqmq_status_string", "hqmq_layout_bits", "hqmq_build_joint", "hqmq_quantize",
    "hqmq_med3x_workspace_bytes", "hqmq_med3x_threshold", "hqmq_outlier_mask", "hqmq_outlier_compact", "hqmq_dequant",
    "hqmq_pack_codes", "hqmq_dequant_packed", "hqmq_attn_workspace_bytes", "hqmq_attn_pick_splits",
    "hqmq_attn_fwd", "hqmq_attn_combine", "hqmq_append_kv", "hqmq_attn_static_scratch_bytes", "hqmq_attn_fwd_static",
]
BENCH_EXPORTS = ["hqmq_bench_read_planes_sink_bytes", "hqmq_bench_read_planes", "hqmq_bench_read_plain", "hqmq_bench_read_lds",
                 "hqmq_bench_empty"]


def library_path() -> Path:
    return _SO


def lib():
    """The loaded shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not _SO.exists():
            raise HqmqError(f"{_SO} is missing: build it with `python -m hqmq_amd.build` (needs hipcc)")
        L = C.CDLL(str(_SO))
        L.hqmq_status_string.restype = C.c_char_p
        L.hqmq_status_string.argtypes = [C.c_int]
        for name in ("hqmq_med3x_workspace_bytes", "hqmq_attn_workspace_bytes", "hqmq_attn_static_scratch_bytes"):
            getattr(L, name).restype = i64
        _lib = L
    return _lib


_bench_lib = None


def bench_lib():
    """The measurement library (read-only probe kernels); loaded by bench.py and hqmq_amd/bench_ceiling.py only."""
    global _bench_lib
    if _bench_lib is None:
        so = _SO.with_name("libhqmq_bench.so")
        if not so.exists():
            raise HqmqError(f"{so} is missing: build it with `python -m hqmq_amd.build` (needs hipcc)")
        L = C.CDLL(str(so))
        L.hqmq_bench_read_planes_sink_bytes.restype = i64
        _bench_lib = L
    return _bench_lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = lib().hqmq_status_string(status).decode()
        raise HqmqError(f"{what} failed: status {status} ({msg})")


def ptr(t):
    """Device (or host) address of a tensor, NULL for None."""
    return vp(t.data_ptr()) if t is not None else vp(0)


def stream_ptr(device=None):
    return vp(torch.cuda.current_stream(device).cuda_stream)


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise HqmqError(f"{name} must be a GPU tensor: the HQMQ kernels have no CPU path")


def layout_bits(secondary_size: int, radius_bits: int):
    ib, mb, ab = C.c_int(), C.c_int(), C.c_int()
    check(lib().hqmq_layout_bits(C.c_int(secondary_size), C.c_int(radius_bits), C.byref(ib), C.byref(mb), C.byref(ab)),
          "hqmq_layout_bits")
    return ib.value, mb.value, ab.value
