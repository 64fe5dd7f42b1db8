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
        a.scale_max_bits = L.ptr(cache.scale_max)
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


_WS = {}

# torch.quantile refuses more than 2^24 elements along the reduced dimension ("quantile() input tensor is too large"),
# which bounds the chunks per head of one Med-C call of the reference (src/quantizers/outlier_aware.py:68).  The
# radix select here has no such bound; check_quantile_limit(..., strict=True) mirrors the reference's refusal.
QUANTILE_LIMIT = 1 << 24


def check_quantile_limit(chunks_per_head: int, strict: bool) -> bool:
    """True when a Med-C call of this size is within torch.quantile's limit.  Beyond it the reference raises; with
    strict=True so does this function (same exception type and message), otherwise the call is an extension."""
    ok = chunks_per_head <= QUANTILE_LIMIT
    if not ok and strict:
        raise RuntimeError("quantile() input tensor is too large")
    return ok


def _workspace(nbytes: int, device, tag: str) -> torch.Tensor:
    """A cached scratch buffer of at least nbytes (grown on demand, reused across calls on the same stream; any content)."""
    dev = torch.device(device)
    key = (tag, dev, torch.cuda.current_stream(dev).cuda_stream)     # calls on different streams may overlap
    buf = _WS.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, device=device)
        _WS[key] = buf
    return buf


def med3x_threshold(x: torch.Tensor, mult: float = 3.0, want_count: bool = True, strict_quantile_limit: bool = False):
    """Per-head (median fp32, threshold in x.dtype, #chunks above threshold int32) over the whole call.
    strict_quantile_limit: raise as the reference does when a head has more than 2^24 chunks in this call."""
    L.require_gpu(x, "x")
    x = _strided_x(x)
    B, H, T, d_h = x.shape
    n = d_h // 4
    check_quantile_limit(B * T * n, strict_quantile_limit)
    dev = x.device
    nbytes = int(L.lib().hqmq_med3x_workspace_bytes(C.c_int(H), C.c_int(_dt(x))))
    ws = _workspace(nbytes, dev, "med3x")
    med = torch.empty(H, dtype=torch.float32, device=dev)
    thr = torch.empty(H, dtype=x.dtype, device=dev)
    cnt = torch.empty(H, dtype=torch.int32, device=dev) if want_count else None     # written for every head
    with torch.cuda.device(dev):
        L.check(L.lib().hqmq_med3x_threshold(
            L.ptr(x), L.i64(x.stride(0)), L.i64(x.stride(1)), L.i64(x.stride(2)), C.c_int(_dt(x)), C.c_int(B), C.c_int(H),
            C.c_int(T), C.c_int(n), C.c_float(mult), L.ptr(ws), L.i64(ws.numel()), L.ptr(med), L.ptr(thr), L.ptr(cnt),
            L.stream_ptr(dev)), "hqmq_med3x_threshold")
    return med, thr, cnt


def outlier_mask(x: torch.Tensor, thr: torch.Tensor) -> torch.Tensor:
    """Boolean (B, H, T, n) mask of chunks whose norm exceeds the per-head threshold."""
    L.require_gpu(x, "x")
    x = _strided_x(x)
    B, H, T, d_h = x.shape
    thr = thr.to(x.dtype).contiguous()
    mask = torch.empty(B, H, T, d_h // 4, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        L.check(L.lib().hqmq_outlier_mask(
            L.ptr(x), L.i64(x.stride(0)), L.i64(x.stride(1)), L.i64(x.stride(2)), C.c_int(_dt(x)), C.c_int(B), C.c_int(H),
            C.c_int(T), C.c_int(d_h // 4), L.ptr(thr), L.ptr(mask), L.stream_ptr(x.device)), "hqmq_outlier_mask")
    return mask.bool()


def outlier_compact(x: torch.Tensor, cache, t_off: int = 0, pos: Optional[torch.Tensor] = None) -> None:
    """Append the flagged chunks of x (rows t_off.. of the cache) to the cache's sideband."""
    x = _strided_x(x)
    B, H, T, d_h = x.shape
    dev = x.device
    if pos is not None:
        pos = pos.to(device=dev, dtype=torch.int32).contiguous()
    rows = L.PackedRows()      # the planes of the same rows: a chunk that finds the sideband full goes back to a plain chunk
    rows.main_plane, rows.aux_plane, rows.scale_plane = L.ptr(cache.main), L.ptr(cache.aux), L.ptr(cache.scale)
    rows.idx_bits, rows.main_bits, rows.aux_bits, rows.qmax = cache.idx_bits, cache.main_bits, cache.aux_bits, cache.qmax
    with torch.cuda.device(dev):
        L.check(L.lib().hqmq_outlier_compact(
            L.ptr(x), L.i64(x.stride(0)), L.i64(x.stride(1)), L.i64(x.stride(2)), C.c_int(_dt(x)), C.c_int(B), C.c_int(H),
            C.c_int(T), C.c_int(d_h // 4), L.ptr(cache.flags), L.i64(cache.t_cap), C.c_int(t_off), L.ptr(pos),
            L.ptr(cache.sideband), L.i64(cache.sb_cap), L.ptr(cache.sb_tile_off), L.ptr(cache.sb_count),
            L.ptr(cache.sb_overflow), L.ptr(cache.sb_coord), C.byref(rows), L.stream_ptr(dev)), "hqmq_outlier_compact")


def append_kv(k: torch.Tensor, v: torch.Tensor, k_cache, v_cache, k_joint, k_slack, v_joint, v_slack, radius_bits: int, *,
              t_off: int = 0, pos: Optional[torch.Tensor] = None, median_mult: Optional[float] = None):
    """Quantize the new rows k, v (B, H, T, d_h) into rows t_off.. of the two PackedTensors (shifted by pos[b]),
    with Med-C extraction into their sidebands when median_mult is given.  Same results as med3x_threshold,
    quantize and outlier_compact for K and then for V; K and V of equal shape share every launch.
    Returns (k_count, v_count), the flagged chunks per head (int32 [H]) or (None, None)."""
    L.require_gpu(k, "k")
    L.require_gpu(v, "v")
    if k.shape[2] == 0 and v.shape[2] == 0:        # an empty tensor has no address to pass
        return None, None
    dev = k.device
    if pos is not None:
        pos = pos.to(device=dev, dtype=torch.int32).contiguous()
    keep = [pos]
    args, counts = [], []
    for tag, x, cache, joint, slack in (("k", k, k_cache, k_joint, k_slack), ("v", v, v_cache, v_joint, v_slack)):
        x = _strided_x(x)
        B, H, T, d_h = x.shape
        if d_h % 4 != 0:
            raise ValueError(f"d_head={d_h} not divisible by 4")
        if joint.dtype != x.dtype or joint.shape[0] != H or not joint.is_contiguous():
            raise ValueError("joint must be a contiguous (H, 24S, 4) table in the dtype of x")
        a = L.AppendArgs()
        q = a.q
        q.x = L.ptr(x)
        q.x_stride_b, q.x_stride_h, q.x_stride_t = x.stride(0), x.stride(1), x.stride(2)
        q.dtype = _dt(x)
        q.B, q.H, q.T, q.n_chunks = B, H, T, d_h // 4
        q.joint, q.slack = L.ptr(joint), L.ptr(slack)
        q.secondary_size, q.radius_bits, q.algo = joint.shape[1] // 24, radius_bits, 0
        q.main_plane, q.aux_plane, q.scale_plane = L.ptr(cache.main), L.ptr(cache.aux), L.ptr(cache.scale)
        q.t_cap, q.t_off = cache.t_cap, t_off
        q.main_bits, q.aux_bits = cache.main_bits, cache.aux_bits
        q.scale_max_bits = L.ptr(cache.scale_max)
        q.pos = L.ptr(pos)
        keep += [x, joint, slack]
        cnt = None
        if median_mult is not None and T > 0:
            nbytes = int(L.lib().hqmq_med3x_workspace_bytes(C.c_int(H), C.c_int(_dt(x))))
            ws = _workspace(nbytes, dev, "med3x_" + tag)
            med = torch.empty(H, dtype=torch.float32, device=dev)
            thr = torch.empty(H, dtype=x.dtype, device=dev)
            cnt = torch.empty(H, dtype=torch.int32, device=dev)      # every path of the library writes all H counts
            keep += [ws, med, thr]
            q.flag_plane = L.ptr(cache.flags)
            a.median_mult = median_mult
            a.med_workspace, a.med_workspace_bytes = L.ptr(ws), ws.numel()
            a.median, a.thr, a.n_out = L.ptr(med), L.ptr(thr), L.ptr(cnt)
            a.sideband, a.sb_cap = L.ptr(cache.sideband), cache.sb_cap
            a.sb_tile_off, a.sb_count = L.ptr(cache.sb_tile_off), L.ptr(cache.sb_count)
            a.overflow, a.sb_coord = L.ptr(cache.sb_overflow), L.ptr(cache.sb_coord)
        args.append(a)
        counts.append(cnt)
    with torch.cuda.device(dev):
        L.check(L.lib().hqmq_append_kv(C.byref(args[0]), C.byref(args[1]), L.stream_ptr(dev)), "hqmq_append_kv")
    return counts[0], counts[1]


def _i32(t: torch.Tensor) -> torch.Tensor:
    t = t if t.dtype == torch.int32 else t.to(torch.int32)
    return t if t.stride(-1) == 1 else t.contiguous()


def dequant(idx, radius_q, radius_scale, joint, r_qmax: int) -> torch.Tensor:
    """Unpacked codes -> dense (B, H, T, 4n) in joint.dtype (rounding of the reference's torch decode)."""
    L.require_gpu(idx, "idx")
    idx, rq = _i32(idx), _i32(radius_q)
    B, H, T, n = idx.shape
    rs = radius_scale.to(joint.dtype)
    if joint.stride(-1) != 1 or joint.stride(1) != 4:
        joint = joint.contiguous()
    out = torch.empty(B, H, T, 4 * n, dtype=joint.dtype, device=idx.device)
    with torch.cuda.device(idx.device):
        L.check(L.lib().hqmq_dequant(
            L.ptr(idx), L.i64(idx.stride(0)), L.i64(idx.stride(1)), L.i64(idx.stride(2)),
            L.ptr(rq), L.i64(rq.stride(0)), L.i64(rq.stride(1)), L.i64(rq.stride(2)),
            L.ptr(rs), L.i64(rs.stride(0)), L.i64(rs.stride(1)), L.i64(rs.stride(2)),
            L.ptr(joint), L.i64(joint.stride(0)), C.c_int(joint.shape[1]), C.c_int(_dt(joint)), C.c_int(B), C.c_int(H),
            C.c_int(T), C.c_int(n), C.c_int(r_qmax), L.ptr(out), L.stream_ptr(idx.device)), "hqmq_dequant")
    return out


def pack_codes(idx, radius_q, cache, T: Optional[int] = None) -> None:
    """Write unpacked int codes into rows [0, T) of a PackedTensor's code planes."""
    idx, rq = _i32(idx), _i32(radius_q)
    B, H, Ti, n = idx.shape
    T = Ti if T is None else T
    with torch.cuda.device(idx.device):
        L.check(L.lib().hqmq_pack_codes(
            L.ptr(idx), L.i64(idx.stride(0)), L.i64(idx.stride(1)), L.i64(idx.stride(2)),
            L.ptr(rq), L.i64(rq.stride(0)), L.i64(rq.stride(1)), L.i64(rq.stride(2)),
            C.c_int(B), C.c_int(H), C.c_int(T), C.c_int(n), C.c_int(cache.idx_bits), C.c_int(cache.main_bits),
            C.c_int(cache.aux_bits), L.ptr(cache.main), L.ptr(cache.aux), L.i64(cache.t_cap), L.stream_ptr(idx.device)),
            "hqmq_pack_codes")


def dequant_packed(cache, T: Optional[int] = None, mode: int = 0) -> torch.Tensor:
    """Packed cache -> dense (B, H, T, d_h); mode 0 = attention rounding, 1 = quantizer fake-quant rounding."""
    T = cache.length if T is None else T
    out = torch.empty(cache.B, cache.H, T, cache.d_head, dtype=cache.dtype, device=cache.device)
    s = cache.c_struct()
    with torch.cuda.device(cache.device):
        L.check(L.lib().hqmq_dequant_packed(
            C.byref(s), C.c_int(L.DT_CODE[cache.dtype]), C.c_int(cache.B), C.c_int(cache.H), C.c_int(T), C.c_int(cache.n),
            L.i64(cache.t_cap), C.c_int(cache.idx_bits), C.c_int(cache.main_bits), C.c_int(cache.aux_bits),
            C.c_int(cache.qmax), C.c_int(mode), L.ptr(out), L.stream_ptr(cache.device)), "hqmq_dequant_packed")
    return out


def pick_splits(B: int, H_q: int, H_kv: int, T_q: int, T_kv: int, ragged: bool = False) -> int:
    return int(L.lib().hqmq_attn_pick_splits(C.c_int(B), C.c_int(H_q), C.c_int(H_kv), C.c_int(T_q), C.c_int(T_kv),
                                             C.c_int(1 if ragged else 0)))


def longest_first(kv_lens: torch.Tensor) -> torch.Tensor:
    """The batch_order for a ragged batch: sequences sorted by length, longest first (int32, on kv_lens' device).
    It stays valid while all sequences grow in step, so a decode loop computes it once."""
    return torch.argsort(kv_lens, descending=True, stable=True).to(torch.int32)


def attn_fwd(Q: torch.Tensor, Kc, Vc, T_kv: int, *, kv_lens: Optional[torch.Tensor] = None,
             kv_starts: Optional[torch.Tensor] = None, batch_order: Optional[torch.Tensor] = None, causal: bool = False,
             causal_offset: int = 0, softmax_scale: Optional[float] = None, n_splits: int = 0,
             out: Optional[torch.Tensor] = None, skip_combine: bool = False,
             force_generic: bool = False, kernel_events: Optional[tuple] = None,
             static_scratch: bool = False, workspace: Optional[torch.Tensor] = None, fp8_table_storage: bool = False):
    """Fused attention of Q (B, H_q, T_q, d_h) over packed K/V (PackedTensor each).
    kernel_events: two raw hipEvent_t handles (ints) that receive the GPU timestamps of the begin and the end of
    the main attention kernel (profiling).
    static_scratch: call hqmq_attn_fwd_static, which keeps the split partials in the library's own device array
    instead of a torch workspace (pass `out` as well and the call allocates nothing on the device).
    fp8_table_storage: both joint tables hold float8 e4m3 numbers (PackedTensor.with_fp8_table) and the kernel may keep
    them as float8 in LDS; same results, see include/hqmq_amd.h.
    skip_combine: leave the split partials unmerged and return (O, partials, n_splits): the partials are in `workspace`
    if given, else in a buffer of their own (never the cached scratch that the next call on the stream overwrites);
    attn_combine(partials, O, n_splits) merges them."""
    L.require_gpu(Q, "Q")
    if Q.stride(-1) != 1:
        Q = Q.contiguous()
    B, Hq, Tq, d_h = Q.shape
    if d_h != Kc.d_head or d_h != Vc.d_head:
        raise AssertionError(f"d_h={d_h} != n_chunks*4={Kc.d_head}")
    if Hq % Kc.H:
        raise AssertionError(f"H_q={Hq} must be divisible by H_kv={Kc.H}")
    if Q.dtype != Kc.dtype:
        raise L.HqmqError(f"Q dtype {Q.dtype} differs from the cache dtype {Kc.dtype}")
    dev = Q.device
    O = out if out is not None else torch.empty_like(Q)
    if softmax_scale is None:
        softmax_scale = d_h ** -0.5
    if n_splits <= 0:
        n_splits = pick_splits(B, Hq, Kc.H, Tq, max(T_kv, 1), kv_lens is not None)
    a = L.AttnArgs()
    a.Q, a.O = L.ptr(Q), L.ptr(O)
    a.q_sb, a.q_sh, a.q_st = Q.stride(0), Q.stride(1), Q.stride(2)
    a.o_sb, a.o_sh, a.o_st = O.stride(0), O.stride(1), O.stride(2)
    a.K, a.V = Kc.c_struct(), Vc.c_struct()
    a.dtype = L.DT_CODE[Q.dtype]
    a.B, a.H_q, a.H_kv, a.T_q, a.T_kv, a.n_chunks = B, Hq, Kc.H, Tq, T_kv, Kc.n
    a.t_cap = Kc.t_cap
    a.idx_bits, a.main_bits, a.aux_bits, a.qmax = Kc.idx_bits, Kc.main_bits, Kc.aux_bits, Kc.qmax
    keep = None
    if kv_lens is not None:
        keep = kv_lens.to(device=dev, dtype=torch.int32).contiguous()
        a.kv_len = L.ptr(keep)
    keep_start = None
    if kv_starts is not None:
        keep_start = kv_starts.to(device=dev, dtype=torch.int32).contiguous()
        if keep_start.numel() != B:
            raise L.HqmqError(f"kv_starts must hold one entry per sequence ({B})")
        a.kv_start = L.ptr(keep_start)
    keep_order = None
    if batch_order is not None:
        keep_order = batch_order.to(device=dev, dtype=torch.int32).contiguous()
        if keep_order.numel() != B:
            raise L.HqmqError(f"batch_order must be a permutation of the {B} sequences")
        a.batch_order = L.ptr(keep_order)
    a.causal, a.causal_offset, a.softmax_scale = int(causal), causal_offset, softmax_scale
    a.n_splits = n_splits
    a.skip_combine = int(skip_combine)
    a.force_generic = int(force_generic)
    a.fp8_table_storage = int(fp8_table_storage)
    a.wide_range = int(bool(getattr(Vc, "wide_range", False)))      # V scales outside [2^-8, 2^15): the generic kernel guards the range
    if kernel_events is not None:
        a.start_event, a.stop_event = C.c_void_p(kernel_events[0]), C.c_void_p(kernel_events[1])
    ws = None
    if static_scratch:
        with torch.cuda.device(dev):
            L.check(L.lib().hqmq_attn_fwd_static(C.byref(a), L.stream_ptr(dev)), "hqmq_attn_fwd_static")
        return O
    if n_splits > 1:
        nbytes = int(L.lib().hqmq_attn_workspace_bytes(C.c_int(B), C.c_int(Hq), C.c_int(Tq), C.c_int(d_h), C.c_int(n_splits)))
        if workspace is not None:
            if workspace.device != dev or workspace.numel() * workspace.element_size() < nbytes:
                raise L.HqmqError(f"workspace must hold {nbytes} bytes on {dev}")
            ws = workspace
        elif skip_combine:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        else:
            ws = _workspace(nbytes, dev, "attn")
        a.workspace, a.workspace_bytes = L.ptr(ws), ws.numel() * ws.element_size()
    with torch.cuda.device(dev):
        L.check(L.lib().hqmq_attn_fwd(C.byref(a), L.stream_ptr(dev)), "hqmq_attn_fwd")
    if skip_combine:
        return O, ws, n_splits
    return O


def attn_combine(partials: Optional[torch.Tensor], O: torch.Tensor, n_splits: int) -> torch.Tensor:
    """Merge the split partials a skip_combine call left behind into O (B, H_q, T_q, d_h)."""
    if n_splits <= 1 or partials is None:
        return O
    B, Hq, Tq, d_h = O.shape
    with torch.cuda.device(O.device):
        L.check(L.lib().hqmq_attn_combine(L.ptr(partials), L.ptr(O), C.c_int(L.DT_CODE[O.dtype]), C.c_int(B), C.c_int(Hq),
                                          C.c_int(Tq), C.c_int(d_h), C.c_int(n_splits), L.i64(O.stride(0)), L.i64(O.stride(1)),
                                          L.i64(O.stride(2)), L.stream_ptr(O.device)), "hqmq_attn_combine")
    return O
