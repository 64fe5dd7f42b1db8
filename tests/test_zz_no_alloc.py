"""hqmq_attn_fwd_static: the attention entry point that allocates nothing (split partials in a device array
that is part of the library) against hqmq_attn_fwd with a caller workspace, through the C ABI.

The two share their kernels and the choice of splits, so the outputs must be bit-identical.  Two calls in a
row, the second on a smaller input: the array keeps the first call's partials and the second must not see them.
"""
import ctypes as C

import pytest
import torch

from tests.helpers import as_bits, kv_input

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a GPU")]
DEV = "cuda"


def _args(L, Q, O, cache, T_kv, n_splits, ws=None):
    a = L.AttnArgs()
    a.Q, a.O = L.ptr(Q), L.ptr(O)
    a.q_sb, a.q_sh, a.q_st = Q.stride(0), Q.stride(1), Q.stride(2)
    a.o_sb, a.o_sh, a.o_st = O.stride(0), O.stride(1), O.stride(2)
    a.K, a.V = cache.K.c_struct(), cache.V.c_struct()
    a.dtype = L.DT_CODE[Q.dtype]
    a.B, a.H_q, a.H_kv, a.T_q, a.T_kv, a.n_chunks = Q.shape[0], Q.shape[1], cache.K.H, Q.shape[2], T_kv, cache.K.n
    a.t_cap = cache.K.t_cap
    a.idx_bits, a.main_bits, a.aux_bits, a.qmax = cache.K.idx_bits, cache.K.main_bits, cache.K.aux_bits, cache.K.qmax
    a.causal, a.causal_offset, a.softmax_scale = 0, 0, Q.shape[3] ** -0.5
    a.n_splits = n_splits
    if ws is not None:
        a.workspace, a.workspace_bytes = L.ptr(ws), ws.numel()
    return a


def _both(L, q, B, Hq, Hkv, T, d_h, dt, seed, n_splits, outliers):
    k = kv_input((B, Hkv, T, d_h), dt, seed, outlier_p=0.02 if outliers else 0).to(DEV)
    v = kv_input((B, Hkv, T, d_h), dt, seed + 1).to(DEV)
    cache = q.new_cache(B, T, d_h, dt, 0)
    q.append(cache, k, v, 0)
    Q = torch.randn(B, Hq, 1, d_h, generator=torch.Generator().manual_seed(seed + 2)).to(dt).to(DEV)
    lib, st = L.lib(), L.stream_ptr(DEV)
    ns = n_splits or int(lib.hqmq_attn_pick_splits(B, Hq, Hkv, 1, T, 0))
    need = int(lib.hqmq_attn_workspace_bytes(B, Hq, 1, d_h, ns))
    ws = torch.empty(max(need, 4), dtype=torch.uint8, device=DEV)
    O_ref, O_new = torch.full_like(Q, 7.0), torch.full_like(Q, -7.0)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    L.check(lib.hqmq_attn_fwd(C.byref(_args(L, Q, O_ref, cache, T, n_splits, ws)), st), "hqmq_attn_fwd")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]          # hipMemGetInfo: sees a hipMalloc inside the library, which torch's counters do not
    L.check(lib.hqmq_attn_fwd_static(C.byref(_args(L, Q, O_new, cache, T, n_splits)), st), "hqmq_attn_fwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before, "device memory was allocated during hqmq_attn_fwd_static"
    assert torch.cuda.memory_allocated() == before
    assert ns > 1, "the case must use split partials"
    assert not torch.isnan(O_new.float()).any()
    assert torch.equal(as_bits(O_new), as_bits(O_ref)), (
        f"T={T} n_splits={ns}: max abs diff {(O_new.float() - O_ref.float()).abs().max().item():.3e}")
    return need


def test_static_scratch_matches_workspace_entry_point():
    import hqmq
    from hqmq_amd import _lib as L
    dt = torch.float16
    q = hqmq.HQMQ(n_layers=1, n_heads=8, secondary_size=96, radius_bits=4, device=DEV)
    big = _both(L, q, 1, 32, 8, 8192, 128, dt, 11, 0, False)          # config 2 shape, 16 splits
    small = _both(L, q, 1, 32, 8, 1100, 128, dt, 21, 0, False)        # then a shorter cache: fewer splits
    assert small < big
    _both(L, q, 2, 32, 8, 640, 128, dt, 31, 5, False)                 # an explicit number of splits
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=4, secondary_size=24, radius_bits=3, device=DEV))
    _both(L, w, 2, 28, 4, 2048, 128, torch.bfloat16, 41, 0, True)     # an outlier cache (sideband path), bf16


def test_static_scratch_limit_is_an_error_not_an_overrun():
    import hqmq
    from hqmq_amd import _lib as L
    dt = torch.float16
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=24, radius_bits=3, device=DEV)
    T = 1024
    x = kv_input((1, 2, T, 64), dt, 5).to(DEV)
    cache = q.new_cache(1, T, 64, dt, 0)
    q.append(cache, x, x, 0)
    lib, st = L.lib(), L.stream_ptr(DEV)
    limit = int(lib.hqmq_attn_static_scratch_bytes())
    assert limit == 8 << 20
    Tq = 1024                                                          # a chunked prefill whose partials exceed the array
    Q = torch.randn(1, 8, Tq, 64, generator=torch.Generator().manual_seed(6)).to(dt).to(DEV)
    O = torch.zeros_like(Q)
    ns = 8
    assert int(lib.hqmq_attn_workspace_bytes(1, 8, Tq, 64, ns)) > limit
    rc = lib.hqmq_attn_fwd_static(C.byref(_args(L, Q, O, cache, T, ns)), st)
    assert rc == -7 and b"static scratch" in lib.hqmq_status_string(rc)
    torch.cuda.synchronize()
    assert float(O.abs().max()) == 0.0                                 # nothing was launched
    a = _args(L, Q[:, :, :1].contiguous(), O[:, :, :1].contiguous(), cache, T, 2)
    a.skip_combine = 1
    assert lib.hqmq_attn_fwd_static(C.byref(a), st) == -7
    # one split needs no partials at all
    Q1 = Q[:, :, :1].contiguous()
    O1, O2 = torch.zeros_like(Q1), torch.zeros_like(Q1)
    L.check(lib.hqmq_attn_fwd_static(C.byref(_args(L, Q1, O1, cache, T, 1)), st), "static, one split")
    L.check(lib.hqmq_attn_fwd(C.byref(_args(L, Q1, O2, cache, T, 1)), st), "one split")
    torch.cuda.synchronize()
    assert torch.equal(as_bits(O1), as_bits(O2)) and float(O1.abs().max()) > 0
