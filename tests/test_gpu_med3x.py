"""GPU parity for Med3x: radix-select median, threshold, mask, flag plane and outlier sideband."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as CO
from oracle import torch_oracle as TO
from tests.helpers import DT, bit_equal, kv_input, unbits

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a GPU")]
DEV = "cuda"


@pytest.mark.parametrize("dn", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 3, 70, 64), (1, 2, 5, 12), (1, 1, 1, 128), (3, 4, 257, 128), (2, 2, 4200, 128)])
def test_median_threshold_count(dn, shape):
    """Even and odd chunk counts, tiny calls (one decode token), all dtypes (fp32 takes the two-pass select)."""
    from hqmq_amd import ops
    dt = DT[dn]
    x = kv_input(shape, dt, seed=sum(shape), outlier_p=0.04)
    want = CO.med3x(x, 3.0)
    med, thr, cnt = ops.med3x_threshold(x.to(DEV), 3.0)
    assert torch.equal(med.cpu(), want["median"])
    assert bit_equal(thr, want["threshold"])
    assert torch.equal(cnt.cpu().long(), want["mask"].sum(dim=(0, 2, 3)))
    assert torch.equal(ops.outlier_mask(x.to(DEV), thr).cpu(), want["mask"])


def test_median_with_duplicates_and_nan():
    from hqmq_amd import ops
    x = torch.ones(1, 2, 8, 16).half()           # every norm equal: both middle ranks fall in one bin
    x[0, 1, :, :] *= torch.arange(1, 9).view(8, 1)
    want = CO.med3x(x)
    med, thr, cnt = ops.med3x_threshold(x.to(DEV))
    assert torch.equal(med.cpu(), want["median"]) and bit_equal(thr, want["threshold"])
    x[0, 0, 2, 5] = float("nan")                 # a NaN norm makes that head's quantile NaN and its mask empty
    want = CO.med3x(x)
    med, thr, cnt = ops.med3x_threshold(x.to(DEV))
    assert torch.isnan(med[0]).item() and float(med[1]) == float(want["median"][1])
    assert int(cnt[0]) == 0 and not ops.outlier_mask(x.to(DEV), thr)[:, 0].any()


def test_outlier_golden_outputs(golden_dir):
    """with_outlier_extraction(...).quantize_K/V reproduce the reference's outputs bit for bit; the running
    outlier rate and bits_per_value match too."""
    import hqmq
    g = np.load(golden_dir / "outlier.npz")
    for cfg in ("s24r3", "s96r4"):
        S, b_r, seed, L, H = (int(v) for v in g[cfg + "_meta"])
        inner = hqmq.HQMQ(n_layers=L, n_heads=H, secondary_size=S, radius_bits=b_r, device=DEV, seed=seed)
        for dn, dt in DT.items():
            w = hqmq.with_outlier_extraction(inner, C=3.0)
            for kv, tag in ((0, "K"), (1, "V")):
                key = f"{cfg}_{dn}_{tag}"
                x = unbits(g[key + "_x"], dt).to(DEV)
                y = w.quantize_K(x, 0) if kv == 0 else w.quantize_V(x, 0)
                assert bit_equal(y, unbits(g[key + "_out"], dt)), key
            rate, n_obs, bpv = g[f"{cfg}_{dn}_rate"]
            assert abs(w.bits_per_value() - bpv) < 1e-6
            assert w._n_observations == int(n_obs) and abs(w._observed_outlier_rate - rate) < 1e-7


def test_generic_wrapper_matches_hqmq_wrapper():
    import hqmq
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=24, radius_bits=3, device=DEV)
    x = kv_input((2, 2, 40, 64), torch.float16, seed=4, outlier_p=0.05).to(DEV)
    a = hqmq.with_outlier_extraction(q, C=3.0).quantize_K(x, 0)
    b = hqmq.with_outlier_extraction(q, C=3.0, generic=True).quantize_K(x, 0)
    assert bit_equal(a, b)


@pytest.mark.parametrize("S,b_r,dn,d_h", [(24, 3, "bf16", 128), (96, 4, "bf16", 64), (192, 6, "fp16", 128), (24, 3, "fp32", 32)])
def test_flags_and_sideband_match_oracle(S, b_r, dn, d_h):
    """Bulk quantize with Med3x into the packed cache: flag plane, sideband order, tile offsets, counts, and
    the dense decode with outliers substituted."""
    import hqmq
    from hqmq_amd import ops
    dt = DT[dn]
    B, H, T = 2, 2, 150
    n = d_h // 4
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=S, radius_bits=b_r, device=DEV, seed=5))
    k = kv_input((B, H, T, d_h), dt, seed=S, outlier_p=0.03)
    v = kv_input((B, H, T, d_h), dt, seed=S + 1, outlier_p=0.01, outlier_gain=(5, 10))
    cache = w.new_cache(B, T, d_h, dt, 0)
    w.append(cache, k.to(DEV), v.to(DEV), 0)
    cache.K.check_overflow()
    for pt, x, kv in ((cache.K, k, 0), (cache.V, v, 1)):
        Jc = CO.joint_table(TO.secondary_raw(1, H, S, 5)[0, :, kv], dt)
        want = CO.outlier_quantize(x, Jc, b_r, 3.0)
        assert int(want["mask"].sum()) > 0
        assert torch.equal(pt.flags[:, :, :T].cpu(), CO.pack_flags(want["mask"]))
        # packed codes: a flagged chunk keeps its idx and carries radius code 0
        rq0 = torch.where(want["mask"], torch.zeros_like(want["rq"]), want["rq"])
        main, aux = CO.pack_rows(want["idx"], rq0, pt.idx_bits, pt.main_bits, pt.aux_bits)
        assert torch.equal(pt.main[:, :, :T].cpu(), main)
        if aux is not None:
            assert torch.equal(pt.aux[:, :, :T].cpu(), aux)
        for b in range(B):
            for h in range(H):
                sb, toff, cnt = CO.pack_sideband(x[b, h], want["mask"][b, h])
                assert int(pt.sb_count[b, h]) == cnt
                assert bit_equal(pt.sideband[b, h, :cnt], sb)
                assert torch.equal(pt.sb_tile_off[b, h, :toff.numel()].cpu(), toff)
                assert torch.equal(pt.sb_coord[b, h, :cnt].cpu(), CO.pack_coords(want["mask"][b, h]))
        assert bit_equal(ops.dequant_packed(pt, T, mode=1), want["out"])
        dense = CO.dequant(want["idx"], want["rq"], want["r_max"], Jc, pt.qmax).view(B, H, T, n, 4)
        dense = torch.where(want["mask"].unsqueeze(-1), x.view(B, H, T, n, 4), dense).reshape(B, H, T, d_h)
        assert bit_equal(ops.dequant_packed(pt, T, mode=0), dense)
    assert cache.nbytes() == sum(pt.B * pt.H * T * pt.row_bytes() + int(pt.sb_count.sum()) * 4 * pt.scale.element_size()
                                 for pt in (cache.K, cache.V))


@pytest.mark.parametrize("dn,d_h", [("fp16", 128), ("bf16", 64)])
def test_bulk_append_compaction_then_more_appends(dn, d_h):
    """A long first append takes the tile-parallel compaction (ragged last tile), the following appends the
    in-order one; flags, sideband order, tile offsets and counts equal the oracle's over all rows."""
    import hqmq
    dt = DT[dn]
    B, H, T1, T2, T3 = 2, 3, 1000, 24, 1
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=24, radius_bits=3, device=DEV))
    cache = w.new_cache(B, T1 + T2 + T3, d_h, dt, 0, sideband_frac=0.5)
    ks = kv_input((B, H, T1 + T2 + T3, d_h), dt, seed=17, outlier_p=0.04)
    cuts = [0, T1, T1 + T2, T1 + T2 + T3]
    for a, b in zip(cuts[:-1], cuts[1:]):
        w.append(cache, ks[:, :, a:b].to(DEV), ks[:, :, a:b].to(DEV), 0)
    cache.K.check_overflow()
    masks = torch.cat([CO.med3x(ks[:, :, a:b].contiguous())["mask"] for a, b in zip(cuts[:-1], cuts[1:])], dim=2)
    assert torch.equal(cache.K.flags[:, :, :cuts[-1]].cpu(), CO.pack_flags(masks))
    for b in range(B):
        for h in range(H):
            sb, toff, cnt = CO.pack_sideband(ks[b, h], masks[b, h])
            assert int(cache.K.sb_count[b, h]) == cnt and cnt > 0
            assert bit_equal(cache.K.sideband[b, h, :cnt], sb)
            assert torch.equal(cache.K.sb_tile_off[b, h, :toff.numel()].cpu(), toff)
            assert torch.equal(cache.K.sb_coord[b, h, :cnt].cpu(), CO.pack_coords(masks[b, h]))


def test_decode_appends_keep_sideband_consistent():
    """Token-by-token appends (each call has its own per-head median, as the reference's cache hook does)
    leave the same planes as the oracle run call by call, across tile boundaries."""
    import hqmq
    dt = torch.bfloat16
    B, H, d_h, steps = 4, 2, 128, 37
    n = d_h // 4
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=24, radius_bits=3, device=DEV))
    cache = w.new_cache(B, steps, d_h, dt, 0, sideband_frac=0.5)
    ks = kv_input((B, H, steps, d_h), dt, seed=7, outlier_p=0.05)
    vs = kv_input((B, H, steps, d_h), dt, seed=8)
    for t in range(steps):
        w.append(cache, ks[:, :, t:t + 1].to(DEV), vs[:, :, t:t + 1].to(DEV), 0)
    cache.K.check_overflow()
    Jc = CO.joint_table(TO.secondary_raw(1, H, 24, 42)[0, :, 0], dt)
    masks = torch.cat([CO.med3x(ks[:, :, t:t + 1].contiguous())["mask"] for t in range(steps)], dim=2)
    assert torch.equal(cache.K.flags[:, :, :steps].cpu(), CO.pack_flags(masks))
    for b in range(B):
        for h in range(H):
            sb, toff, cnt = CO.pack_sideband(ks[b, h], masks[b, h])
            assert int(cache.K.sb_count[b, h]) == cnt and bit_equal(cache.K.sideband[b, h, :cnt], sb)
            assert torch.equal(cache.K.sb_tile_off[b, h, :toff.numel()].cpu(), toff)
    assert w._n_observations == 0 and len(w._pending) == 2 * steps     # no device sync per call
    w.bits_per_value()
    assert w._n_observations == 2 * steps


@pytest.mark.parametrize("dn,d_h,med,ragged", [("bf16", 128, True, True), ("fp16", 64, True, False), ("fp16", 128, False, True),
                                               ("fp32", 32, True, False)])
def test_shared_launches_equal_single_tensor_calls(dn, d_h, med, ragged):
    """append() sends K and V through every stage together (one launch per stage when the shapes allow it, one
    after the other for fp32 and for bulk appends); every plane, the sideband and the counters equal those of the
    single-tensor calls, for a bulk append followed by short ones."""
    import hqmq
    dt = DT[dn]
    B, H, T0 = 3, 2, 640
    steps = [T0, 1, 0, 1, 5, 1, 16, 3]        # an empty append changes nothing
    total = sum(steps) + 8
    inner = hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=24, radius_bits=3, device=DEV)
    w = hqmq.with_outlier_extraction(inner) if med else inner
    mult = w.median_mult if med else None
    make = lambda: w.new_cache(B, total, d_h, dt, 0, sideband_frac=0.5) if med else w.new_cache(B, total, d_h, dt, 0)
    both, single = make(), make()
    ks = kv_input((B, H, total, d_h), dt, seed=3, outlier_p=0.05).to(DEV)
    vs = kv_input((B, H, total, d_h), dt, seed=4, outlier_p=0.02).to(DEV)
    pos = torch.tensor([0, 3, 7], dtype=torch.int32, device=DEV) if ragged else None
    t = 0
    for n_new in steps:
        k, v = ks[:, :, t:t + n_new], vs[:, :, t:t + n_new]
        w.append(both, k, v, 0, pos=pos)
        if n_new:
            inner._append_one(single.K, k, 0, 0, pos, median_mult=mult)
            inner._append_one(single.V, v, 0, 1, pos, median_mult=mult)
        if pos is not None:
            pos = pos + n_new
        t += n_new
    names = ["main", "aux", "scale"] + (["flags", "sideband", "sb_tile_off", "sb_count", "sb_coord", "sb_overflow"] if med else [])
    for a, b in ((both.K, single.K), (both.V, single.V)):
        for name in names:
            x, y = getattr(a, name), getattr(b, name)
            if x is None and y is None:
                continue
            assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), name
        assert a.length == b.length
    if med:
        assert int(both.V.sb_count.sum()) > 0


def test_sideband_overflow_is_reported():
    import hqmq
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=1, secondary_size=24, radius_bits=3, device=DEV))
    cache = w.new_cache(1, 512, 128, torch.float16, 0, sideband_frac=0.001)   # room for 64 chunks only
    x = kv_input((1, 1, 512, 128), torch.float16, seed=3, outlier_p=0.2).to(DEV)
    w.append(cache, x, x, 0)
    with pytest.raises(hqmq.HqmqError):
        cache.K.check_overflow()


def test_full_size_median_properties():
    """Config-3 scale per head (8.4 M chunk norms): the selected median splits the norms in half and the
    count above the threshold equals a direct count (size-independent properties; no CPU sort of 8 M values
    per head in the test)."""
    from hqmq_amd import ops
    x = kv_input((8, 2, 32768, 128), torch.float16, seed=11, lognormal=False, outlier_p=0.02).to(DEV)
    med, thr, cnt = ops.med3x_threshold(x, 3.0)
    mask = ops.outlier_mask(x, thr)                      # direct count vs the histogram-derived count
    assert torch.equal(mask.sum(dim=(0, 2, 3)).to(torch.int32), cnt)
    norms = x.view(8, 2, 32768, 32, 4).float().norm(dim=-1)    # torch on the GPU, approximate: for the split check only
    for h in range(2):
        nh = norms[:, h].reshape(-1)
        N = nh.numel()
        slack = N // 1000                                        # torch's norm may round a few values the other way
        assert int((nh < med[h]).sum()) <= N // 2 + slack and int((nh > med[h]).sum()) <= N // 2 + slack
    assert 0.01 < float(cnt.sum()) / norms.numel() < 0.04


@pytest.mark.parametrize("dn,S,b_r,T,p,single", [("fp16", 96, 4, 600, 0.06, False), ("bf16", 24, 3, 600, 0.06, False), ("fp16", 192, 6, 100, 0.1, False),
                                                 ("bf16", 96, 4, 8, 0.4, False), ("fp16", 24, 3, 8, 0.4, False), ("fp16", 96, 4, 100, 0.1, True)])
def test_full_sideband_degrades_to_plain_chunks(dn, S, b_r, T, p, single):
    """A sideband that is too small: the flagged chunks that find no room (the last ones of a (b, h) stream in
    (row, chunk) order) are stored as plain HQMQ chunks (flag cleared, the quantizer's radius code), so the cache
    decodes them to the inner quantizer's value, never to zero (the reference never loses an outlier,
    outlier_aware.py:86).  Planes, counters and the dense decode against the oracle, through every compaction path: the
    tile-parallel passes (T = 600), the in-order kernel (T = 100), the quantize launch itself (T = 8), and the
    single-tensor entry points (`single`); then attention over such a cache with both kernels."""
    import hqmq
    from hqmq_amd import ops
    from tests.helpers import assert_attention_close, masked_two_refs
    dt = DT[dn]
    B, H, d_h = 2, 2, 128
    n = d_h // 4
    inner = hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=S, radius_bits=b_r, device=DEV, seed=5)
    w = hqmq.with_outlier_extraction(inner)
    k = kv_input((B, H, T, d_h), dt, seed=S + T, outlier_p=p)
    v = kv_input((B, H, T, d_h), dt, seed=S + T + 1, outlier_p=p, outlier_gain=(20, 40))
    cache = w.new_cache(B, T, d_h, dt, 0, sideband_frac=1e-6)
    cap = cache.K.sb_cap
    assert cap == 64
    if single:
        w.inner._append_one(cache.K, k.to(DEV), 0, 0, None, median_mult=3.0)       # med3x, quantize and compaction as three calls
        w.inner._append_one(cache.V, v.to(DEV), 0, 1, None, median_mult=3.0)
    else:
        w.append(cache, k.to(DEV), v.to(DEV), 0)
    assert cache.K.overflowed() and cache.V.overflowed()
    with pytest.raises(Exception):
        cache.K.check_overflow()
    for pt, x, kv in ((cache.K, k, 0), (cache.V, v, 1)):
        Jc = CO.joint_table(TO.secondary_raw(1, H, S, 5)[0, :, kv], dt)
        want = CO.outlier_quantize(x, Jc, b_r, 3.0)
        order = want["mask"].reshape(B, H, T * n).long().cumsum(-1).reshape(B, H, T, n)      # 1-based rank in (row, chunk) order
        kept = want["mask"] & (order <= cap)
        assert int((want["mask"] & ~kept).sum()) > 0
        assert torch.equal(pt.flags[:, :, :T].cpu(), CO.pack_flags(kept))
        rq0 = torch.where(kept, torch.zeros_like(want["rq"]), want["rq"])
        main, aux = CO.pack_rows(want["idx"], rq0, pt.idx_bits, pt.main_bits, pt.aux_bits)
        assert torch.equal(pt.main[:, :, :T].cpu(), main)
        if aux is not None:
            assert torch.equal(pt.aux[:, :, :T].cpu(), aux)
        for b in range(B):
            for h in range(H):
                sb, _, cnt = CO.pack_sideband(x[b, h], kept[b, h])
                assert cnt == cap and int(pt.sb_count[b, h]) == int(want["mask"][b, h].sum())       # the counter keeps counting
                assert bit_equal(pt.sideband[b, h, :cap], sb)
                assert torch.equal(pt.sb_coord[b, h, :cap].cpu(), CO.pack_coords(kept[b, h]))
        expect = torch.where(kept.unsqueeze(-1), x.view(B, H, T, n, 4), want["inner_out"].view(B, H, T, n, 4)).reshape(B, H, T, d_h)
        assert bit_equal(ops.dequant_packed(pt, T, mode=1), expect)
    Q = torch.randn(B, 4, 1, d_h, generator=torch.Generator().manual_seed(9)).to(dt).to(DEV)
    refs = masked_two_refs(cache, Q, T)
    scale = max(1.0, float(refs[0].abs().max()))
    for generic in (False, True):
        O = hqmq.fused_attention_packed(Q, cache, force_generic=generic)
        assert torch.isfinite(O).all()
        assert_attention_close(O, *refs, base=2e-3 * scale, what=f"generic={generic}")
