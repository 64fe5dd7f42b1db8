"""Range, limits and cache-consistency cases around the attention and quantizer entry points (GPU)."""
import pytest
import torch

from oracle import c_oracle as CO
from oracle import torch_oracle as TO
from tests.helpers import assert_attention_close, attention_refs, bit_equal, dense_from_codes, kv_input

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a GPU")]
DEV = "cuda"


@pytest.mark.parametrize("k_gain,v_gain", [(1.0, 1e5), (1e5, 1e5), (1e-3, 3e7), (1.0, 1e-6), (1e-6, 3e-8)])
@pytest.mark.parametrize("med3x", [False, True])
def test_bf16_scales_beyond_fp16_range(k_gain, v_gain, med3x):
    """bf16 K / V far outside the fp16 range (per-token scales up to ~1e9) or far below its normal range (scales
    down to ~1e-7, whose products with the softmax weights would be fp16 subnormals).  The quantize kernel tracks the
    largest scale; outside [2^-8, 2^15) the cache is marked wide_range and attention takes the layout-generic kernel,
    which carries the K scale in fp32, the softmax weights with a power-of-two offset taken from that bound and the
    verbatim chunks rescaled, so every fp16 matrix product stays finite and normal.  Checked against the CPU oracle
    through the packed and the unpacked entry points, with the tolerance relative to the output's magnitude."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.bfloat16
    B, Hq, Hkv, T, d_h, S, b_r = 2, 8, 2, 300, 128, 96, 4
    k = (kv_input((B, Hkv, T, d_h), torch.float32, 71, outlier_p=0.02 if med3x else 0) * k_gain).to(dt)
    v = (kv_input((B, Hkv, T, d_h), torch.float32, 72) * v_gain).to(dt)
    Q = torch.randn(B, Hq, 1, d_h, generator=torch.Generator().manual_seed(73)).to(dt)
    q = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV)
    w = hqmq.with_outlier_extraction(q, C=3.0) if med3x else q
    cache = w.new_cache(B, T, d_h, dt, 0, **({"sideband_frac": 0.5} if med3x else {}))
    w.append(cache, k.to(DEV), v.to(DEV), 0)
    if v_gain > 1:
        assert float(cache.V.scale.float().max()) > 65504.0                  # beyond fp16
    else:
        assert float(cache.V.scale.float().max()) < 2.0 ** -8                # P * scale would be subnormal in fp16
    vmax = cache.V.scale_max.view(torch.float32)
    assert float(vmax) == float(cache.V.scale[:, :, :T].float().max())       # the quantize kernel tracked the maximum
    assert cache.V.wide_range                                                # read back after the bulk append
    qmax = (1 << b_r) - 1
    dense = {}
    for tag, x, kv in (("K", k, 0), ("V", v, 1)):
        J = CO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, kv], dt)
        r = CO.outlier_quantize(x, J, b_r, 3.0) if med3x else CO.quantize(x, J, b_r, dense=False)
        dense[tag + "_D"] = dense_from_codes(r, J, qmax, x)
        dense[tag + "_x"] = dense_from_codes(r, J, qmax, x, exact=True)
        if tag == "K":
            codes = r
    refs = attention_refs(Q, dense["K_D"], dense["V_D"], dense["K_x"], dense["V_x"])
    scale = float(refs[0].abs().max())
    assert scale > 100.0 if v_gain > 1 else scale < 1e-4
    for generic in (False, True):
        for ns in (1, 3):
            O = hqmq.fused_attention_packed(Q.to(DEV), cache, n_splits=ns, force_generic=generic)
            assert torch.isfinite(O.float()).all(), (generic, ns)
            assert_attention_close(O, *refs, base=2e-3 * scale, what=f"generic={generic} n_splits={ns}")
    if not med3x:      # the reference's unpacked argument list (scales handed over as a tensor)
        cv = CO.quantize(v, CO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, 1], dt), b_r, dense=False)
        Jk = CO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, 0], dt).to(DEV)
        Jv = CO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, 1], dt).to(DEV)
        O = hqmq.fused_attention(Q.to(DEV), codes["idx"].to(DEV), codes["rq"].to(DEV), codes["r_max"].to(DEV), Jk,
                                 cv["idx"].to(DEV), cv["rq"].to(DEV), cv["r_max"].to(DEV), Jv, r_qmax=qmax, causal=False)
        assert torch.isfinite(O.float()).all()
        assert_attention_close(O, *refs, base=2e-3 * scale, what="unpacked")


def test_skip_combine_partials_are_the_callers_own():
    """Two attention calls with skip_combine on one stream: each leaves its partials in a buffer of its own, and
    merging them afterwards gives the fused results."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.float16
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=96, radius_bits=4, device=DEV)
    outs, parts = [], []
    for seed in (1, 2):
        k, v = kv_input((1, 2, 2048, 128), dt, seed).to(DEV), kv_input((1, 2, 2048, 128), dt, seed + 10).to(DEV)
        cache = q.new_cache(1, 2048, 128, dt, 0)
        q.append(cache, k, v, 0)
        Q = torch.randn(1, 8, 1, 128, generator=torch.Generator().manual_seed(seed)).to(dt).to(DEV)
        ref = hqmq.fused_attention_packed(Q, cache, n_splits=4)
        O, ws, ns = ops.attn_fwd(Q, cache.K, cache.V, 2048, n_splits=4, skip_combine=True)
        outs.append((O, ref))
        parts.append((ws, ns))
    assert parts[0][0].data_ptr() != parts[1][0].data_ptr()
    for (O, ref), (ws, ns) in zip(outs, parts):
        assert torch.equal(ops.attn_combine(ws, O, ns), ref)


def test_codebook_cache_follows_the_parameter():
    """The cached joint tables are rebuilt when secondary_raw is replaced, re-pointed (.data = w) or changed in place
    by an op that torch records; after a write through .data, invalidate_codebooks() does it."""
    import hqmq
    dt = torch.float16
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=24, radius_bits=3, device=DEV)
    x = kv_input((1, 2, 64, 64), dt, 5).to(DEV)
    base = q.encode_K(x, 0)["idx"].clone()
    g = torch.Generator().manual_seed(99)

    def fresh():
        return torch.randn(q.secondary_raw.shape, generator=g).to(DEV)

    def oracle_idx():
        J = CO.joint_table(q.secondary_raw.detach().cpu()[0, :, 0], dt)
        return CO.quantize(x.cpu(), J, 3, dense=False)["idx"]

    q.secondary_raw = torch.nn.Parameter(fresh())                  # a new parameter object
    a = q.encode_K(x, 0)["idx"]
    assert not torch.equal(a, base) and torch.equal(a.cpu(), oracle_idx())
    q.secondary_raw.data = fresh()                                 # new storage behind the same parameter
    b = q.encode_K(x, 0)["idx"]
    assert not torch.equal(b, a) and torch.equal(b.cpu(), oracle_idx())
    with torch.no_grad():
        q.secondary_raw.copy_(fresh())                             # an in-place op torch counts
    c = q.encode_K(x, 0)["idx"]
    assert not torch.equal(c, b) and torch.equal(c.cpu(), oracle_idx())
    q.secondary_raw.data.copy_(fresh())                            # invisible to the parameter: say so explicitly
    q.invalidate_codebooks()
    d = q.encode_K(x, 0)["idx"]
    assert not torch.equal(d, c) and torch.equal(d.cpu(), oracle_idx())


@pytest.mark.parametrize("S,b_r", [(200, 3), (213, 6)])
def test_outlier_cache_with_tables_beyond_the_fast_kernels_slot(S, b_r):
    """Codebooks of 4609..5112 codewords fit the plain kernels' LDS slots but not the smaller V slot of the outlier
    variants: such caches take the layout-generic kernel (same results as asking for it explicitly)."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.float16
    B, Hq, Hkv, T, d_h = 2, 8, 2, 200, 128
    k = kv_input((B, Hkv, T, d_h), dt, 81, outlier_p=0.03).to(DEV)
    v = kv_input((B, Hkv, T, d_h), dt, 82, outlier_p=0.03, outlier_gain=(5, 10)).to(DEV)
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV), C=3.0)
    cache = w.new_cache(B, T, d_h, dt, 0, sideband_frac=0.5)
    w.append(cache, k, v, 0)
    cache.K.check_overflow()
    assert 4608 < cache.K.joint.shape[1] <= 5120 and int(cache.K.sb_count.sum()) > 0
    Q = torch.randn(B, Hq, 1, d_h, generator=torch.Generator().manual_seed(83)).to(dt).to(DEV)
    O = hqmq.fused_attention_packed(Q, cache)
    Og = hqmq.fused_attention_packed(Q, cache, force_generic=True)
    assert torch.equal(O, Og)
    Kd = ops.dequant_packed(cache.K, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    Vd = ops.dequant_packed(cache.V, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float(), Kd) * d_h ** -0.5
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, -1), Vd)
    assert (O.float() - ref).abs().max().item() < 2e-3 * max(1.0, float(ref.abs().max()))
    # the plain cache of the same codebook still runs the specialised kernel and agrees with the generic one
    plain = w.inner.new_cache(B, T, d_h, dt, 0)
    w.inner.append(plain, k, v, 0)
    Op, Opg = hqmq.fused_attention_packed(Q, plain), hqmq.fused_attention_packed(Q, plain, force_generic=True)
    assert (Op.float() - Opg.float()).abs().max().item() < 1e-3 * max(1.0, float(Opg.abs().max()))


def test_strict_quantile_limit_mirrors_the_reference(monkeypatch):
    """torch.quantile refuses more than 2^24 elements per row; the Med-C wrapper raises the same error on request
    and otherwise extends the range (the radix select has no such bound)."""
    import hqmq
    from hqmq_amd import ops
    monkeypatch.setattr(ops, "QUANTILE_LIMIT", 1000)              # stand-in for 2^24: 1 x 40 x 32 chunks per head
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=24, radius_bits=3, device=DEV), C=3.0)
    x = kv_input((1, 2, 40, 128), torch.float16, 91).to(DEV)
    w.quantize_K(x, 0)                                             # extension: accepted
    w.strict_quantile_limit = True
    with pytest.raises(RuntimeError, match="quantile\\(\\) input tensor is too large"):
        w.quantize_K(x, 0)
    w.quantize_K(x[:, :, :30], 0)                                  # 960 chunks per head: within the limit


def test_range_flag_follows_decode_appends():
    """A cache of ordinary magnitude stays on the specialised kernels; a later token with a huge scale is noticed at
    the next range check (every RANGE_CHECK_EVERY small appends, or on request) and moves it to the guarded kernel."""
    import hqmq
    dt = torch.bfloat16
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=96, radius_bits=4, device=DEV)
    cache = q.new_cache(1, 512, 128, dt, 0)
    x = kv_input((1, 2, 300, 128), dt, 5).to(DEV)
    q.append(cache, x, x, 0)
    assert not cache.V.wide_range
    Q = torch.randn(1, 8, 1, 128, generator=torch.Generator().manual_seed(6)).to(dt).to(DEV)
    base = hqmq.fused_attention_packed(Q, cache)
    big = (kv_input((1, 2, 1, 128), torch.float32, 7) * 1e7).to(dt).to(DEV)
    cache.V.RANGE_CHECK_EVERY = 3
    for i in range(3):
        q.append(cache, x[:, :, i:i + 1], big if i == 0 else x[:, :, i:i + 1], 0)
    assert cache.V.wide_range and not cache.K.wide_range
    O = hqmq.fused_attention_packed(Q, cache)
    assert torch.isfinite(O.float()).all() and float(O.float().abs().max()) > 10 * float(base.float().abs().max())
    assert torch.equal(O, hqmq.fused_attention_packed(Q, cache, force_generic=True))


def test_range_check_after_every_append_leaves_no_window():
    """RANGE_CHECK_EVERY = 1 (per cache or on the class): the largest scale is read back after every append, so the
    very first attention call after a token whose scale left [2^-8, 2^15) already takes the guarded kernel; with the
    default the same call meets the unguarded kernel until the next check (the documented window)."""
    import hqmq
    dt = torch.bfloat16
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=96, radius_bits=4, device=DEV)
    x = kv_input((1, 2, 300, 128), dt, 5).to(DEV)
    big = (kv_input((1, 2, 1, 128), torch.float32, 7) * 1e7).to(dt).to(DEV)
    Q = torch.randn(1, 8, 1, 128, generator=torch.Generator().manual_seed(6)).to(dt).to(DEV)
    outs = {}
    for every in (1, 256):
        cache = q.new_cache(1, 512, 128, dt, 0)
        cache.K.RANGE_CHECK_EVERY = cache.V.RANGE_CHECK_EVERY = every
        q.append(cache, x, x, 0)
        q.append(cache, x[:, :, :1], big, 0)
        assert cache.V.wide_range == (every == 1)
        outs[every] = hqmq.fused_attention_packed(Q, cache)
    assert torch.isfinite(outs[1].float()).all()
    cache.V.refresh_range()                         # the check the default would have run later
    assert cache.V.wide_range and torch.equal(hqmq.fused_attention_packed(Q, cache), outs[1])


def test_outlier_kernels_with_huge_k_and_ordinary_v_stay_on_the_fast_path():
    """bf16 K of magnitude 1e3 whose outlier chunks (x 50-200) lie beyond the fp16 range, with ordinary V: only V's
    scales decide the routing (P * V scale is what must stay inside fp16), so the cache stays on the specialised outlier
    kernels, whose K side keeps the scales in fp32 and feeds the verbatim bf16 chunks to bf16 matrix products (the
    layout-generic kernel scales them down by the bound of the K scales): finite and within the two-reference bound.
    (Q is of magnitude 1e-3, so that the scores are of order one: queries are converted to fp16 by both kernels.)"""
    import hqmq
    from tests.helpers import masked_two_refs
    dt = torch.bfloat16
    B, H, T, d_h = 2, 2, 700, 128
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=24, radius_bits=3, device=DEV), C=3.0)
    k = (kv_input((B, H, T, d_h), torch.float32, 31, outlier_p=0.02) * 1e3).to(dt).to(DEV)
    v = kv_input((B, H, T, d_h), dt, 32, outlier_p=0.02, outlier_gain=(5, 10)).to(DEV)
    cache = w.new_cache(B, T, d_h, dt, 0, sideband_frac=0.25)
    w.append(cache, k, v, 0)
    cache.K.check_overflow()
    assert not cache.V.wide_range
    assert float(k.float().abs().max()) > 65504.0
    Q = (torch.randn(B, 8, 1, d_h, generator=torch.Generator().manual_seed(33)) * 1e-3).to(dt).to(DEV)
    refs = masked_two_refs(cache, Q, T)
    for generic in (False, True):
        O = hqmq.fused_attention_packed(Q, cache, force_generic=generic)
        assert torch.isfinite(O.float()).all()
        assert_attention_close(O, *refs, base=2e-3 * max(1.0, float(refs[0].abs().max())), what=f"generic={generic}")
