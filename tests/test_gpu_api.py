"""The reference's GPU smoke tests (tests/test_gpu.py there), run against this build's package."""
import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a GPU")]
DEV = "cuda"


def test_quantize_on_gpu():
    import hqmq
    q = hqmq.HQMQ(n_layers=2, n_heads=2, secondary_size=24, radius_bits=3, device="cuda", init="random")
    K = torch.randn(1, 2, 16, 128, dtype=torch.bfloat16, device="cuda")
    Kq = q.quantize_K(K, layer_idx=0)
    assert Kq.shape == K.shape and Kq.device == K.device and Kq.dtype == K.dtype
    diff = (K.float() - Kq.float()).abs().mean().item()
    corr = torch.corrcoef(torch.stack([K.float().flatten(), Kq.float().flatten()]))[0, 1].item()
    assert diff > 1e-4 and corr > 0.7          # the reference's round-trip sanity bounds (tests/test_smoke.py:178-192)


def test_fp32_round_trip_shapes():
    import hqmq
    q = hqmq.HQMQ(n_layers=2, n_heads=2, secondary_size=24, radius_bits=3, device="cuda")
    K = torch.randn(1, 2, 16, 128, dtype=torch.float32, device="cuda")
    Kq = q.quantize_K(K, layer_idx=0)
    assert Kq.shape == K.shape and Kq.dtype == K.dtype


def test_padded_quantizer_on_gpu():
    import hqmq
    p = hqmq.PaddedHQMQ(n_layers=1, n_heads=2, d_head=45, secondary_size=24, radius_bits=3, device="cuda")
    x = torch.randn(1, 2, 9, 45, device="cuda", dtype=torch.float16)
    y = p.quantize_K(x, 0)
    assert y.shape == x.shape
    padded = torch.nn.functional.pad(x, (0, 3))
    assert torch.equal(y, p.inner.quantize_K(padded, 0)[..., :45])


def test_device_info_reports_real_gpu():
    import hqmq
    info = hqmq.device_info()
    assert info["gpu"] is not None and info["variant_auto_dispatched"] == "cdna4"
    assert info["arch"].startswith("gfx950")


def test_fp8_codebook_option():
    """use_fp8_codebook=True is the reference's Hopper behaviour: the joint tables rounded to float8_e4m3fn, fp16
    arithmetic.  It equals the plain call on the rounded tables bit for bit, dense attention over a cache decoded
    with them within the usual bound, and it is the default of the hopper / blackwell names."""
    import hqmq
    from hqmq import kernels
    from hqmq_amd import ops
    B, H_q, H_kv, T, dh, S, r_qmax = 1, 4, 1, 32, 32, 24, 7
    torch.manual_seed(0)
    Q = torch.randn(B, H_q, T, dh, dtype=torch.float16, device="cuda") * 0.3
    idx = torch.randint(0, 24 * S, (B, H_kv, T, dh // 4), dtype=torch.int32, device="cuda")
    rq = torch.randint(1, r_qmax + 1, (B, H_kv, T, dh // 4), dtype=torch.int32, device="cuda")
    rs = torch.rand((B, H_kv, T), dtype=torch.float16, device="cuda") + 0.5
    joint = torch.randn((H_kv, 24 * S, 4), dtype=torch.float16, device="cuda")
    joint = joint / joint.norm(dim=-1, keepdim=True).clamp(min=1e-6)
    j8 = kernels.encode_joint_fp8(joint).to(torch.float16)
    assert not torch.equal(j8, joint)
    a = hqmq.fused_attention(Q, idx, rq, rs, joint, idx, rq, rs, joint, r_qmax=r_qmax, causal=True)
    b = hqmq.fused_attention(Q, idx, rq, rs, joint, idx, rq, rs, joint, r_qmax=r_qmax, causal=True, use_fp8_codebook=True)
    on_rounded = hqmq.fused_attention(Q, idx, rq, rs, j8, idx, rq, rs, j8, r_qmax=r_qmax, causal=True)
    assert torch.equal(b, on_rounded) and not torch.equal(a, b)
    ref = hqmq.fused_attention_reference(Q, idx, rq, rs, j8, idx, rq, rs, j8, r_qmax=r_qmax, causal=True)
    assert (b.float() - ref.float()).abs().max().item() < 2e-3
    c = kernels.fused_attention_hopper(Q, idx, rq, rs, joint, idx, rq, rs, joint, r_qmax=r_qmax, causal=True)
    d = kernels.fused_attention_blackwell(Q, idx, rq, rs, joint, idx, rq, rs, joint, r_qmax=r_qmax, causal=True,
                                          use_fp8_codebook=False)
    assert torch.equal(b, c) and torch.equal(a, d)
    # the packed path: same option, per cache
    q = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=96, radius_bits=4, device=DEV), C=3.0)
    g = torch.Generator().manual_seed(5)
    k, v = torch.randn(2, 2, 100, 128, generator=g).half().to(DEV), torch.randn(2, 2, 100, 128, generator=g).half().to(DEV)
    k[:, :, ::9, 8:12] *= 30.0
    cache = q.new_cache(2, 100, 128, torch.float16, 0)
    q.append(cache, k, v, 0)
    Qp = torch.randn(2, 8, 1, 128, generator=g).half().to(DEV)
    table_before = cache.K.joint.clone()
    O8 = hqmq.fused_attention_packed(Qp, cache, use_fp8_codebook=True)
    O16 = hqmq.fused_attention_packed(Qp, cache)
    from hqmq_amd.packed import PackedKV
    view = PackedKV(cache.K.with_fp8_table(), cache.V.with_fp8_table())
    Kd = ops.dequant_packed(view.K, 100, 0).float().repeat_interleave(4, 1)
    Vd = ops.dequant_packed(view.V, 100, 0).float().repeat_interleave(4, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", Qp.float(), Kd) * 128 ** -0.5
    refp = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, -1), Vd)
    assert (O8.float() - refp).abs().max().item() < 2e-3 * max(1.0, float(refp.abs().max()))
    assert not torch.equal(O8, O16) and torch.equal(cache.K.joint, table_before)      # the cache keeps its own table


def test_encode_joint_fp8():
    from hqmq.kernels import encode_joint_fp8
    joint = torch.randn(2, 24 * 24, 4, dtype=torch.float16, device="cuda")
    joint = joint / joint.norm(dim=-1, keepdim=True).clamp(min=1e-6)
    j8 = encode_joint_fp8(joint)
    assert j8.dtype == torch.float8_e4m3fn and j8.shape == joint.shape


def test_native_library_is_what_ran():
    """The kernels come from the in-tree shared library, loaded into this process."""
    from hqmq_amd import _lib as L
    so = str(L.library_path())
    with open("/proc/self/maps") as f:
        assert any(so in line for line in f)


@pytest.mark.parametrize("d_head,S,b_r", [(80, 96, 4), (70, 24, 3), (160, 24, 4), (100, 96, 4)])
def test_padded_quantizer_packed_path(d_head, S, b_r):
    """PaddedHQMQ on the packed path: heads that are no multiple of 4 (or no size the attention kernels take) are
    zero-padded into the planes; the planes decode to the fake-quant tensor bit for bit and fused attention equals
    dense attention over it."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.float16
    B, Hq, Hkv, T = 2, 8, 2, 200
    q = hqmq.PaddedHQMQ(n_layers=1, n_heads=Hkv, d_head=d_head, secondary_size=S, radius_bits=b_r, device=DEV)
    g = torch.Generator().manual_seed(d_head)
    k, v = torch.randn(B, Hkv, T, d_head, generator=g).to(dt).to(DEV), torch.randn(B, Hkv, T, d_head, generator=g).to(dt).to(DEV)
    cache = q.new_cache(B, T, dt, 0)
    q.append(cache, k[:, :, :150], v[:, :, :150], 0)
    q.append(cache, k[:, :, 150:], v[:, :, 150:], 0)
    assert cache.K.d_head == q.d_head_stored >= d_head
    kq, vq = q.quantize_K(k, 0), q.quantize_V(v, 0)
    dk = ops.dequant_packed(cache.K, T, mode=1)
    assert torch.equal(dk[..., :d_head].contiguous().view(torch.int16), kq.contiguous().view(torch.int16))
    assert int(dk[..., q.d_head_padded:].abs().sum()) == 0          # whole padding chunks decode to exactly zero
    Q = torch.randn(B, Hq, 1, d_head, generator=g).to(dt).to(DEV)
    O = hqmq.fused_attention_packed(Q, cache)
    Kd = ops.dequant_packed(cache.K, T, 0)[..., :d_head].float().repeat_interleave(Hq // Hkv, 1)
    Vd = ops.dequant_packed(cache.V, T, 0)[..., :d_head].float().repeat_interleave(Hq // Hkv, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float(), Kd) * d_head ** -0.5
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, -1), Vd)
    assert O.shape == Q.shape and (O.float() - ref).abs().max().item() < 2e-3


@pytest.mark.parametrize("S,b_r,dn,outl", [(96, 4, "fp16", False), (192, 6, "fp16", True), (192, 6, "bf16", False), (96, 4, "bf16", True)])
def test_fp8_table_storage_gives_the_same_result(S, b_r, dn, outl):
    """use_fp8_codebook rounds the joint tables to e4m3; fp8_table_storage additionally keeps them as float8 in LDS
    (the reference's Hopper path stores fp8 and promotes after the gather, hqmq_attention_hopper.py:43-53,133-135).
    Every e4m3 number is exact in fp16, so the two storages must agree bit for bit."""
    import hqmq
    dt = torch.float16 if dn == "fp16" else torch.bfloat16
    B, Hq, Hkv, T, d_h = 2, 8, 2, 1500, 128
    g = torch.Generator().manual_seed(S)
    k, v = torch.randn(B, Hkv, T, d_h, generator=g), torch.randn(B, Hkv, T, d_h, generator=g)
    if outl:
        k[:, :, ::7, 8:12] *= 30.0
        v[:, :, ::5, 64:68] *= 20.0
    q = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV)
    w = hqmq.with_outlier_extraction(q, C=3.0) if outl else q
    cache = w.new_cache(B, T, d_h, dt, 0, **({"sideband_frac": 0.25} if outl else {}))
    w.append(cache, k.to(dt).to(DEV), v.to(dt).to(DEV), 0)
    Q = torch.randn(B, Hq, 1, d_h, generator=g).to(dt).to(DEV)
    plain = hqmq.fused_attention_packed(Q, cache)
    for ns in (0, 1, 3):
        a = hqmq.fused_attention_packed(Q, cache, use_fp8_codebook=True, n_splits=ns)
        b = hqmq.fused_attention_packed(Q, cache, use_fp8_codebook=True, fp8_table_storage=True, n_splits=ns)
        assert torch.equal(a, b), ns
        assert not torch.equal(a, plain)
    with pytest.raises(hqmq.HqmqError):
        hqmq.fused_attention_packed(Q, cache, fp8_table_storage=True)
