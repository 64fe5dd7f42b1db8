"""GPU parity for the fused attention kernel: golden outputs of the reference's torch path, dense attention
over the dequantized cache (CPU oracle, double accumulation), and size-independent properties at full size.

Tolerance: 2e-3 max abs (1e-3 for fp32 caches, the reference's own test bound) wherever the softmax is diffuse
(every long-context decode shape).  Short or outlier-dominated cases, whose outputs are O(1..30), are held to the
bound of tests/helpers.py:assert_attention_close, which adds the fp16 product noise and the reference's own
rounding spread.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle as CO
from oracle import torch_oracle as TO
from tests.helpers import (DT, assert_attention_close, attention_refs, attn_tolerance, bit_equal, dense_from_codes,
                           exact_dense, gpu_attention_refs, kv_input, masked_two_refs, unbits, unpack_planes)
from tests.test_oracle import ATTN_CASES, load_attn_case

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a GPU")]
DEV = "cuda"


def assert_close(got, ref, dtype, base=2e-3, what=""):
    ref = ref.float().cpu()
    err = (got.float().cpu() - ref).abs()
    tol = attn_tolerance(ref, dtype, base)
    worst = float((err - tol).max())
    assert worst <= 0, f"{what}: max abs err {float(err.max()):.3e}, exceeds tolerance by {worst:.3e}"


@pytest.mark.parametrize("case", ATTN_CASES)
def test_golden_unpacked_api(case, golden_dir):
    """hqmq.fused_attention with the reference's argument list against the reference's own torch output."""
    import hqmq
    m, t = load_attn_case(np.load(golden_dir / "attention.npz"), case)
    d = {k: v.to(DEV) for k, v in t.items()}
    base = 1e-3 if m["dtype"] == torch.float32 else 2e-3
    for kw in (dict(), dict(n_splits=1), dict(n_splits=3), dict(block_q=64, block_kv=64, num_warps=4, num_stages=2,
                                                               optimized=False)):
        O = hqmq.fused_attention(d["Q"], d["K_idx"], d["K_rq"], d["K_rs"], d["K_joint"], d["V_idx"], d["V_rq"],
                                 d["V_rs"], d["V_joint"], r_qmax=m["qmax"], causal=m["causal"], **kw)
        assert O.shape == d["Q"].shape and O.dtype == d["Q"].dtype
        assert_close(O, t["O"], m["dtype"], base, f"{case} {kw}")
    Oref = hqmq.fused_attention_reference(d["Q"], d["K_idx"], d["K_rq"], d["K_rs"], d["K_joint"], d["V_idx"], d["V_rq"],
                                          d["V_rs"], d["V_joint"], r_qmax=m["qmax"], causal=m["causal"])
    assert_close(Oref, t["O"], m["dtype"], base, f"{case} unfused")


def test_reference_gpu_test_recipe():
    """The reference's only numerical kernel test (tests/test_gpu.py:24-49): fp32, causal, max abs diff < 1e-3."""
    import hqmq
    B, H_q, H_kv, T, dh, S, r_qmax = 1, 4, 1, 64, 32, 24, 7
    K_size = 24 * S
    torch.manual_seed(0)
    Q = torch.randn(B, H_q, T, dh, dtype=torch.float32, device=DEV) * 0.3
    idx = torch.randint(0, K_size, (B, H_kv, T, dh // 4), dtype=torch.int32, device=DEV)
    rq = torch.randint(1, r_qmax + 1, (B, H_kv, T, dh // 4), dtype=torch.int32, device=DEV)
    rs = torch.rand((B, H_kv, T), dtype=torch.float32, device=DEV) + 0.5
    joint = torch.randn((H_kv, K_size, 4), dtype=torch.float32, device=DEV)
    joint = joint / joint.norm(dim=-1, keepdim=True).clamp(min=1e-6)
    O_ref = hqmq.fused_attention_reference(Q, idx, rq, rs, joint, idx, rq, rs, joint, r_qmax=r_qmax, causal=True)
    O_fused = hqmq.fused_attention(Q, idx, rq, rs, joint, idx, rq, rs, joint, r_qmax=r_qmax, causal=True)
    assert (O_ref - O_fused).abs().max().item() < 1e-3
    cpu = CO.attention_dense(Q.cpu(), CO.dequant(idx.cpu(), rq.cpu(), rs.cpu(), joint.cpu(), r_qmax),
                             CO.dequant(idx.cpu(), rq.cpu(), rs.cpu(), joint.cpu(), r_qmax), causal=True)
    assert (cpu - O_fused.cpu()).abs().max().item() < 1e-3


def build_cache(q, k, v, outliers):
    cache = q.new_cache(k.shape[0], k.shape[2], k.shape[3], k.dtype, 0)
    q.append(cache, k.to(DEV), v.to(DEV), 0)
    if outliers:
        cache.K.check_overflow()
        cache.V.check_overflow()
    return cache


CASES = [
    # name, B, H_q, H_kv, T_q, T_kv, d_h, S, b_r, dtype, outliers, causal, causal_offset, kv_lens
    ("config2 shape, fp16 s96_r4", 1, 32, 8, 1, 1000, 128, 96, 4, "fp16", False, False, 0, None),
    ("config3 shape, fp16 s192_r6 + Med3x", 2, 28, 4, 1, 300, 128, 192, 6, "fp16", True, False, 0, None),
    ("config4 shape, bf16 s24_r3 + Med3x, ragged", 3, 32, 8, 1, 400, 128, 24, 3, "bf16", True, False, 0, [400, 130, 257]),
    ("config5 shape, bf16 s96_r4 + Med3x, d_h=64", 2, 64, 8, 1, 777, 64, 96, 4, "bf16", True, False, 0, None),
    ("square causal prefill", 1, 8, 2, 100, 100, 128, 96, 4, "fp16", False, True, 0, None),
    ("rectangular causal, top-left aligned", 1, 4, 2, 5, 190, 64, 24, 3, "fp16", False, True, 0, None),
    ("chunked prefill, bottom-right aligned", 2, 8, 4, 7, 133, 128, 96, 4, "fp16", False, True, 126, None),
    ("fp32 cache", 2, 4, 2, 3, 90, 32, 96, 4, "fp32", False, False, 0, None),
    ("d_h=256", 1, 4, 2, 1, 200, 256, 96, 4, "fp16", False, False, 0, None),
    ("empty and short sequences", 3, 8, 2, 1, 64, 64, 24, 3, "fp16", False, False, 0, [0, 1, 64]),
    # s192 with four radius bits (the codec of the reference's published prefill figure): 16 + 1 bit layout
    ("s192_r4 decode, 16+1 bits", 1, 32, 8, 1, 500, 128, 192, 4, "fp16", False, False, 0, None),
    ("s192_r4 square causal prefill, two column groups", 1, 32, 8, 160, 160, 128, 192, 4, "fp16", False, True, 0, None),
    ("s192_r4 + Med3x bf16 decode", 2, 8, 4, 1, 333, 128, 192, 4, "bf16", True, False, 0, None),
    # the other widths of the layout rule at d_h 128
    ("s96_r6 decode, 16+2 bits", 1, 32, 8, 1, 500, 128, 96, 6, "fp16", False, False, 0, None),
    ("s192_r5 + Med3x prefill chunk, 16+2 bits", 1, 8, 2, 40, 300, 128, 192, 5, "bf16", True, True, 260, None),
    ("s24_r4 decode ragged, 12+2 bits", 3, 8, 4, 1, 400, 128, 24, 4, "bf16", False, False, 0, [400, 77, 256]),
    ("s24_r4 + Med3x decode, 12+2 bits", 2, 8, 4, 1, 200, 128, 24, 4, "fp16", True, False, 0, None),
    ("s96_r3 decode, 12+3 bits", 1, 32, 8, 1, 500, 128, 96, 3, "fp16", False, False, 0, None),
    ("s24_r5 square causal prefill, 12+3 bits, two column groups", 1, 32, 8, 160, 160, 128, 24, 5, "fp16", False, True, 0, None),
    # head counts around the rotation of the KV heads from sequence to sequence (a block's head is not its index
    # in the grid: (index + sequence slot) mod H_kv, with 8 / H_kv sequences sharing a rotation below eight heads)
    ("nine sequences, one KV head", 9, 4, 1, 1, 96, 128, 96, 4, "fp16", False, False, 0, None),
    ("six ragged sequences, two KV heads + Med3x", 6, 4, 2, 1, 150, 128, 24, 3, "bf16", True, False, 0, [150, 7, 64, 33, 150, 99]),
    ("five sequences, three KV heads", 5, 6, 3, 1, 120, 64, 96, 4, "fp16", False, False, 0, None),
    ("two sequences, sixteen KV heads", 2, 16, 16, 1, 100, 128, 96, 4, "fp16", False, False, 0, None),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_attention_matches_dense_oracle(case):
    import hqmq
    from hqmq_amd import ops
    name, B, Hq, Hkv, Tq, Tkv, d_h, S, b_r, dn, outl, causal, off, lens = case
    dt = DT[dn]
    seed = sum(map(ord, name))
    k = kv_input((B, Hkv, Tkv, d_h), dt, seed, lognormal=False, outlier_p=0.02 if outl else 0)
    v = kv_input((B, Hkv, Tkv, d_h), dt, seed + 1, lognormal=False, outlier_p=0.02 if outl else 0, outlier_gain=(5, 10))
    Q = torch.randn(B, Hq, Tq, d_h, generator=torch.Generator().manual_seed(seed + 2)).to(dt)
    q = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV)
    if outl:
        q = hqmq.with_outlier_extraction(q, C=3.0)
    cache = build_cache(q, k, v, outl)
    qmax = (1 << b_r) - 1
    dense = {}
    for tag, x, kv, pt in (("K", k, 0, cache.K), ("V", v, 1, cache.V)):
        J = CO.joint_table(TO.secondary_raw(1, Hkv, S, 42)[0, :, kv], dt)
        r = CO.outlier_quantize(x, J, b_r, 3.0) if outl else CO.quantize(x, J, b_r, dense=False)
        dense[tag + "_D"] = dense_from_codes(r, J, qmax, x)
        dense[tag + "_x"] = dense_from_codes(r, J, qmax, x, exact=True)
        assert bit_equal(ops.dequant_packed(pt, Tkv, 0), dense[tag + "_D"])      # the cache holds the oracle's codes
    refs = attention_refs(Q, dense["K_D"], dense["V_D"], dense["K_x"], dense["V_x"], kv_lens=lens, causal=causal,
                          causal_offset=off)
    base = 1e-3 if dt == torch.float32 else 2e-3
    outs = []
    for ns in (1, 2, 0):
        O = hqmq.fused_attention_packed(Q.to(DEV), cache, causal=causal, causal_offset=off, n_splits=ns, T_kv=Tkv,
                                        kv_lens=None if lens is None else torch.tensor(lens))
        worst = assert_attention_close(O, *refs, base=base, what=f"{name} n_splits={ns}")
        if not outl:
            assert worst < 2 * base + 4 * 2.0 ** -11 * float(refs[0].abs().max())   # plain bound, no spread allowance
        outs.append(O)
    if lens is not None and 0 in lens:
        assert float(outs[0][lens.index(0)].abs().max()) == 0.0      # nothing to attend to -> zeros, not NaN


def test_torch_sdpa_agrees_on_the_same_cache():
    """Dense SDPA on the GPU over the dequantized cache (the check benchmark config 2 asks for)."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.float16
    q = hqmq.HQMQ(n_layers=1, n_heads=8, secondary_size=96, radius_bits=4, device=DEV)
    k, v = kv_input((1, 8, 4096, 128), dt, 1, lognormal=False), kv_input((1, 8, 4096, 128), dt, 2, lognormal=False)
    cache = build_cache(q, k, v, False)
    Q = torch.randn(1, 32, 1, 128, generator=torch.Generator().manual_seed(3)).to(dt).to(DEV)
    Kd, Vd = ops.dequant_packed(cache.K, 4096, 0), ops.dequant_packed(cache.V, 4096, 0)
    ref = torch.nn.functional.scaled_dot_product_attention(Q, Kd.repeat_interleave(4, 1), Vd.repeat_interleave(4, 1))
    O = hqmq.fused_attention_packed(Q, cache)
    assert (O.float() - ref.float()).abs().max().item() < 2e-3


@pytest.mark.parametrize("T", [4096, 8192, 16384, 32768])
def test_config2_full_size_properties(T):
    """Benchmark config 2 at full size (32 / 8 heads, d_h=128, s96_r4, fp16, one query token):
    split invariance, zero padding rows ignored, agreement with dense fp32 attention on the GPU, 2e-3 bound."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.float16
    q = hqmq.HQMQ(n_layers=1, n_heads=8, secondary_size=96, radius_bits=4, device=DEV)
    g = torch.Generator().manual_seed(T)
    k, v = torch.randn(1, 8, T, 128, generator=g).to(dt), torch.randn(1, 8, T, 128, generator=g).to(dt)
    Q = torch.randn(1, 32, 1, 128, generator=g).to(dt).to(DEV)
    cache = build_cache(q, k, v, False)
    outs = [hqmq.fused_attention_packed(Q, cache, n_splits=ns) for ns in (0, 1, 7, 64)]
    for o in outs[1:]:
        assert (o.float() - outs[0].float()).abs().max().item() < 2e-4       # split-KV merge is exact up to fp32 order
    Kd, Vd = ops.dequant_packed(cache.K, T, 0).float(), ops.dequant_packed(cache.V, T, 0).float()
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float().view(1, 8, 4, 128), Kd) * 128 ** -0.5
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, dim=-1), Vd).reshape(1, 32, 1, 128)
    assert (outs[0].float() - ref).abs().max().item() < 2e-3
    # a sequence-length argument shorter than the cache behaves like a shorter cache
    half = hqmq.fused_attention_packed(Q, cache, kv_lens=torch.tensor([T // 2]), T_kv=T)
    s2 = s[..., :T // 2]
    ref2 = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s2, dim=-1), Vd[:, :, :T // 2]).reshape(1, 32, 1, 128)
    assert (half.float() - ref2).abs().max().item() < 2e-3


def test_decode_loop_with_append_config4_shape():
    """Config 4 shape in miniature: ragged batch, each step quantize-and-appends one bf16 token per sequence
    (s24_r3, Med3x) and attends with per-sequence lengths; compared with the oracle after the last step."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.bfloat16
    B, Hq, Hkv, d_h, steps = 4, 32, 8, 128, 3
    lens0 = [100, 17, 64, 1]
    Tmax = max(lens0) + steps
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=24, radius_bits=3, device=DEV))
    cache = w.new_cache(B, Tmax, d_h, dt, 0, sideband_frac=0.25)
    k_all = kv_input((B, Hkv, Tmax, d_h), dt, 21, outlier_p=0.02)
    v_all = kv_input((B, Hkv, Tmax, d_h), dt, 22)
    pos = torch.tensor(lens0, dtype=torch.int32, device=DEV)
    # prefill each sequence separately (its own Med3x statistics), then step together
    ref_k = torch.zeros(B, Hkv, Tmax, d_h, dtype=dt)
    ref_v = torch.zeros(B, Hkv, Tmax, d_h, dtype=dt)
    ref_kx, ref_vx = ref_k.float(), ref_v.float()       # the same caches without rounding to bf16
    Jk = CO.joint_table(TO.secondary_raw(1, Hkv, 24, 42)[0, :, 0], dt)
    Jv = CO.joint_table(TO.secondary_raw(1, Hkv, 24, 42)[0, :, 1], dt)

    def oracle_dense(x, J):
        r = CO.outlier_quantize(x, J, 3, 3.0)
        return dense_from_codes(r, J, 7, x), dense_from_codes(r, J, 7, x, exact=True)

    for b, L0 in enumerate(lens0):
        sub = w.new_cache(1, Tmax, d_h, dt, 0, sideband_frac=0.25)
        w.append(sub, k_all[b:b + 1, :, :L0].to(DEV), v_all[b:b + 1, :, :L0].to(DEV), 0)
        for dst, src in ((cache.K, sub.K), (cache.V, sub.V)):
            for name in ("main", "aux", "scale", "flags", "sideband", "sb_tile_off", "sb_count", "sb_coord"):
                getattr(dst, name)[b] = getattr(src, name)[0]
        dk, dv = oracle_dense(k_all[b:b + 1, :, :L0].contiguous(), Jk), oracle_dense(v_all[b:b + 1, :, :L0].contiguous(), Jv)
        ref_k[b, :, :L0], ref_kx[b, :, :L0] = dk[0][0], dk[1][0]
        ref_v[b, :, :L0], ref_vx[b, :, :L0] = dv[0][0], dv[1][0]
    for s in range(steps):
        idx = (pos.cpu().long()).tolist()
        k_new = torch.stack([k_all[b, :, idx[b]:idx[b] + 1] for b in range(B)])
        v_new = torch.stack([v_all[b, :, idx[b]:idx[b] + 1] for b in range(B)])
        w.append(cache, k_new.to(DEV), v_new.to(DEV), 0, pos=pos)
        dk, dv = oracle_dense(k_new.contiguous(), Jk), oracle_dense(v_new.contiguous(), Jv)
        for b in range(B):
            ref_k[b, :, idx[b]], ref_kx[b, :, idx[b]] = dk[0][b, :, 0], dk[1][b, :, 0]
            ref_v[b, :, idx[b]], ref_vx[b, :, idx[b]] = dv[0][b, :, 0], dv[1][b, :, 0]
        pos += 1
        Q = torch.randn(B, Hq, 1, d_h, generator=torch.Generator().manual_seed(30 + s)).to(dt)
        O = hqmq.fused_attention_packed(Q.to(DEV), cache, kv_lens=pos, T_kv=Tmax)
        refs = attention_refs(Q, ref_k, ref_v, ref_kx, ref_vx, kv_lens=pos.cpu().tolist())
        assert_attention_close(O, *refs, base=2e-3, what=f"step {s}")
    cache.K.check_overflow()
    dense = ops.dequant_packed(cache.K, Tmax, 0).cpu()
    for b, L in enumerate(pos.cpu().tolist()):
        assert bit_equal(dense[b, :, :L], ref_k[b, :, :L])


def test_argument_checks():
    import hqmq
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=24, radius_bits=3, device=DEV)
    cache = q.new_cache(1, 64, 64, torch.float16, 0)
    x = torch.randn(1, 2, 64, 64, device=DEV).half()
    q.append(cache, x, x, 0)
    with pytest.raises(AssertionError):
        hqmq.fused_attention_packed(torch.randn(1, 3, 1, 64, device=DEV).half(), cache)       # H_q % H_kv
    with pytest.raises(AssertionError):
        hqmq.fused_attention_packed(torch.randn(1, 4, 1, 32, device=DEV).half(), cache)       # d_h mismatch
    with pytest.raises(hqmq.HqmqError):
        hqmq.fused_attention_packed(torch.randn(1, 4, 1, 64, device=DEV), cache)              # dtype mismatch
    with pytest.raises(hqmq.HqmqError):
        q.append(cache, x, x, 0)                                                              # capacity exceeded


def _two_reference_check(O, Q, cache, xs, lens, what):
    """Every sequence of a decode batch against two fp32 references computed on the GPU from the cache's own codes
    (read by tests/helpers.py:unpack_planes, not by the library): attention over the cache decoded with the
    reference's roundings to the cache dtype (hqmq_attention.py:61-64 of the reference, via dequant_packed) and over
    the unrounded product.  Bound: tests/helpers.py:assert_attention_close, i.e.
      |O - exact| <= 2e-3 + 8 * 2^-11 * sum_t p_t |V_t|                (fp16 products, fp32 accumulation)
      |O - ref_D| <= the same + |ref_D - exact|                        (the reference's own rounding spread).
    Returns the maxima (|O - exact|, |O - ref_D|, |ref_D - exact|, max |ref_D|)."""
    from hqmq_amd import ops
    B = Q.shape[0]
    T = int(max(lens))
    Kd_all, Vd_all = ops.dequant_packed(cache.K, T, 0), ops.dequant_packed(cache.V, T, 0)
    worst = [0.0, 0.0, 0.0, 0.0]
    for b in range(B):
        L = int(lens[b])
        kx, vx = xs(b, L)
        K_x, V_x = exact_dense(cache.K, b, L, kx), exact_dense(cache.V, b, L, vx)
        K_D, V_D = Kd_all[b, :, :L].float(), Vd_all[b, :, :L].float()
        # the library's dense decode and the independent reader agree up to the roundings to the cache dtype
        eps = 2.0 ** -8 if cache.K.dtype == torch.bfloat16 else 2.0 ** -11
        assert float(((K_D - K_x).abs() - 3.1 * eps * K_x.abs()).max()) <= 1e-6, f"{what}: K decode of sequence {b}"
        ref_d, ref_x, a_abs = gpu_attention_refs(Q[b, :, 0], K_D, V_D, K_x, V_x)
        assert_attention_close(O[b, :, 0], ref_d.cpu(), ref_x.cpu(), a_abs.cpu(), base=2e-3, what=f"{what} sequence {b} (L={L})")
        got = O[b, :, 0].float()
        for i, v in enumerate(((got - ref_x).abs().max(), (got - ref_d).abs().max(), (ref_d - ref_x).abs().max(), ref_d.abs().max())):
            worst[i] = max(worst[i], float(v))
    print(f"\n{what}: max |O - exact| {worst[0]:.3e}, max |O - ref_D| {worst[1]:.3e}, reference rounding spread "
          f"max |ref_D - exact| {worst[2]:.3e}, max |ref_D| {worst[3]:.3e}")
    return worst


def test_config4_full_size_properties():
    """Benchmark config 4 at full size: 32 / 8 heads, d_h 128, batch 64, per-sequence contexts U{1024..16384} (seeded),
    bf16 activations with lognormal channel scales, s24_r3 + Med3x.  Bulk append, crop to the contexts, one decode
    step (quantize-and-append of one token per sequence at pos, then attention with kv_lens), checked per sequence
    against both fp32 references; the batch order and the split count must not change the result."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.bfloat16
    B, Hq, Hkv, d = 64, 32, 8, 128
    lens = torch.randint(1024, 16385, (B,), generator=torch.Generator().manual_seed(4)).to(torch.int32)
    T = int(lens.max()) + 64
    k = torch.empty(B, Hkv, T, d, dtype=dt, device=DEV)
    v = torch.empty(B, Hkv, T, d, dtype=dt, device=DEV)
    g = torch.Generator().manual_seed(44)
    ck, cv = torch.exp(0.5 * torch.randn(1, Hkv, 1, d, generator=g)), torch.exp(0.5 * torch.randn(1, Hkv, 1, d, generator=g))
    for b in range(B):                                          # CPU-seeded, one sequence at a time
        k[b] = (torch.randn(Hkv, T, d, generator=g) * ck[0]).to(dt).to(DEV)
        v[b] = (torch.randn(Hkv, T, d, generator=g) * cv[0]).to(dt).to(DEV)
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=24, radius_bits=3, device=DEV), C=3.0)
    cache = w.new_cache(B, T, d, dt, 0, sideband_frac=0.125)
    w.append(cache, k, v, 0)
    cache.K.check_overflow()
    cache.V.check_overflow()
    lens_dev = lens.to(DEV)
    cache.crop_(lens_dev)
    # the decode step: one new token per sequence, appended at its own position (its own Med3x statistics: one call)
    k1 = (torch.randn(B, Hkv, 1, d, generator=g) * ck).to(dt).to(DEV)
    v1 = (torch.randn(B, Hkv, 1, d, generator=g) * cv).to(dt).to(DEV)
    pos = lens_dev.clone()
    w.append(cache, k1, v1, 0, pos=pos)
    pos += 1
    cache.K.check_overflow()
    cache.V.check_overflow()
    Q = torch.randn(B, Hq, 1, d, generator=g).to(dt).to(DEV)
    order = ops.longest_first(pos)
    O = hqmq.fused_attention_packed(Q, cache, kv_lens=pos, T_kv=T, batch_order=order)
    rate = float(cache.K.sb_count.sum()) / (Hkv * float(pos.sum()) * d / 4)
    assert 0.002 < rate < 0.05, rate

    def xs(b, L):       # what was quantized into rows [0, L) of sequence b: the bulk rows, then the appended token
        return (torch.cat([k[b, :, :L - 1], k1[b]], dim=1), torch.cat([v[b, :, :L - 1], v1[b]], dim=1))
    worst = _two_reference_check(O, Q, cache, xs, pos.cpu().tolist(), "config 4 at full size")
    assert worst[3] > 0.3                                       # outputs are O(1): the bound is not vacuous
    # scheduling and splitting do not change the result beyond the merge's fp32 rounding
    O2 = hqmq.fused_attention_packed(Q, cache, kv_lens=pos, T_kv=T)
    assert torch.equal(O2, O)
    O3 = hqmq.fused_attention_packed(Q, cache, kv_lens=pos, T_kv=T, n_splits=5, batch_order=order)
    assert (O3.float() - O.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, worst[3])     # one bf16 ulp of the output
    Og = hqmq.fused_attention_packed(Q[:4], hqmq.PackedKV(_first(cache.K, 4), _first(cache.V, 4)), kv_lens=pos[:4], T_kv=T,
                                     force_generic=True)
    assert (Og.float() - O[:4].float()).abs().max().item() <= 2.0 ** -7 * max(1.0, worst[3])


def _first(pt, nb):
    """A view of the first nb sequences of a PackedTensor (same planes, no copy)."""
    import copy
    o = copy.copy(pt)
    o.B = nb
    for name in ("main", "aux", "scale", "flags", "sideband", "sb_tile_off", "sb_count", "sb_coord"):
        t = getattr(pt, name)
        if t is not None:
            setattr(o, name, t[:nb])
    return o


@pytest.mark.parametrize("cfg", [3, 5])
def test_config3_and_5_full_size_properties(cfg):
    """Benchmark configs 3 (28/4 heads, batch 8, 32k, s192_r6 + Med3x, fp16, 2 % of K chunks x50-200) and
    5 (64/8 heads, d_h 64, batch 4, 131072, s96_r4 + Med3x, bf16, 1 % of chunks x100) at full size: agreement with
    dense fp32 attention over the dequantized cache, split invariance, and the specialised kernel against the
    layout-generic one.  Outputs reach |O| ~ 4 (config 3) and ~ 350 (config 5), so bounds are relative to that."""
    import hqmq
    from hqmq_amd.bench_configs import dense_check, synth
    if cfg == 3:
        B, Hq, Hkv, d, S, b_r, dt, T = 8, 28, 4, 128, 192, 6, torch.float16, 32768
        k, v = synth((B, Hkv, T, d), dt, 31, outlier_p=0.02), synth((B, Hkv, T, d), dt, 32)
    else:
        B, Hq, Hkv, d, S, b_r, dt, T = 4, 64, 8, 64, 96, 4, torch.bfloat16, 131072
        k = synth((B, Hkv, T, d), dt, 51, outlier_p=0.01, gain=(100.0, 100.0))
        v = synth((B, Hkv, T, d), dt, 52, outlier_p=0.01, gain=(100.0, 100.0))
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV), C=3.0)
    cache = w.new_cache(B, T, d, dt, 0, sideband_frac=0.125)
    w.append(cache, k, v, 0)
    cache.K.check_overflow()
    cache.V.check_overflow()
    rate = float(cache.K.sb_count.sum()) / (B * Hkv * T * d / 4)
    assert 0.005 < rate < 0.03
    Q = torch.randn(B, Hq, 1, d, generator=torch.Generator().manual_seed(7)).to(dt).to(DEV)
    O = hqmq.fused_attention_packed(Q, cache)
    worst = _two_reference_check(O, Q, cache, lambda b, L: (k[b, :, :L], v[b, :, :L]), [T] * B, f"config {cfg} at full size")
    del k, v
    err, ref_max = dense_check(Q, cache, None, T)
    scale = max(1.0, ref_max)
    assert err < 2e-3 * scale, (err, ref_max)
    for ns in (1, 5):
        o = hqmq.fused_attention_packed(Q, cache, n_splits=ns)
        assert (o.float() - O.float()).abs().max().item() < 1e-3 * scale
    og = hqmq.fused_attention_packed(Q, cache, force_generic=True)
    assert (og.float() - O.float()).abs().max().item() < 1e-3 * scale


@pytest.mark.parametrize("d_h,Tq,hot,dn", [(64, 1, (2, 5), "fp16"), (64, 144, (2, 5), "fp16"), (64, 1, (0, 1, 2, 3), "bf16"),
                                            (128, 1, (0, 1, 2, 8, 30), "fp16"), (128, 9, (3, 17), "bf16")])
def test_clustered_outlier_channels(d_h, Tq, hot, dn):
    """Outlier *channels*: the same chunk positions are flagged in most tokens (up to 25 % of all chunks, several per
    lane and more than 64 per half-step), decode and chunked prefill; specialised and layout-generic kernels
    against dense fp32 attention over the dequantized cache."""
    import hqmq
    from hqmq_amd import ops
    dt = DT[dn]
    B, Hq, Hkv, T = 2, 8, 2, 150
    g = torch.Generator().manual_seed(3)
    k, v = torch.randn(B, Hkv, T, d_h, generator=g), torch.randn(B, Hkv, T, d_h, generator=g)
    for c in hot:
        k[..., 4 * c:4 * c + 4] *= 12.0
        v[..., 4 * c:4 * c + 4] *= 12.0
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=96, radius_bits=4, device=DEV), C=3.0)
    cache = w.new_cache(B, T, d_h, dt, 0, sideband_frac=0.5)
    w.append(cache, k.to(dt).to(DEV), v.to(dt).to(DEV), 0)
    cache.K.check_overflow()
    cache.V.check_overflow()
    assert float(cache.K.sb_count.sum()) / (B * Hkv * T * d_h / 4) > 0.02
    Q = torch.randn(B, Hq, Tq, d_h, generator=g).to(dt).to(DEV)
    off = T - Tq
    mask = torch.arange(T, device=DEV).view(1, 1, 1, T) <= (torch.arange(Tq, device=DEV).view(1, 1, Tq, 1) + off)
    refs = masked_two_refs(cache, Q, T, mask)
    for generic in (False, True):
        for ns in (0, 3):
            O = hqmq.fused_attention_packed(Q, cache, causal=True, causal_offset=off, force_generic=generic, n_splits=ns)
            assert_attention_close(O, *refs, base=2e-3, what=f"generic={generic} n_splits={ns}")


def _planted(B, H, T, d, seed, dt):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, H, T, d, generator=g)
    hit = torch.rand(B, H, T, d // 4, 1, generator=g) < 0.04
    x = torch.where(hit, x.view(B, H, T, d // 4, 4) * 40.0, x.view(B, H, T, d // 4, 4)).reshape(B, H, T, d)
    return x.to(dt).to(DEV)


def test_crop_then_append_again_equals_never_appended():
    """crop_ puts the outlier list and its tile offsets back to the state after the last kept row: rows appended,
    cropped and appended again give the same planes, the same list and the same attention output as a cache that
    never saw the cropped rows (same calls otherwise, so the per-call medians agree)."""
    import hqmq
    dt = torch.float16
    B, Hq, Hkv, T, d_h = 2, 8, 2, 200, 128
    k, v = _planted(B, Hkv, T, d_h, 11, dt), _planted(B, Hkv, T, d_h, 12, dt)
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=96, radius_bits=4, device=DEV), C=3.0)
    a = w.new_cache(B, T + 40, d_h, dt, 0, sideband_frac=0.5)
    w.append(a, k[:, :, :150], v[:, :, :150], 0)
    w.append(a, k[:, :, 150:], v[:, :, 150:], 0)
    b = w.new_cache(B, T + 40, d_h, dt, 0, sideband_frac=0.5)
    w.append(b, k[:, :, :150], v[:, :, :150], 0)
    w.append(b, k[:, :, 40:75], v[:, :, 40:75], 0)          # 35 rows that are dropped again (the cut is inside a tile)
    b.crop_(150)
    assert b.length == 150
    w.append(b, k[:, :, 150:], v[:, :, 150:], 0)
    for pa, pb in ((a.K, b.K), (a.V, b.V)):
        assert int(pa.sb_count.min()) > 0 and torch.equal(pa.sb_count, pb.sb_count)
        assert torch.equal(pa.sb_tile_off, pb.sb_tile_off)
        for x, y in ((pa.main, pb.main), (pa.flags, pb.flags), (pa.scale.view(torch.int16), pb.scale.view(torch.int16))):
            assert torch.equal(x[:, :, :T], y[:, :, :T])
        for bb in range(B):
            for h in range(Hkv):
                c = int(pa.sb_count[bb, h])
                assert torch.equal(pa.sideband[bb, h, :c].view(torch.int16), pb.sideband[bb, h, :c].view(torch.int16))
                assert torch.equal(pa.sb_coord[bb, h, :c], pb.sb_coord[bb, h, :c])
    Q = torch.randn(B, Hq, 1, d_h, generator=torch.Generator().manual_seed(13)).to(dt).to(DEV)
    Oa = hqmq.fused_attention_packed(Q, a, causal=False)
    for generic in (False, True):
        assert torch.equal(hqmq.fused_attention_packed(Q, b, causal=False, force_generic=generic),
                           Oa if not generic else hqmq.fused_attention_packed(Q, a, causal=False, force_generic=True))


def test_crop_per_sequence_then_decode_appends():
    """Ragged crop (tile-aligned and not), then appends at pos: specialised and layout-generic kernels against dense
    attention over the dequantized cache with per-sequence lengths."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.bfloat16
    B, Hq, Hkv, T, d_h = 3, 8, 2, 160, 64
    k, v = _planted(B, Hkv, T, d_h, 21, dt), _planted(B, Hkv, T, d_h, 22, dt)
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=96, radius_bits=4, device=DEV), C=3.0)
    cache = w.new_cache(B, T + 64, d_h, dt, 0, sideband_frac=0.5)
    w.append(cache, k, v, 0)
    lens = torch.tensor([150, 128, 37], dtype=torch.int32, device=DEV)
    cache.crop_(lens)
    pos = lens.clone()
    for step in range(20):                                   # crosses tile boundaries in every sequence
        w.append(cache, k[:, :, step:step + 1], v[:, :, step:step + 1], 0, pos=pos)
        pos += 1
    cache.K.check_overflow()
    Tm = int(pos.max())
    Q = torch.randn(B, Hq, 1, d_h, generator=torch.Generator().manual_seed(23)).to(dt).to(DEV)
    Kd = ops.dequant_packed(cache.K, Tm, 0).float().repeat_interleave(Hq // Hkv, 1)
    Vd = ops.dequant_packed(cache.V, Tm, 0).float().repeat_interleave(Hq // Hkv, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float(), Kd) * d_h ** -0.5
    mask = torch.arange(Tm, device=DEV).view(1, 1, 1, Tm) < pos.view(B, 1, 1, 1)
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s.masked_fill(~mask, float("-inf")), -1), Vd)
    # the appended rows really are the new tokens: row lens[b] + i decodes to (about) k[b, :, i]
    for bb in range(B):
        got = ops.dequant_packed(cache.K, Tm, 0)[bb, :, int(lens[bb]):int(lens[bb]) + 20].float()
        assert (got - k[bb, :, :20].float()).abs().mean().item() < 0.25 * k[bb, :, :20].float().abs().mean().item()
    refs = masked_two_refs(cache, Q, Tm, mask)
    for generic in (False, True):
        O = hqmq.fused_attention_packed(Q, cache, causal=False, kv_lens=pos, T_kv=Tm, force_generic=generic)
        assert_attention_close(O, *refs, base=2e-3, what=f"generic={generic}")
        assert (O.float() - ref).abs().max().item() < 2e-2 * max(1.0, float(ref.abs().max())), generic       # and the plain fp32 einsum, loosely


@pytest.mark.parametrize("med3x,Tq", [(False, 1), (True, 1), (True, 24)])
def test_left_padded_batch(med3x, Tq):
    """kv_starts: the tokens in front of every sequence's first real one are invisible (left padding), decode and
    chunked prefill, both kernels, against dense attention with the explicit mask."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.float16
    B, Hq, Hkv, T, d_h = 4, 8, 2, 300, 128
    if med3x:
        k, v = _planted(B, Hkv, T, d_h, 31, dt), _planted(B, Hkv, T, d_h, 32, dt)
    else:
        g = torch.Generator().manual_seed(31)
        k, v = torch.randn(B, Hkv, T, d_h, generator=g).to(dt).to(DEV), torch.randn(B, Hkv, T, d_h, generator=g).to(dt).to(DEV)
    q = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=96, radius_bits=4, device=DEV)
    w = hqmq.with_outlier_extraction(q, C=3.0) if med3x else q
    cache = w.new_cache(B, T, d_h, dt, 0, **({"sideband_frac": 0.5} if med3x else {}))
    w.append(cache, k, v, 0)
    starts = torch.tensor([0, 7, 64, 201], dtype=torch.int32, device=DEV)
    Q = torch.randn(B, Hq, Tq, d_h, generator=torch.Generator().manual_seed(33)).to(dt).to(DEV)
    off = T - Tq
    Kd = ops.dequant_packed(cache.K, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    Vd = ops.dequant_packed(cache.V, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float(), Kd) * d_h ** -0.5
    kk = torch.arange(T, device=DEV).view(1, 1, 1, T)
    mask = (kk <= torch.arange(Tq, device=DEV).view(1, 1, Tq, 1) + off) & (kk >= starts.view(B, 1, 1, 1))
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s.masked_fill(~mask, float("-inf")), -1), Vd)
    tol = 2e-3 * max(1.0, float(ref.abs().max()))
    for generic in (False, True):
        for ns in (0, 1, 3):
            O = hqmq.fused_attention_packed(Q, cache, causal=True, causal_offset=off, kv_starts=starts, n_splits=ns,
                                            force_generic=generic)
            assert (O.float() - ref).abs().max().item() < tol, (generic, ns)
    # a start behind everything a query may see: that row attends to nothing and comes back as zeros
    late = torch.full((B,), T, dtype=torch.int32, device=DEV)
    O = hqmq.fused_attention_packed(Q, cache, causal=True, causal_offset=off, kv_starts=late)
    assert int(O.abs().sum()) == 0


def test_batch_order_is_scheduling_only():
    """batch_order changes which sequence's blocks start first, never the result: bit-equal outputs for the natural
    order, longest-first and a shuffled permutation, ragged batch with outliers, both kernels."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.bfloat16
    B, Hq, Hkv, T, d_h = 6, 8, 2, 260, 128
    k, v = _planted(B, Hkv, T, d_h, 41, dt), _planted(B, Hkv, T, d_h, 42, dt)
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=24, radius_bits=3, device=DEV), C=3.0)
    cache = w.new_cache(B, T, d_h, dt, 0, sideband_frac=0.5)
    w.append(cache, k, v, 0)
    lens = torch.tensor([260, 17, 128, 255, 1, 64], dtype=torch.int32, device=DEV)
    Q = torch.randn(B, Hq, 1, d_h, generator=torch.Generator().manual_seed(43)).to(dt).to(DEV)
    lf = ops.longest_first(lens)
    assert lf.tolist() == [0, 3, 2, 5, 1, 4]
    for generic in (False, True):
        base = hqmq.fused_attention_packed(Q, cache, kv_lens=lens, T_kv=T, n_splits=2, force_generic=generic)
        for order in (lf, torch.tensor([4, 2, 0, 5, 3, 1], dtype=torch.int32, device=DEV)):
            O = hqmq.fused_attention_packed(Q, cache, kv_lens=lens, T_kv=T, n_splits=2, force_generic=generic, batch_order=order)
            assert torch.equal(O, base)


@pytest.mark.parametrize("dn,kv_lens,S,b_r", [("fp16", None, 96, 4), ("bf16", [13000, 6200], 96, 4), ("bf16", None, 24, 3)])
def test_long_ranges_per_block(dn, kv_lens, S, b_r):
    """Plain s96_r4 and s24_r3 caches with more than 6144 tokens per block run with twelve wavefronts per block (ranges
    of whole 32-token half-steps, a merge over twelve partials): against the layout-generic kernel and dense attention."""
    import hqmq
    from hqmq_amd import ops
    dt = DT[dn]
    B, Hq, Hkv, T, d_h = 2, 8, 2, 13000, 128
    g = torch.Generator().manual_seed(51)
    k, v = torch.randn(B, Hkv, T, d_h, generator=g).to(dt).to(DEV), torch.randn(B, Hkv, T, d_h, generator=g).to(dt).to(DEV)
    q = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV)
    cache = q.new_cache(B, T, d_h, dt, 0)
    q.append(cache, k, v, 0)
    lens = None if kv_lens is None else torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
    Q = (torch.randn(B, Hq, 1, d_h, generator=g) * 2.0).to(dt).to(DEV)          # a peaked softmax: the merge weights matter
    Kd = ops.dequant_packed(cache.K, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    Vd = ops.dequant_packed(cache.V, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float(), Kd) * d_h ** -0.5
    if lens is not None:
        s = s.masked_fill(torch.arange(T, device=DEV).view(1, 1, 1, T) >= lens.view(B, 1, 1, 1), float("-inf"))
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, -1), Vd)
    vis = None if lens is None else torch.arange(T, device=DEV).view(1, 1, 1, T) < lens.view(B, 1, 1, 1)
    refs = masked_two_refs(cache, Q, T, vis)
    assert (refs[0].to(DEV) - ref).abs().max().item() < 1e-3 * max(1.0, float(ref.abs().max()))     # the helper against the plain einsum
    for ns in (1, 2):
        O = hqmq.fused_attention_packed(Q, cache, kv_lens=lens, T_kv=T, n_splits=ns)
        Og = hqmq.fused_attention_packed(Q, cache, kv_lens=lens, T_kv=T, n_splits=ns, force_generic=True)
        Or = hqmq.fused_attention_packed(Q, cache, kv_lens=lens, T_kv=T, n_splits=ns, force_generic=2)        # register-tile kernel
        for name, o in (("specialised", O), ("generic", Og), ("register tiles", Or)):
            assert_attention_close(o, *refs, base=2e-3, what=f"{name} n_splits={ns}")


def test_long_ranges_per_block_outliers_d64():
    """The d_h 64 outlier variant also runs twelve wavefronts per block above 6144 tokens per block."""
    import hqmq
    from hqmq_amd import ops
    dt = torch.bfloat16
    B, Hq, Hkv, T, d_h = 2, 16, 2, 13000, 64
    k, v = _planted(B, Hkv, T, d_h, 61, dt), _planted(B, Hkv, T, d_h, 62, dt)
    w = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=96, radius_bits=4, device=DEV), C=3.0)
    cache = w.new_cache(B, T, d_h, dt, 0, sideband_frac=0.25)
    w.append(cache, k, v, 0)
    cache.K.check_overflow()
    cache.V.check_overflow()
    Q = torch.randn(B, Hq, 1, d_h, generator=torch.Generator().manual_seed(63)).to(dt).to(DEV)
    Kd = ops.dequant_packed(cache.K, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    Vd = ops.dequant_packed(cache.V, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float(), Kd) * d_h ** -0.5
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, -1), Vd)
    refs = masked_two_refs(cache, Q, T)
    assert (refs[0].to(DEV) - ref).abs().max().item() < 1e-3 * max(1.0, float(ref.abs().max()))
    for ns in (1, 2):
        O = hqmq.fused_attention_packed(Q, cache, n_splits=ns)
        Og = hqmq.fused_attention_packed(Q, cache, n_splits=ns, force_generic=True)
        assert_attention_close(O, *refs, base=2e-3, what=f"specialised n_splits={ns}")
        assert_attention_close(Og, *refs, base=2e-3, what=f"generic n_splits={ns}")


@pytest.mark.parametrize("S,b_r,dn,d_h", [(96, 4, "fp16", 128), (24, 3, "bf16", 128), (192, 6, "fp16", 128), (96, 4, "bf16", 64)])
def test_prefill_two_column_groups(S, b_r, dn, d_h):
    """Chunked prefill with enough columns for a block per CU runs two column groups per wavefront on plain caches
    (an odd number of groups, a last group that is partly padding, causal limits that differ inside a wavefront):
    against dense attention and the layout-generic kernel."""
    import hqmq
    from hqmq_amd import ops
    dt = DT[dn]
    B, Hq, Hkv, T, Tq = 2, 8, 2, 700, 299
    g = torch.Generator().manual_seed(71)
    k, v = torch.randn(B, Hkv, T, d_h, generator=g).to(dt).to(DEV), torch.randn(B, Hkv, T, d_h, generator=g).to(dt).to(DEV)
    q = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV)
    cache = q.new_cache(B, T, d_h, dt, 0)
    q.append(cache, k, v, 0)
    Q = torch.randn(B, Hq, Tq, d_h, generator=g).to(dt).to(DEV)
    off = T - Tq
    Kd = ops.dequant_packed(cache.K, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    Vd = ops.dequant_packed(cache.V, T, 0).float().repeat_interleave(Hq // Hkv, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", Q.float(), Kd) * d_h ** -0.5
    mask = torch.arange(T, device=DEV).view(1, 1, 1, T) <= (torch.arange(Tq, device=DEV).view(1, 1, Tq, 1) + off)
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s.masked_fill(~mask, float("-inf")), -1), Vd)
    refs = masked_two_refs(cache, Q, T, mask)
    assert (refs[0].to(DEV) - ref).abs().max().item() < 1e-3 * max(1.0, float(ref.abs().max()))
    for ns in (2, 4):                       # 2 splits x 38 pairs of column groups x 4 (b, h) = 304 blocks
        O = hqmq.fused_attention_packed(Q, cache, causal=True, causal_offset=off, n_splits=ns)
        assert_attention_close(O, *refs, base=2e-3, what=f"n_splits={ns}")
    Og = hqmq.fused_attention_packed(Q, cache, causal=True, causal_offset=off, n_splits=2, force_generic=True)
    assert_attention_close(Og, *refs, base=2e-3, what="generic")
    # the same with per-sequence limits on both sides (left padding and a shorter second sequence)
    starts = torch.tensor([0, 70], dtype=torch.int32, device=DEV)
    lens = torch.tensor([T, 650], dtype=torch.int32, device=DEV)
    kk = torch.arange(T, device=DEV).view(1, 1, 1, T)
    mask2 = mask & (kk >= starts.view(B, 1, 1, 1)) & (kk < lens.view(B, 1, 1, 1))
    ref2 = torch.einsum("bhqk,bhkd->bhqd", torch.nan_to_num(torch.softmax(s.masked_fill(~mask2, float("-inf")), -1)), Vd)
    O2 = hqmq.fused_attention_packed(Q, cache, causal=True, causal_offset=off, n_splits=2, kv_starts=starts, kv_lens=lens, T_kv=T)
    refs2 = masked_two_refs(cache, Q, T, mask2)
    assert (refs2[0].to(DEV) - ref2).abs().max().item() < 1e-3 * max(1.0, float(ref2.abs().max()))
    assert_attention_close(O2, *refs2, base=2e-3, what="left padding and a shorter sequence")


@pytest.mark.parametrize("dn,T,B,Tq,causal,ns,lens", [
    ("fp16", 32, 1, 1, False, 0, None), ("fp16", 96, 1, 1, False, 0, None), ("fp16", 1000, 1, 1, False, 0, None),
    ("fp16", 8192, 1, 1, False, 0, None), ("fp16", 777, 3, 1, False, 2, None), ("fp16", 5000, 2, 1, False, 0, [4100, 37]),
    ("fp16", 2048, 1, 3, True, 0, None), ("bf16", 4096, 1, 1, False, 0, None), ("bf16", 20000, 2, 1, False, 3, None),
    ("bf16", 300, 1, 4, True, 0, None), ("fp16", 33, 1, 1, False, 1, None), ("fp16", 3000, 2, 1, False, 5, [0, 2999])])
def test_lds_landing_kernel_equals_register_tile_kernel(dn, T, B, Tq, causal, ns, lens):
    """Plain s96_r4 caches at d_h 128 take the kernel whose loads land in LDS (tables, query rows and planes through
    global_load_lds, hand-written waits).  It performs the arithmetic of the register-tile kernel in the same order, so
    the two must agree bit for bit (force_generic=2 selects the register-tile kernel); both are held to the
    two-reference bound, and so is the layout-generic kernel."""
    import hqmq
    dt = DT[dn]
    Hq, Hkv, d_h = 8, 2, 128
    g = torch.Generator().manual_seed(T + 7 * B)
    k, v = torch.randn(B, Hkv, T, d_h, generator=g).to(dt).to(DEV), torch.randn(B, Hkv, T, d_h, generator=g).to(dt).to(DEV)
    q = hqmq.HQMQ(n_layers=2, n_heads=Hkv, secondary_size=96, radius_bits=4, device=DEV)
    cache = q.new_cache(B, T, d_h, dt, layer_idx=1)
    q.append(cache, k, v, 1)
    Q = torch.randn(B, Hq, Tq, d_h, generator=g).to(dt).to(DEV)
    kv_lens = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
    off = T - Tq
    kw = dict(causal=causal, causal_offset=off if causal else 0, n_splits=ns, kv_lens=kv_lens, T_kv=T)
    O = hqmq.fused_attention_packed(Q, cache, **kw)
    Or = hqmq.fused_attention_packed(Q, cache, force_generic=2, **kw)
    Og = hqmq.fused_attention_packed(Q, cache, force_generic=True, **kw)
    assert torch.equal(O, Or)
    kk = torch.arange(T, device=DEV).view(1, 1, 1, T)
    mask = torch.ones(B, 1, Tq, T, dtype=torch.bool, device=DEV)
    if causal:
        mask = mask & (kk <= torch.arange(Tq, device=DEV).view(1, 1, Tq, 1) + off)
    if kv_lens is not None:
        mask = mask & (kk < kv_lens.view(B, 1, 1, 1))
    refs = masked_two_refs(cache, Q, T, mask)
    assert_attention_close(O, *refs, base=2e-3, what="LDS landing")
    assert_attention_close(Og, *refs, base=2e-3, what="generic")
