"""GPU parity: joint table, quantize, dense decode and the packed planes, through the C ABI,
bit-exact against the CPU oracle and the reference's golden outputs."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as CO
from oracle import torch_oracle as TO
from tests.helpers import DT, bit_equal, kv_input, unbits

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a GPU")]
DEV = "cuda"
CODEBOOKS = [(24, 3), (96, 4), (192, 6)]


def _ops():
    from hqmq_amd import ops
    return ops


def edge_cases(x):
    """zero chunk, zero token, huge chunk, axis-aligned and half-unit directions, fp16-subnormal norms"""
    dt = x.dtype
    x[0, 0, 3, 8:12] = 0
    x[-1, -1, 5, :] = 0
    x[0, -1, 7, 0:4] *= 100
    x[-1, 0, 9, 4:8] = torch.tensor([1., 0, 0, 0]).to(dt)
    x[-1, 0, 10, :4] = torch.tensor([.5, .5, .5, .5]).to(dt)
    x[0, 0, 11, :8] = torch.tensor([3e-8, 0, 0, 0, 1e-7, 1e-7, 0, 0]).to(dt)
    x[0, 0, 12, :4] = torch.tensor([0.7071, 0.7071, 0, 0]).to(dt)
    return x


@pytest.mark.parametrize("S,b_r", CODEBOOKS)
@pytest.mark.parametrize("dn", ["fp32", "fp16", "bf16"])
def test_joint_and_quantize_match_oracle(S, b_r, dn):
    ops, dt = _ops(), DT[dn]
    raw = TO.secondary_raw(1, 3, S, 5)[0, :, 0]
    Jc = CO.joint_table(raw, dt)
    J, slack = ops.build_joint(raw.to(DEV), dt)
    assert bit_equal(J, Jc)
    assert float(slack.max()) < {torch.float32: 1e-6, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dt]
    x = edge_cases(kv_input((2, 3, 200, 64), dt, seed=S))
    want = CO.quantize(x, Jc, b_r)
    for algo in (0, 1):           # closed-form filter + re-score, and the brute-force scan
        stats = torch.zeros(2, dtype=torch.int32, device=DEV)
        got = ops.quantize(x.to(DEV), J, slack, b_r, want_dense=True, algo=algo, stats=stats)
        assert torch.equal(got["idx"].cpu(), want["idx"]), f"algo {algo}"
        assert torch.equal(got["rq"].cpu(), want["rq"])
        assert bit_equal(got["r_max"], want["r_max"])
        assert bit_equal(got["out"], want["out"])
        if algo == 0:             # the filter must do the work; the exhaustive fallback is for rare lanes only
            assert int(stats[0]) < 0.01 * x.numel() / 4


def test_quantize_golden_outputs(golden_dir):
    """quantize_K / quantize_V through the public classes reproduce the reference's dense output bit for bit."""
    import hqmq
    g = np.load(golden_dir / "quantizer.npz")
    for cfg in ("s24r3", "s96r4", "s192r6"):
        S, b_r, seed, L, H = (int(v) for v in g[cfg + "_meta"])
        q = hqmq.HQMQ(n_layers=L, n_heads=H, secondary_size=S, radius_bits=b_r, device=DEV, seed=seed)
        assert torch.equal(q.secondary_raw.detach().cpu(), torch.from_numpy(g[cfg + "_raw"]))
        for dn, dt in DT.items():
            for kv, tag in ((0, "K"), (1, "V")):
                key = f"{cfg}_{dn}_{tag}"
                x = unbits(g[key + "_x"], dt).to(DEV)
                assert bit_equal(q._get_codebook(1, kv, x), unbits(g[key + "_joint"], dt)), key
                y = q.quantize_K(x, 1) if kv == 0 else q.quantize_V(x, 1)
                assert y.shape == x.shape and y.dtype == x.dtype and y.device == x.device
                assert bit_equal(y, unbits(g[key + "_out"], dt)), key


@pytest.mark.parametrize("dn", ["fp16", "bf16"])
def test_adversarial_ties(dn):
    """Inputs built to tie: chunks that are exact codewords, their negatives and midpoints of two codewords."""
    ops, dt = _ops(), DT[dn]
    S, b_r = 24, 3
    raw = TO.secondary_raw(1, 1, S, 11)[0, :, 0]
    Jc = CO.joint_table(raw, dt)
    J, slack = ops.build_joint(raw.to(DEV), dt)
    Jf = Jc[0].float()
    rows = [Jf, -Jf, 3 * Jf, Jf + Jf.roll(1, 0), Jf + Jf.roll(S, 0), TO.cell24().repeat(24, 1)]
    x = torch.cat(rows, 0).reshape(1, 1, -1, 16).to(dt)
    want = CO.quantize(x, Jc, b_r)
    got = ops.quantize(x.to(DEV), J, slack, b_r)
    assert torch.equal(got["idx"].cpu(), want["idx"]) and torch.equal(got["rq"].cpu(), want["rq"])


@pytest.mark.parametrize("S,b_r", CODEBOOKS)
@pytest.mark.parametrize("dn", ["fp16", "bf16"])
@pytest.mark.parametrize("d_h", [16, 64, 128, 256])
def test_single_token_calls_match_oracle(S, b_r, dn, d_h):
    """Calls with one token per sequence (the decode-step append) search with the secondaries split over the
    block's token slots; indices, radius codes and scales equal the oracle's, edge cases and ties included."""
    ops, dt = _ops(), DT[dn]
    H, N = 2, 160
    raw = TO.secondary_raw(1, H, S, 9)[0, :, 0]
    Jc = CO.joint_table(raw, dt)
    J, slack = ops.build_joint(raw.to(DEV), dt)
    x = kv_input((N, H, 1, d_h), dt, seed=21, outlier_p=0.02)
    e = edge_cases(x.transpose(0, 2).contiguous())          # the helper plants along the token axis
    x = e.transpose(0, 2).contiguous()
    Jf = Jc[0].float()                                      # exact codewords, negatives and midpoints: ties
    ties = torch.cat([Jf[:40], -Jf[40:80], Jf[:40] + Jf.roll(1, 0)[:40], Jf[:40] + Jf.roll(S, 0)[:40]], 0).to(dt)
    flat = ties.reshape(-1)
    n_tok = flat.numel() // d_h
    x[:n_tok, 0, 0] = flat[:n_tok * d_h].reshape(n_tok, d_h)
    want = CO.quantize(x, Jc, b_r)
    got = ops.quantize(x.to(DEV), J, slack, b_r, want_dense=True)
    assert torch.equal(got["idx"].cpu(), want["idx"])
    assert torch.equal(got["rq"].cpu(), want["rq"])
    assert bit_equal(got["r_max"], want["r_max"])
    assert bit_equal(got["out"], want["out"])


@pytest.mark.parametrize("S,b_r,dn,d_h", [(24, 3, "bf16", 128), (96, 4, "fp16", 128), (192, 6, "fp16", 64), (96, 4, "bf16", 32)])
def test_token_by_token_appends_equal_one_bulk_append(S, b_r, dn, d_h):
    """The split search of single-token appends and the bulk search leave the same planes."""
    import hqmq
    dt = DT[dn]
    B, H, T = 3, 2, 37
    q = hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=S, radius_bits=b_r, device=DEV)
    k = edge_cases(kv_input((B, H, T, d_h), dt, seed=5, outlier_p=0.03)).to(DEV)
    v = kv_input((B, H, T, d_h), dt, seed=6).to(DEV)
    bulk, steps = q.new_cache(B, T, d_h, dt, 0), q.new_cache(B, T, d_h, dt, 0)
    q.append(bulk, k, v, 0)
    for t in range(T):
        q.append(steps, k[:, :, t:t + 1], v[:, :, t:t + 1], 0)
    for a, b in ((bulk.K, steps.K), (bulk.V, steps.V)):
        for name in ("main", "aux", "scale"):
            x, y = getattr(a, name), getattr(b, name)
            if x is not None:
                assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), name


def test_strided_input_and_error_paths():
    import hqmq
    ops = _ops()
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=24, radius_bits=3, device=DEV)
    base = kv_input((2, 2, 33, 128), torch.float16, seed=3).to(DEV)
    view = base[:, :, 1::2, 32:96]                      # non-contiguous over T and d_h
    assert bit_equal(q.quantize_K(view, 0), q.quantize_K(view.contiguous(), 0))
    tr = base.transpose(1, 2).contiguous().transpose(1, 2)   # (B, T, H, d) memory, as attention layers hand it over
    assert bit_equal(q.quantize_V(tr, 0), q.quantize_V(base, 0))
    with pytest.raises(ValueError):
        q.quantize_K(torch.randn(1, 2, 4, 30, device=DEV), 0)
    assert q.quantize_K(base[:, :, :0], 0).shape == (2, 2, 0, 128)      # empty call


def test_full_size_config1_round_trip():
    """Benchmark config 1 at full size (8 KV heads, d_h=128, T=2048, s24_r3 + Med3x, fp16): codes, scales,
    mask and the fake-quant tensor bit-exact against the oracle; MSE reported."""
    import hqmq
    dt = torch.float16
    x = kv_input((1, 8, 2048, 128), dt, seed=1)
    q = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=1, n_heads=8, secondary_size=24, radius_bits=3, device=DEV, seed=42), C=3.0)
    for kv in (0, 1):
        Jc = CO.joint_table(TO.secondary_raw(1, 8, 24, 42)[0, :, kv], dt)
        want = CO.outlier_quantize(x, Jc, 3, 3.0)
        got = q.encode(x.to(DEV), 0, kv)
        assert torch.equal(got["idx"].cpu(), want["idx"]) and torch.equal(got["rq"].cpu(), want["rq"])
        assert bit_equal(got["r_max"], want["r_max"]) and torch.equal(got["mask"].cpu(), want["mask"])
        assert torch.equal(got["median"].cpu(), want["median"]) and bit_equal(got["threshold"], want["threshold"])
        y = q.quantize_K(x.to(DEV), 0) if kv == 0 else q.quantize_V(x.to(DEV), 0)
        assert bit_equal(y, want["out"])
        mse = float(((y.float().cpu() - x.float()) ** 2).mean())
        assert mse < 0.1 * float((x.float() ** 2).mean())
    assert q._n_observations == 0 or q.bits_per_value() > 3.0     # stats fold lazily
    assert q.bits_per_value() > q.inner.bits_per_value()


def test_full_size_filter_equals_bruteforce():
    """Size-independent property at config-2 scale (8 heads x 32768 tokens, s96_r4): the filtered search and
    the exhaustive scan are two implementations of the same rule and must pick identical codes."""
    ops = _ops()
    raw = TO.secondary_raw(1, 8, 96, 42)[0, :, 0]
    J, slack = ops.build_joint(raw.to(DEV), torch.float16)
    x = torch.randn(1, 8, 32768, 128, generator=torch.Generator().manual_seed(9)).half().to(DEV)
    a = ops.quantize(x, J, slack, 4, algo=0)
    b = ops.quantize(x, J, slack, 4, algo=1)
    assert torch.equal(a["idx"], b["idx"]) and torch.equal(a["rq"], b["rq"]) and bit_equal(a["r_max"], b["r_max"])
    # and a slice of it against the CPU oracle
    want = CO.quantize(x[:, :, 1000:1256].cpu(), CO.joint_table(raw, torch.float16), 4, dense=False)
    assert torch.equal(a["idx"][:, :, 1000:1256].cpu(), want["idx"]) and torch.equal(a["rq"][:, :, 1000:1256].cpu(), want["rq"])


@pytest.mark.parametrize("S", [24, 96, 192])
@pytest.mark.parametrize("dn", ["fp16", "bf16"])
def test_filter_equals_bruteforce_where_scores_tie(S, dn):
    """The candidate threshold follows the rounding of the scores to the cache dtype; inputs whose best scores share
    one rounded value are where a threshold set too high would drop the winner.  Chunks next to codewords, halfway
    between two codewords, sparse and widely scaled rows: the filtered search must pick what the exhaustive scan
    picks (2 M chunks per case)."""
    ops, dt = _ops(), DT[dn]
    H, T, d_h = 8, 8192, 128
    g = torch.Generator(device=DEV).manual_seed(1000 + S)
    raw = torch.randn(H, S, 4, generator=g, device=DEV)
    J, slack = ops.build_joint(raw, dt)
    K = J.shape[1]

    def rows_of(pick):
        return torch.gather(J.float(), 1, pick[..., None].expand(-1, -1, 4)).reshape(H, T, d_h)

    r1 = rows_of(torch.randint(0, K, (H, T * d_h // 4), generator=g, device=DEV))
    r2 = rows_of(torch.randint(0, K, (H, T * d_h // 4), generator=g, device=DEV))
    scale = torch.exp(torch.randn(1, H, T, 1, generator=g, device=DEV))
    cases = {
        "near_codeword": (r1 * (1 + 1e-3 * torch.randn(H, T, d_h, generator=g, device=DEV)))[None] * scale,
        "between_two": ((r1 + r2) * 0.5)[None],
        "sparse": torch.randn(1, H, T, d_h, generator=g, device=DEV) * (torch.rand(1, H, T, d_h, generator=g, device=DEV) < 0.3),
        "scaled": torch.randn(1, H, T, d_h, generator=g, device=DEV) * scale ** 3,
    }
    for name, x in cases.items():
        x = x.to(dt)
        a = ops.quantize(x, J, slack, 4, algo=0)
        b = ops.quantize(x, J, slack, 4, algo=1)
        assert torch.equal(a["idx"], b["idx"]) and torch.equal(a["rq"], b["rq"]), name


# ---------------------------------------------------------------- dense decode
@pytest.mark.parametrize("S,b_r", CODEBOOKS)
@pytest.mark.parametrize("dn", ["fp32", "fp16", "bf16"])
def test_dequant_matches_oracle(S, b_r, dn):
    from hqmq.kernels import decode_dequant
    dt = DT[dn]
    qmax = (1 << b_r) - 1
    g = torch.Generator().manual_seed(S)
    idx = torch.randint(0, 24 * S, (2, 3, 37, 16), generator=g, dtype=torch.int32)
    rq = torch.randint(0, qmax + 1, (2, 3, 37, 16), generator=g, dtype=torch.int32)
    rs = (torch.rand(2, 3, 37, generator=g) + 0.5).to(dt)
    J = CO.joint_table(TO.secondary_raw(1, 3, S, 2)[0, :, 1], dt)
    out = decode_dequant(idx.to(DEV), rq.to(DEV), rs.to(DEV), J.to(DEV), qmax)
    assert out.dtype == dt and bit_equal(out, CO.dequant(idx, rq, rs, J, qmax))
    out8 = decode_dequant(idx.to(DEV), rq.to(torch.int8).to(DEV), rs.to(DEV), J.to(DEV), qmax)   # any int dtype for rq
    assert bit_equal(out8, out)


def test_dequant_known_answer():
    """The reference's own kernel check (experiments/32a_kernel_debug.py:23-45): joint = arange, all radii = 1
    -> the output is the gathered integers."""
    from hqmq.kernels import decode_dequant
    B, H, T, d_head, S = 1, 1, 4, 8, 4
    K, r_qmax = 24 * S, 15
    torch.manual_seed(0)
    idx = torch.randint(0, K, (B, H, T, d_head // 4), dtype=torch.int32, device=DEV)
    rq = torch.full((B, H, T, d_head // 4), r_qmax, dtype=torch.int32, device=DEV)
    rs = torch.ones((B, H, T), dtype=torch.float32, device=DEV)
    joint = torch.arange(H * K * 4, dtype=torch.float32, device=DEV).view(H, K, 4)
    out = decode_dequant(idx, rq, rs, joint, r_qmax)
    want = joint[0][idx.long().view(-1)].view(B, H, T, d_head)
    assert torch.equal(out, want)


# ---------------------------------------------------------------- packed planes
@pytest.mark.parametrize("S,b_r", CODEBOOKS)
@pytest.mark.parametrize("dn,d_h", [("fp16", 128), ("bf16", 64), ("fp32", 32)])
def test_packed_planes_match_oracle(S, b_r, dn, d_h):
    import hqmq
    ops, dt = _ops(), DT[dn]
    B, H, T = 2, 2, 70
    q = hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=S, radius_bits=b_r, device=DEV, seed=5)
    k = kv_input((B, H, T, d_h), dt, seed=S + d_h)
    v = kv_input((B, H, T, d_h), dt, seed=S + d_h + 1)
    cache = q.new_cache(B, T, d_h, dt, layer_idx=0)
    q.append(cache, k[:, :, :41].to(DEV), v[:, :, :41].to(DEV), 0)       # two appends, the second mid-tile
    q.append(cache, k[:, :, 41:].to(DEV), v[:, :, 41:].to(DEV), 0)
    assert cache.length == T and cache.K.t_cap % 64 == 0
    for pt, x, kv in ((cache.K, k, 0), (cache.V, v, 1)):
        Jc = CO.joint_table(TO.secondary_raw(1, H, S, 5)[0, :, kv], dt)
        want = CO.quantize(x, Jc, b_r)
        main, aux = CO.pack_rows(want["idx"], want["rq"], pt.idx_bits, pt.main_bits, pt.aux_bits)
        assert torch.equal(pt.main[:, :, :T].cpu(), main)
        if aux is not None:
            assert torch.equal(pt.aux[:, :, :T].cpu(), aux)
        assert bit_equal(pt.scale[:, :, :T], want["r_max"])
        assert int(pt.main[:, :, T:].abs().sum()) == 0                    # rows past the end stay untouched
        # dense decode of the planes: both roundings
        assert bit_equal(ops.dequant_packed(pt, T, mode=1), want["out"])
        assert bit_equal(ops.dequant_packed(pt, T, mode=0), CO.dequant(want["idx"], want["rq"], want["r_max"], Jc, pt.qmax))
        # codes packed from the unpacked representation give the same bytes
        pt2 = q.new_cache(B, T, d_h, dt, 0).K
        ops.pack_codes(want["idx"].to(DEV), want["rq"].to(DEV), pt2)
        assert torch.equal(pt2.main.cpu(), pt.main.cpu()) and (aux is None or torch.equal(pt2.aux.cpu(), pt.aux.cpu()))
    per_token = cache.K.row_bytes()
    assert per_token == {(24, 128): 54, (96, 128): 66, (192, 128): 78}.get((S, d_h), per_token)


def test_ragged_append_with_positions():
    """Per-sequence positions: each sequence's new token lands on its own row."""
    import hqmq
    dt = torch.bfloat16
    B, H, d_h = 3, 2, 128
    q = hqmq.HQMQ(n_layers=1, n_heads=H, secondary_size=24, radius_bits=3, device=DEV)
    cache = q.new_cache(B, 64, d_h, dt, 0)
    pos = torch.tensor([5, 0, 40], dtype=torch.int32, device=DEV)
    k = kv_input((B, H, 2, d_h), dt, seed=1)
    v = kv_input((B, H, 2, d_h), dt, seed=2)
    q.append(cache, k.to(DEV), v.to(DEV), 0, pos=pos)
    want = CO.quantize(k, CO.joint_table(TO.secondary_raw(1, H, 24, 42)[0, :, 0], dt), 3)
    main, aux = CO.pack_rows(want["idx"], want["rq"], cache.K.idx_bits, cache.K.main_bits, cache.K.aux_bits)
    for b, p in enumerate(pos.tolist()):
        assert torch.equal(cache.K.main[b, :, p:p + 2].cpu(), main[b])
        assert torch.equal(cache.K.aux[b, :, p:p + 2].cpu(), aux[b])
        assert bit_equal(cache.K.scale[b, :, p:p + 2], want["r_max"][b])
        untouched = torch.ones(64, dtype=torch.bool)
        untouched[p:p + 2] = False
        assert int(cache.K.main[b][:, untouched].abs().sum()) == 0


@pytest.mark.parametrize("S,b_r", [(24, 3), (24, 4), (7, 2), (96, 4), (96, 3), (96, 6), (192, 6), (192, 4), (300, 5)])
@pytest.mark.parametrize("d_h", [16, 20, 80, 128, 160, 256])
def test_packed_planes_of_every_layout_and_head_size(S, b_r, d_h):
    """The planes a quantize call packs, read back by the independent bit reader of tests/helpers.py, hold the codes,
    flags and scales the same call returns: every width the layout rule produces (8 / 12 / 16 bits in the main plane,
    0 - 4 in the aux plane), head sizes whose lanes do and do not sit side by side in a wavefront (n = 4 ... 64, with
    20 and 40 not powers of two), one-token, short and bulk calls, with and without Med3x, and the filter search
    against the exhaustive scan (algo = 1) on the same input."""
    from hqmq_amd.packed import PackedTensor
    from tests.helpers import unpack_planes
    ops = _ops()
    g = torch.Generator().manual_seed(1000 * S + 10 * d_h + b_r)
    H, n = 2, d_h // 4
    for dn in ("fp16", "bf16"):
        dt = DT[dn]
        J, slack = ops.build_joint(torch.randn(H, S, 4, generator=g).to(DEV), dt)
        for B, T, outl in ((2, 1, True), (1, 5, False), (2, 70, True)):
            if outl and n > 32:
                continue                                                     # the sideband takes at most 32 chunks per token
            spread = torch.exp(torch.randn(B, H, T, n, 1, generator=g)).expand(B, H, T, n, 4).reshape(B, H, T, d_h)
            x = (torch.randn(B, H, T, d_h, generator=g) * spread).to(dt).to(DEV)
            pt = PackedTensor(B, H, T, d_h, S, b_r, dt, DEV, joint=J, outliers=outl)
            thr = ops.med3x_threshold(x, 3.0)[1] if outl else None
            r = ops.quantize(x, J, slack, b_r, want_codes=True, thr=thr, want_mask=outl, cache=pt, t_off=0)
            scan = ops.quantize(x, J, slack, b_r, want_codes=True, algo=1)
            assert torch.equal(r["idx"], scan["idx"]) and torch.equal(r["rq"], scan["rq"]), (dn, B, T)
            for b in range(B):
                idx, rq, flags = unpack_planes(pt, b, T)
                want_rq = r["rq"][b].long()
                if outl:
                    assert torch.equal(flags, r["mask"][b].bool()), (dn, B, T, "flags")
                    want_rq = torch.where(r["mask"][b].bool(), torch.zeros_like(want_rq), want_rq)   # flagged: radius code 0
                assert torch.equal(idx, r["idx"][b].long()) and torch.equal(rq, want_rq), (dn, B, T, "codes")
                assert bit_equal(pt.scale[b, :, :T], r["r_max"][b]), (dn, B, T, "scales")
