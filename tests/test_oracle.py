"""Pins the two CPU oracles: against the reference's own outputs (golden fixtures), against each
other, and against what the mathematics fixes.  CPU only."""
import itertools

import numpy as np
import pytest
import torch

from oracle import c_oracle as CO
from oracle import torch_oracle as TO
from tests.helpers import DT, bit_equal, read_bits, unbits

ORACLES = [("torch", TO), ("c", CO)]


# ---------------------------------------------------------------- known answers the reference itself tests
@pytest.mark.parametrize("name,orc", ORACLES)
def test_24cell_known_answers(name, orc):
    """Reference tests/test_smoke.py:54-91: 24 unit vectors, max off-diagonal cosine 0.5, closed under quat_mul."""
    pts = orc.cell24().float()
    assert pts.shape == (24, 4)
    assert torch.allclose(pts.norm(dim=-1), torch.ones(24), atol=1e-6)
    cos = pts @ pts.T
    cos.fill_diagonal_(-2)
    assert abs(cos.max().item() - 0.5) < 1e-4
    pts_set = {tuple(round(float(v), 5) for v in p) for p in pts}
    for i, j in itertools.product(range(24), range(24)):
        if name == "torch":
            prod = TO.quat_mul(pts[i], pts[j])
        else:
            prod = CO.quat_mul(pts[i], pts[j], torch.float32)
        assert tuple(round(float(v), 5) for v in prod) in pts_set


def test_24cell_order_defines_index():
    """p < 8: axis p//2, + for even p; p >= 8: bit (3-j) of p-8 set -> component j is -1/2."""
    a, b = TO.cell24(), CO.cell24()
    assert torch.equal(a, b)
    assert a[0].tolist() == [1, 0, 0, 0] and a[1].tolist() == [-1, 0, 0, 0] and a[7].tolist() == [0, 0, 0, -1]
    assert a[8].tolist() == [.5, .5, .5, .5] and a[9].tolist() == [.5, .5, .5, -.5] and a[23].tolist() == [-.5] * 4


def test_quat_mul_textbook():
    """i*j = k, j*k = i, k*i = j, i*i = -1; norm multiplicative."""
    e = torch.eye(4)
    one, i, j, k = e[0], e[1], e[2], e[3]
    for (x, y, z) in ((i, j, k), (j, k, i), (k, i, j)):
        assert torch.equal(TO.quat_mul(x, y), z) and torch.equal(CO.quat_mul(x, y, torch.float32), z)
        assert torch.equal(TO.quat_mul(y, x), -z)
    assert torch.equal(TO.quat_mul(i, i), -one)
    g = torch.Generator().manual_seed(0)
    a, b = torch.randn(100, 4, generator=g).double(), torch.randn(100, 4, generator=g).double()
    assert torch.allclose(TO.quat_mul(a, b).norm(dim=-1), a.norm(dim=-1) * b.norm(dim=-1), atol=1e-12)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_c_converters_match_torch(dtype):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(100000, generator=g) * torch.exp(6 * torch.randn(100000, generator=g))
    x = torch.cat([x, torch.tensor([0., -0., 65504., 65519.9, 65520., 1e-8, 2.98e-8, 2.9802322e-8, 5.96e-8, 6e-5,
                                    6.1e-5, float("inf"), -float("inf"), 1e30, 3.4e38])])
    assert torch.equal(CO.round_array(x, dtype), x.to(dtype).float())


# ---------------------------------------------------------------- golden fixtures written from the reference
@pytest.mark.parametrize("name,orc", ORACLES)
def test_quantizer_golden(name, orc, golden_dir):
    """joint table and quantize_K/V output identical, bit for bit, to the reference's (incl. NaN positions)."""
    g = np.load(golden_dir / "quantizer.npz")
    for cfg in ("s24r3", "s96r4", "s192r6"):
        S, b_r, seed, L, H = (int(v) for v in g[cfg + "_meta"])
        raw = torch.from_numpy(g[cfg + "_raw"])
        assert torch.equal(raw, TO.secondary_raw(L, H, S, seed))
        for dn, dt in DT.items():
            for kv, tag in ((0, "K"), (1, "V")):
                key = f"{cfg}_{dn}_{tag}"
                x = unbits(g[key + "_x"], dt)
                J = orc.joint_table(raw[1, :, kv], dt)
                assert bit_equal(J, unbits(g[key + "_joint"], dt)), key
                out = orc.quantize(x, J, b_r)["out"]
                assert bit_equal(out, unbits(g[key + "_out"], dt)), key


@pytest.mark.parametrize("name,orc", ORACLES)
def test_outlier_golden(name, orc, golden_dir):
    g = np.load(golden_dir / "outlier.npz")
    for cfg in ("s24r3", "s96r4"):
        S, b_r, seed, L, H = (int(v) for v in g[cfg + "_meta"])
        raw = torch.from_numpy(g[cfg + "_raw"])
        for dn, dt in DT.items():
            rates = []
            for kv, tag in ((0, "K"), (1, "V")):
                key = f"{cfg}_{dn}_{tag}"
                x = unbits(g[key + "_x"], dt)
                r = orc.outlier_quantize(x, orc.joint_table(raw[0, :, kv], dt), b_r, 3.0)
                assert bit_equal(r["out"], unbits(g[key + "_out"], dt)), key
                rates.append(float(r["mask"].float().mean()))
            ref_rate = g[f"{cfg}_{dn}_rate"]
            assert abs(np.mean(rates) - ref_rate[0]) < 1e-6 and ref_rate[1] == 2


ATTN_CASES = ("sq_fp32", "gqa_dec_fp16", "gqa_dec_bf16", "rect_causal_fp16", "rect_full_fp32")


def load_attn_case(g, name):
    B, Hq, Hkv, Tq, Tkv, d_h, S, qmax, causal = (int(v) for v in g[name + "_meta"])
    dt = DT[str(g[name + "_dtype"])]
    t = {}
    for tag in ("K", "V"):
        t[tag + "_idx"] = torch.from_numpy(g[f"{name}_{tag}_idx"])
        t[tag + "_rq"] = torch.from_numpy(g[f"{name}_{tag}_rq"])
        t[tag + "_rs"] = unbits(g[f"{name}_{tag}_rs"], dt)
        t[tag + "_joint"] = unbits(g[f"{name}_{tag}_joint"], dt)
    t.update(Q=unbits(g[name + "_Q"], dt), O=unbits(g[name + "_O"], dt), Kdense=unbits(g[name + "_Kdense"], dt))
    return dict(B=B, Hq=Hq, Hkv=Hkv, Tq=Tq, Tkv=Tkv, d_h=d_h, S=S, qmax=qmax, causal=bool(causal), dtype=dt), t


@pytest.mark.parametrize("case", ATTN_CASES)
def test_attention_golden(case, golden_dir):
    g = np.load(golden_dir / "attention.npz")
    m, t = load_attn_case(g, case)
    # dense decode: both oracles bit-exact against the reference
    assert bit_equal(TO.decode_kv(t["K_idx"], t["K_rq"], t["K_rs"], t["K_joint"], m["qmax"]), t["Kdense"])
    assert bit_equal(CO.dequant(t["K_idx"], t["K_rq"], t["K_rs"], t["K_joint"], m["qmax"]), t["Kdense"])
    # attention: torch oracle is the same library routine -> bit-exact; C oracle (double) within the dtype's rounding
    O = TO.attention(t["Q"], t["K_idx"], t["K_rq"], t["K_rs"], t["K_joint"], t["V_idx"], t["V_rq"], t["V_rs"],
                     t["V_joint"], m["qmax"], m["causal"])
    assert bit_equal(O, t["O"])
    Vd = CO.dequant(t["V_idx"], t["V_rq"], t["V_rs"], t["V_joint"], m["qmax"])
    Oc = CO.attention_dense(t["Q"], t["Kdense"], Vd, causal=m["causal"])
    tol = {torch.float32: 2e-6, torch.float16: 1.5e-3, torch.bfloat16: 1.2e-2}[m["dtype"]]
    assert (Oc - t["O"].float()).abs().max().item() < tol


# ---------------------------------------------------------------- the two oracles against each other
@pytest.mark.parametrize("S,b_r", [(24, 3), (96, 4), (192, 6), (1, 2)])
@pytest.mark.parametrize("dn", ["fp32", "fp16", "bf16"])
def test_c_matches_torch(S, b_r, dn):
    dt = DT[dn]
    raw = TO.secondary_raw(1, 3, S, 5)[0, :, 0]
    J, Jc = TO.joint_table(raw, dt), CO.joint_table(raw, dt)
    assert bit_equal(J, Jc)
    g = torch.Generator().manual_seed(S)
    x = (torch.randn(2, 3, 40, 64, generator=g) * torch.exp(0.5 * torch.randn(2, 3, 1, 64, generator=g))).to(dt)
    x[0, 0, 3, 8:12] = 0
    x[1, 1, 5, :] = 0
    x[0, 2, 7, 0:4] *= 100
    x[1, 0, 9, 4:8] = torch.tensor([1., 0, 0, 0]).to(dt)
    x[0, 1, 11, :8] = torch.tensor([3e-8, 0, 0, 0, 1e-7, 1e-7, 0, 0]).to(dt)
    a, c = TO.quantize(x, J, b_r), CO.quantize(x, J, b_r)
    assert torch.equal(a["idx"], c["idx"]) and torch.equal(a["rq"], c["rq"])
    for k in ("rq_f", "r_max", "out"):
        assert bit_equal(a[k], c[k]), k
    hit = torch.rand(2, 3, 40, 16, generator=g) < 0.04
    xo = torch.where(hit.unsqueeze(-1), x.view(2, 3, 40, 16, 4) * 120, x.view(2, 3, 40, 16, 4)).reshape(2, 3, 40, 64)
    a, c = TO.outlier_quantize(xo, J, b_r), CO.outlier_quantize(xo, J, b_r)
    assert torch.equal(a["median"], c["median"]) and bit_equal(a["threshold"], c["threshold"])
    assert torch.equal(a["mask"], c["mask"]) and bit_equal(a["norms"], c["norms"]) and bit_equal(a["out"], c["out"])
    odd = xo[:1, :, :5, :12].contiguous()   # odd count per head: the median is the middle element
    a, c = TO.med3x(odd), CO.med3x(odd)
    assert torch.equal(a["median"], c["median"]) and torch.equal(a["mask"], c["mask"])


# ---------------------------------------------------------------- what the mathematics fixes
@pytest.mark.parametrize("dn", ["fp32", "fp16", "bf16"])
def test_joint_table_invariants(dn):
    dt = DT[dn]
    S = 7
    raw = TO.secondary_raw(1, 2, S, 3)[0, :, 1]
    J = CO.joint_table(raw, dt).float().view(2, 24, S, 4)
    sec = (raw / raw.norm(dim=-1, keepdim=True)).to(dt).float()
    assert torch.equal(J[:, 0], sec)                                  # p = 0 is the identity: rows k = s are q_s
    assert torch.equal(J[:, 1], -sec)                                 # p = 1 is -1
    for p in range(2, 8):                                             # axis units: signed permutations, exact
        assert torch.equal(J[:, p].abs().sort(dim=-1).values, sec.abs().sort(dim=-1).values)
    assert (J.norm(dim=-1) - 1).abs().max() < {torch.float32: 1e-6, torch.float16: 3e-3, torch.bfloat16: 2e-2}[dt]
    exact = TO.quat_mul(TO.cell24().double().view(1, 24, 1, 4), sec.double().view(2, 1, S, 4))
    assert (J.double() - exact).abs().max() < {torch.float32: 3e-7, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dt]


@pytest.mark.parametrize("dn", ["fp32", "fp16", "bf16"])
def test_argmax_properties_bruteforce(dn):
    """idx maximises the rounded similarity and is the first index that does (pure-Python scan)."""
    dt = DT[dn]
    raw = TO.secondary_raw(1, 1, 5, 9)[0, :, 0]
    J = CO.joint_table(raw, dt)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 1, 6, 8, generator=g).to(dt)
    r = CO.quantize(x, J, 3)
    xc = x.view(6, 2, 4)
    rad = xc.norm(dim=-1, keepdim=True).clamp(min=1e-8)
    u = (xc / rad).float()
    Jf = J[0].float()
    for t in range(6):
        for c in range(2):
            sims = [float(torch.tensor(sum(float(u[t, c, j]) * float(Jf[k, j]) for j in range(4))).to(dt)) for k in range(120)]
            k_star = int(r["idx"][0, 0, t, c])
            best = max(sims)
            # the double-precision sum may differ from the fp32 chain by less than one rounding step
            assert sims[k_star] >= best - 2 * float(torch.finfo(dt).eps) * abs(best)


def test_single_secondary_reduces_to_nearest_24cell_vertex():
    """S = 1 with q_s = 1: the codeword is the nearest 24-cell vertex, whose similarity has the closed
    form max(max_i |u_i|, sum_i |u_i| / 2)."""
    raw = torch.tensor([[[2.0, 0, 0, 0]]])
    J = CO.joint_table(raw, torch.float32)
    assert torch.equal(J[0], CO.cell24())
    g = torch.Generator().manual_seed(4)
    x = torch.randn(1, 1, 500, 4, generator=g)
    r = CO.quantize(x, J, 4)
    u = x.view(500, 4) / x.view(500, 4).norm(dim=-1, keepdim=True)
    closed = torch.maximum(u.abs().max(dim=-1).values, u.abs().sum(dim=-1) / 2)
    got = (u * J[0][r["idx"].view(500).long()]).sum(-1)
    assert torch.allclose(got, closed, atol=1e-6)


@pytest.mark.parametrize("dn", ["fp16", "bf16", "fp32"])
def test_radius_code_invariants(dn):
    dt = DT[dn]
    raw = TO.secondary_raw(1, 2, 24, 1)[0, :, 0]
    J = CO.joint_table(raw, dt)
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(2, 2, 50, 32, generator=g) * 3).to(dt)
    for b_r in (3, 4, 6):
        qmax = (1 << b_r) - 1
        r = CO.quantize(x, J, b_r)
        assert int(r["rq"].min()) >= 0 and int(r["rq"].max()) == qmax
        assert torch.equal(r["rq"].amax(dim=-1), torch.full((2, 2, 50), qmax, dtype=torch.int32))  # the max chunk gets qmax
        assert bit_equal(r["r_max"], x.view(2, 2, 50, 8, 4).norm(dim=-1).amax(dim=-1))


def test_median_is_sort_midpoint():
    g = torch.Generator().manual_seed(6)
    for T in (7, 8):      # odd and even chunk counts
        x = torch.randn(1, 2, T, 12, generator=g).half()
        m = CO.med3x(x)
        norms = x.view(1, 2, T, 3, 4).norm(dim=-1).permute(1, 0, 2, 3).reshape(2, -1).float()
        s = norms.sort(dim=-1).values
        N = s.shape[1]
        mid = (s[:, (N - 1) // 2] + s[:, N // 2]) * 0.5
        assert torch.allclose(m["median"], mid, rtol=0, atol=0)
        thr = (m["median"] * 3.0).half()
        assert torch.equal(m["mask"], x.view(1, 2, T, 3, 4).norm(dim=-1) > thr.view(1, 2, 1, 1))


def test_zero_chunk_and_zero_token_semantics():
    """fp16: clamp(min=1e-8) is a no-op, a zero chunk has a NaN direction -> index 0; a zero token has scale 0 -> NaN out.
    bf16: the clamp yields 1.0012e-8, directions are 0 -> index 0, output is finite."""
    raw = TO.secondary_raw(1, 1, 24, 0)[0, :, 0]
    x = torch.randn(1, 1, 3, 16, generator=torch.Generator().manual_seed(7))
    x[0, 0, 0, 4:8] = 0
    x[0, 0, 1, :] = 0
    for dt, nan_rows in ((torch.float16, True), (torch.bfloat16, False)):
        J = CO.joint_table(raw, dt)
        a, c = TO.quantize(x.to(dt), J, 3), CO.quantize(x.to(dt), J, 3)
        assert int(c["idx"][0, 0, 0, 1]) == 0 and torch.equal(c["idx"][0, 0, 1], torch.zeros(4, dtype=torch.int32))
        assert bool(torch.isnan(c["out"][0, 0, 1].float()).all()) == nan_rows
        assert bit_equal(a["out"], c["out"]) and torch.equal(a["idx"], c["idx"])


# ---------------------------------------------------------------- packed layout (this build's own format)
@pytest.mark.parametrize("ib,mb,ab,n", [(10, 12, 1, 32), (12, 16, 0, 32), (13, 16, 3, 32), (12, 16, 0, 16), (10, 12, 1, 8)])
def test_pack_rows_round_trip(ib, mb, ab, n):
    g = torch.Generator().manual_seed(n + ib)
    rb = mb + ab - ib
    idx = torch.randint(0, 1 << ib, (3, 5, n), generator=g, dtype=torch.int32)
    rq = torch.randint(0, 1 << rb, (3, 5, n), generator=g, dtype=torch.int32)
    main, aux = CO.pack_rows(idx, rq, ib, mb, ab)
    assert main.shape[-1] == n * mb // 8 and (aux is None) == (ab == 0)
    for r, t in itertools.product(range(3), range(5)):
        for c in range(n):
            code = read_bits(main[r, t].numpy(), c * mb, mb)
            if ab:
                code |= read_bits(aux[r, t].numpy(), c * ab, ab) << mb
            assert code == int(idx[r, t, c]) | (int(rq[r, t, c]) << ib)


def test_pack_flags_and_sideband():
    g = torch.Generator().manual_seed(8)
    T, n = 37, 16
    x = torch.randn(T, 4 * n, generator=g).half()
    mask = torch.rand(T, n, generator=g) < 0.1
    flags = CO.pack_flags(mask)
    for t in range(T):
        for c in range(n):
            assert read_bits(flags[t].numpy(), c, 1) == int(mask[t, c])
    sb, toff, cnt = CO.pack_sideband(x, mask)
    assert cnt == int(mask.sum()) and torch.equal(sb, x.view(T, n, 4)[mask])
    for i in range(toff.numel()):
        assert int(toff[i]) == int(mask[:16 * i].sum())
