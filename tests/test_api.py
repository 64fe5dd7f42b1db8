"""CPU-side checks: public API surface (mirrors the reference's tests/test_smoke.py), host logic,
and that the C-ABI library loads and exports every symbol the header declares."""
import ctypes as C
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent


def test_import_and_version():
    import hqmq
    assert hqmq.__version__ == "0.1.0"


def test_public_api_surface():
    import hqmq
    for name in ["HQMQ", "PaddedHQMQ", "OutlierAwareHQMQQuantizer", "OutlierAwareGenericQuantizer", "fused_attention",
                 "fused_attention_reference", "with_outlier_extraction", "device_info", "kernels_ada", "kernels_hopper",
                 "kernels_blackwell", "fused_attention_packed", "PackedKV"]:
        assert hasattr(hqmq, name), name


def test_kernels_submodule():
    from hqmq import kernels
    for name in ["fused_attention_ada", "fused_attention_hopper", "fused_attention_blackwell", "fused_attention_reference",
                 "decode_dequant", "encode_joint_fp8", "hopper_available", "blackwell_available"]:
        assert hasattr(kernels, name), name
    assert kernels.hopper_available() is False and kernels.blackwell_available() is False


def test_reference_import_paths():
    from src.quantizers.hqmq import HQMQQuantizer, quat_mul
    from src.quantizers.spherical import _make_24cell_codebook
    from src.quantizers.outlier_aware import OutlierAwareHQMQQuantizer
    from src.quantizers.outlier_generic import OutlierAwareGenericQuantizer
    from src.quantizers.hqmq_padded import PaddedHQMQQuantizer
    from src.quantizers.base import KVQuantizer
    from src.quantizers.hqmq_attention import fused_hqmq_attention_triton, fused_hqmq_attention_torch
    from src.quantizers.hqmq_kernel import hqmq_decode_triton
    from src.quantizers.hqmq_attention_hopper import fused_hqmq_attention_hopper, encode_joint_fp8, hopper_available
    from src.quantizers.hqmq_attention_blackwell import fused_hqmq_attention_blackwell, blackwell_available
    import hqmq
    assert hqmq.HQMQ is HQMQQuantizer and issubclass(HQMQQuantizer, KVQuantizer)
    assert callable(quat_mul) and callable(_make_24cell_codebook)


def test_24cell_codebook_host_mirror():
    from src.quantizers.spherical import _make_24cell_codebook
    from src.quantizers.hqmq import quat_mul
    from oracle import c_oracle as CO
    pts = _make_24cell_codebook()
    assert pts.shape == (24, 4) and torch.equal(pts, CO.cell24())
    assert torch.allclose(pts.norm(dim=-1), torch.ones(24), atol=1e-6)
    cos = pts @ pts.T
    cos.fill_diagonal_(-2)
    assert abs(cos.max().item() - 0.5) < 1e-4
    pts_set = {tuple(round(float(x), 5) for x in p) for p in pts}
    for i in range(24):
        for j in range(0, 24, 5):
            prod = quat_mul(pts[i:i + 1], pts[j:j + 1])[0]
            assert tuple(round(float(x), 5) for x in prod) in pts_set


@pytest.mark.parametrize("S,b_r,expected", [(24, 3, 3.04), (96, 4, 3.79), (192, 6, 4.54)])
def test_bits_per_value(S, b_r, expected):
    from src.quantizers.hqmq import HQMQQuantizer
    q = HQMQQuantizer(n_layers=1, n_heads=1, secondary_size=S, radius_bits=b_r, device="cpu", init="random")
    assert abs(q.bits_per_value() - expected) < 0.01


def test_construct_and_wrappers():
    import hqmq
    q = hqmq.HQMQ(n_layers=4, n_heads=2, secondary_size=24, radius_bits=3, device="cpu", init="random")
    assert q.chunk_dim == 4 and q.secondary_size == 24 and q.radius_bits == 3 and q.name == "HQMQ_s24_r3"
    assert q.secondary_raw.shape == (4, 2, 2, 24, 4) and q.secondary_raw.dtype == torch.float32
    from oracle import torch_oracle as TO
    assert torch.equal(q.secondary_raw.detach(), TO.secondary_raw(4, 2, 24, 42))      # same seeded parameters
    w = hqmq.with_outlier_extraction(q, C=3.0)
    assert w.median_mult == 3.0 and w.threshold_mode == "median_mult" and w.inner is q
    assert w.name == "OutlierMed3_HQMQ_s24_r3"
    assert abs(w.bits_per_value() - ((1 - 0.03) * q.bits_per_value() + 0.03 * 16 + 0.25)) < 1e-12
    gw = hqmq.with_outlier_extraction(q, C=3.0, generic=True)
    assert gw.chunk_dim == 4 and gw.inner is q
    p = hqmq.PaddedHQMQ(n_layers=2, n_heads=2, d_head=45, secondary_size=24, radius_bits=3, device="cpu")
    assert (p.d_head_orig, p.d_head_padded, p.pad_count) == (45, 48, 3)
    assert abs(p.bits_per_value() - q.bits_per_value() * 48 / 45) < 1e-12
    with pytest.raises(ValueError):
        hqmq.HQMQ(n_layers=1, n_heads=1, magnitude_mode="bogus", device="cpu")
    with pytest.raises(ValueError):
        hqmq.HQMQ(n_layers=1, n_heads=1, init="bogus", device="cpu")
    with pytest.raises(AssertionError):
        hqmq.OutlierAwareHQMQQuantizer(object())


def test_device_info_without_gpu():
    import hqmq
    info = hqmq.device_info()
    assert isinstance(info, dict) and "variant_auto_dispatched" in info
    if not torch.cuda.is_available():
        assert info["variant_auto_dispatched"] == "cpu"


def test_no_cpu_fallback():
    """The product path refuses CPU tensors instead of computing somewhere else."""
    import hqmq
    q = hqmq.HQMQ(n_layers=1, n_heads=2, secondary_size=24, radius_bits=3, device="cpu")
    with pytest.raises(hqmq.HqmqError):
        q.quantize_K(torch.randn(1, 2, 4, 16), 0)
    with pytest.raises(hqmq.HqmqError):
        hqmq.with_outlier_extraction(q).quantize_V(torch.randn(1, 2, 4, 16), 0)
    idx = torch.zeros(1, 1, 4, 4, dtype=torch.int32)
    with pytest.raises(hqmq.HqmqError):
        hqmq.fused_attention(torch.randn(1, 1, 4, 16), idx, idx, torch.ones(1, 1, 4), torch.randn(1, 576, 4),
                             idx, idx, torch.ones(1, 1, 4), torch.randn(1, 576, 4), r_qmax=7)
    with pytest.raises(hqmq.HqmqError):
        hqmq.kernels.decode_dequant(idx, idx, torch.ones(1, 1, 4), torch.randn(1, 576, 4), 7)


def test_unsupported_branches_raise():
    import hqmq
    for kw in (dict(jl_dim=2), dict(magnitude_mode="free"), dict(log_radius=True), dict(robust_radius_scale=True),
               dict(radius_bits=0), dict(radius_bits=16)):
        q = hqmq.HQMQ(n_layers=1, n_heads=1, device="cpu", **kw)
        with pytest.raises(NotImplementedError):
            q._check_supported()
    q = hqmq.HQMQ(n_layers=1, n_heads=1, device="cpu")
    q.set_training(True, tau=0.5)
    assert q.tau == 0.5
    with pytest.raises(NotImplementedError):
        q._check_supported()


# ---------------------------------------------------------------- C ABI
def _declared_functions():
    text = (ROOT / "include" / "hqmq_amd.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hqmq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from hqmq_amd import _lib as L
    lib = L.lib()
    names = _declared_functions()
    assert len(names) >= 14
    for name in names:
        assert hasattr(lib, name), f"{name} declared in include/hqmq_amd.h but not exported"
    assert sorted(L.EXPORTS) == names
    assert lib.hqmq_version() == 0x000200
    assert lib.hqmq_status_string(-2).decode().startswith("a size")


def test_layout_bits():
    from hqmq_amd import _lib as L
    assert L.layout_bits(24, 3) == (10, 12, 1)      # s24_r3: 13 bits per chunk
    assert L.layout_bits(96, 4) == (12, 16, 0)      # s96_r4: 16
    assert L.layout_bits(192, 6) == (13, 16, 3)     # s192_r6: 19
    assert L.layout_bits(1, 2) == (5, 8, 0)
    assert L.lib().hqmq_layout_bits(C.c_int(0), C.c_int(3), None, None, None) == -2


def test_argument_errors_are_reported_not_launched():
    """Bad arguments come back as negative statuses before any HIP call (safe without a GPU)."""
    from hqmq_amd import _lib as L
    lib = L.lib()
    assert lib.hqmq_build_joint(None, C.c_int(1), C.c_int(24), C.c_int(1), None, None, None) == -1
    a = L.QuantizeArgs()
    assert lib.hqmq_quantize(C.byref(a), None) == -1
    assert lib.hqmq_quantize(None, None) == -1
    assert lib.hqmq_attn_fwd(None, None) == -1
    ak, av = L.AppendArgs(), L.AppendArgs()
    assert lib.hqmq_append_kv(None, C.byref(av), None) == -1
    assert lib.hqmq_append_kv(C.byref(ak), C.byref(av), None) == -1      # no input, no table
    ak.median_mult = 3.0                                                # Med3x without a flag plane or a threshold output
    assert lib.hqmq_append_kv(C.byref(ak), C.byref(av), None) == -1
    assert lib.hqmq_dequant(None, *([L.i64(0)] * 3), None, *([L.i64(0)] * 3), None, *([L.i64(0)] * 3), None, L.i64(0),
                            C.c_int(1), C.c_int(1), C.c_int(1), C.c_int(1), C.c_int(1), C.c_int(1), C.c_int(1), None, None) == -1
    assert int(lib.hqmq_attn_workspace_bytes(C.c_int(1), C.c_int(32), C.c_int(1), C.c_int(128), C.c_int(64))) == 32 * 64 * 132 * 4      # (m, l, two unused, acc[128]) per split
    assert int(lib.hqmq_med3x_workspace_bytes(C.c_int(8), C.c_int(1))) == 8 * (32768 + 16) * 4
    with pytest.raises(L.HqmqError):
        L.check(-3, "x")


def test_algorithmic_bytes_per_token():
    """Row sizes of the packed layout equal the figures the roofline is priced on:
    54 / 66 / 78 bytes per (token, head, tensor) at d_h=128, 34 at d_h=64 (s96_r4), +n/8 with flags."""
    from hqmq_amd import _lib as L
    for S, b_r, d_h, want in ((24, 3, 128, 54), (96, 4, 128, 66), (192, 6, 128, 78), (96, 4, 64, 34)):
        ib, mb, ab = L.layout_bits(S, b_r)
        n = d_h // 4
        assert (n * mb + 7) // 8 + (n * ab + 7) // 8 + 2 == want
        assert n * (ib + b_r) // 8 + 2 == want


def test_memory_table_uses_packed_layout():
    """The memory table counts what the planes store: whole bits per code, scale, and with Med3x flags + sideband."""
    from hqmq_amd import memory_table as MT
    assert [MT.row_bytes(128, S, b) for S, b in MT.CONFIGS] == [54, 58, 62, 66, 70, 78]
    assert MT.row_bytes(64, 96, 4) == 34
    assert MT.row_bytes(128, 192, 6, med3x=0.02) == 78 + 4 + 0.02 * 32 * 8
    rows = MT.table()
    r = next(x for x in rows if x["model"] == "Llama-3-8B" and x["seq_len"] == 32768)
    assert r["fp16_MB"] == 2 * 32 * 8 * 32768 * 128 * 2 / 1e6
    assert abs(r["hqmq_s96_r4_MB"] - 2 * 32 * 8 * 32768 * 66 / 1e6) < 1e-9
    # never below the reference's analytic figure (fractional log2 bits), and within 8 % of it
    for S, b in MT.CONFIGS:
        k = f"hqmq_s{S}_r{b}"
        assert r[k + "_analytic_MB"] <= r[k + "_MB"] <= 1.08 * r[k + "_analytic_MB"]


def test_crop_bookkeeping_on_cpu():
    """PackedTensor.crop_ is plain torch: after a crop, the entry count and the tile offsets equal what appending
    only the kept rows would have left, and no flag stays behind in a dropped row."""
    import numpy as np
    from hqmq_amd.packed import PackedTensor, TILE
    rng = np.random.default_rng(0)
    B, H, T, d_h = 3, 2, 150, 64
    n = d_h // 4
    pt = PackedTensor(B, H, T, d_h, 96, 4, torch.float16, "cpu", outliers=True, sideband_frac=1.0)
    bits = rng.random((B, H, T, n)) < 0.07
    flags = np.zeros((B, H, pt.t_cap, n // 8), np.uint8)
    for c in range(n):
        flags[:, :, :T, c // 8] |= (bits[..., c].astype(np.uint8) << (c % 8))
    per_row = bits.sum(-1)                                             # (B, H, T)

    def state(lengths):                                                # what in-order appends of `lengths` rows leave
        off = np.full((B, H, pt.t_cap // TILE), 0x7fffffff, np.int64)
        cnt = np.zeros((B, H), np.int64)
        for b in range(B):
            for t in range(-(-lengths[b] // TILE)):
                off[b, :, t] = per_row[b, :, :t * TILE].sum(-1)
            cnt[b] = per_row[b, :, :lengths[b]].sum(-1)
        return off, cnt
    off, cnt = state([T] * B)
    pt.flags.copy_(torch.from_numpy(flags))
    pt.sb_tile_off.copy_(torch.from_numpy(off).to(torch.int32))
    pt.sb_count.copy_(torch.from_numpy(cnt).to(torch.int32))
    pt.length = T
    lens = [150, 96, 37]                                               # no-op, tile-aligned, inside a tile
    pt.crop_(torch.tensor(lens, dtype=torch.int32))
    off2, cnt2 = state(lens)
    assert np.array_equal(pt.sb_count.numpy(), cnt2) and np.array_equal(pt.sb_tile_off.numpy(), off2)
    for b in range(B):
        assert int(pt.flags[b, :, lens[b]:].sum()) == 0 and np.array_equal(pt.flags[b, :, :lens[b]].numpy(), flags[b, :, :lens[b]])
    pt.crop_(20)                                                       # an int crops every sequence
    off3, cnt3 = state([20] * B)
    assert pt.length == 20 and np.array_equal(pt.sb_count.numpy(), cnt3) and np.array_equal(pt.sb_tile_off.numpy(), off3)


def test_quantile_limit_check():
    """The reference's Med-C median is torch.quantile, which refuses more than 2^24 elements per row
    (src/quantizers/outlier_aware.py:68 of the reference); the check that mirrors it on request."""
    from hqmq_amd import ops
    assert ops.QUANTILE_LIMIT == 1 << 24
    assert ops.check_quantile_limit(1 << 24, strict=True) is True
    assert ops.check_quantile_limit((1 << 24) + 1, strict=False) is False
    with pytest.raises(RuntimeError, match="too large"):
        ops.check_quantile_limit((1 << 24) + 1, strict=True)
    x = torch.zeros(2 ** 24 + 1)
    with pytest.raises(RuntimeError, match="too large"):          # the behaviour being mirrored
        torch.quantile(x, 0.5)
