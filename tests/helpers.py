"""Shared test helpers: bit-exact comparison, fixture decoding, seeded inputs."""
import numpy as np
import torch

DT = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


def as_bits(t: torch.Tensor) -> torch.Tensor:
    t = t.detach().cpu().contiguous()
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def bit_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Same NaN positions and identical bit patterns everywhere else."""
    a, b = a.detach().cpu(), b.detach().cpu()
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    na, nb = torch.isnan(a.float()), torch.isnan(b.float())
    return bool(torch.equal(na, nb) and torch.equal(as_bits(a)[~na], as_bits(b)[~nb]))


def unbits(a: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).view(dtype)


def kv_input(shape, dtype, seed, lognormal=True, outlier_p=0.0, outlier_gain=(50.0, 200.0)):
    """Seeded K/V-like tensor: N(0,1), optional per-channel lognormal(0, 0.5) scale and planted outlier chunks."""
    g = torch.Generator().manual_seed(seed)
    B, H, T, d = shape
    x = torch.randn(B, H, T, d, generator=g)
    if lognormal:
        x = x * torch.exp(0.5 * torch.randn(B, H, 1, d, generator=g))
    if outlier_p > 0:
        n = d // 4
        hit = torch.rand(B, H, T, n, generator=g) < outlier_p
        gain = outlier_gain[0] + (outlier_gain[1] - outlier_gain[0]) * torch.rand(B, H, T, n, 1, generator=g)
        x = torch.where(hit.unsqueeze(-1), x.view(B, H, T, n, 4) * gain, x.view(B, H, T, n, 4)).reshape(B, H, T, d)
    return x.to(dtype)


def attn_tolerance(ref: torch.Tensor, dtype: torch.dtype, base: float = 2e-3) -> torch.Tensor:
    """Element-wise bound: `base` absolute (the stated 2e-3; 1e-3 for fp32 as in the reference's own test)
    plus (4 * eps_D + 4 * 2^-11) * |ref|.  The relative term matters only for outputs well above 1 (a peaked
    softmax over outlier values, where a bf16 result cannot even represent 2e-3): the dense K/V the oracle
    attends over carries three roundings to the cache dtype D per element and the output a fourth
    (eps_D = largest relative rounding error: 2^-11 fp16, 2^-8 bf16, 0 fp32), which a kernel that decodes
    in registers does not reproduce; the kernel itself multiplies in fp16 (2^-11 per product)."""
    eps_d = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    return base + (4.0 * eps_d + 4.0 * 2.0 ** -11) * ref.abs()


def read_bits(row: np.ndarray, bitpos: int, nbits: int) -> int:
    """Python reader of the packed little-endian bit stream (independent of the C and HIP packers)."""
    v = 0
    for i in range(nbits):
        p = bitpos + i
        v |= ((int(row[p >> 3]) >> (p & 7)) & 1) << i
    return v


def dense_from_codes(r: dict, J: torch.Tensor, qmax: int, x: torch.Tensor = None, exact: bool = False) -> torch.Tensor:
    """Oracle codes (idx, rq, r_max[, mask]) -> dense (B, H, T, 4n) cache on the CPU.

    exact=False: the reference's decode in the cache dtype (three roundings per element);
    exact=True:  the same product in float64, returned as fp32 (no rounding to the cache dtype).
    Flagged chunks (r["mask"]) are taken verbatim from x."""
    from oracle import c_oracle as CO
    idx, rq, rs = r["idx"], r["rq"], r["r_max"]
    B, H, T, n = idx.shape
    if exact:
        cw = torch.stack([J[h].double()[idx[:, h].long()] for h in range(H)], dim=1)       # (B, H, T, n, 4)
        rad = rq.double() * rs.double().unsqueeze(-1) / qmax
        d = (cw * rad.unsqueeze(-1)).float()
        d = torch.nan_to_num(d, nan=0.0)
    else:
        d = CO.dequant(idx, rq, rs, J, qmax).view(B, H, T, n, 4)
    if r.get("mask") is not None and x is not None:
        d = torch.where(r["mask"].unsqueeze(-1), x.view(B, H, T, n, 4).to(d.dtype), d)
    return d.reshape(B, H, T, 4 * n)


def attention_refs(Q, K_D, V_D, K_x, V_x, **kw):
    """(reference output over the D-rounded cache, output over the unrounded cache, attention-weighted |V|),
    all fp32 on the CPU with double accumulation."""
    from oracle import c_oracle as CO
    ref_d = CO.attention_dense(Q, K_D, V_D, **kw)
    ref_x = CO.attention_dense(Q.float(), K_x, V_x, **kw)
    a_abs = CO.attention_dense(Q.float(), K_x, V_x.abs(), **kw)
    return ref_d, ref_x, a_abs


def assert_attention_close(got, ref_d, ref_x, a_abs, base=2e-3, what=""):
    """The kernel decodes K and V in registers (fp16 products, fp32 accumulation) and never rounds them
    to the cache dtype, so it is held to: within `base` + fp16 noise (8 * 2^-11 of the attention-weighted
    |V|) of exact arithmetic on the codes, and no further from the reference's output than that plus the
    reference's own rounding spread |ref_d - ref_x|.  For diffuse attention (every long-context decode
    shape) both reduce to the plain `base` = 2e-3."""
    got = got.float().cpu()
    noise = base + 8.0 * 2.0 ** -11 * a_abs
    e_x = (got - ref_x).abs()
    e_d = (got - ref_d).abs()
    spread = (ref_d - ref_x).abs()
    w1 = float((e_x - noise).max())
    w2 = float((e_d - noise - spread).max())
    assert w1 <= 0 and w2 <= 0, (f"{what}: |O - exact| max {float(e_x.max()):.3e} (over by {w1:.3e}), "
                                 f"|O - ref| max {float(e_d.max()):.3e} (over by {w2:.3e}), "
                                 f"reference rounding spread max {float(spread.max()):.3e}")
    return float(e_d.max())


def unpack_planes(pt, b: int, L: int):
    """Independent reader (plain torch ops, on the cache's device) of rows [0, L) of sequence b of a PackedTensor:
    (idx, rq) int64 of shape (H, L, n) and the flag bits as a bool tensor of the same shape (None without Med3x).
    Little-endian bit streams: main_bits per code in the main row, the remaining aux_bits in the aux row."""
    n, ib, mb, ab = pt.n, pt.idx_bits, pt.main_bits, pt.aux_bits
    dev = pt.main.device

    def fields(plane, width):
        H = plane.shape[0]
        bit = (plane.unsqueeze(-1).to(torch.int32) >> torch.arange(8, device=dev, dtype=torch.int32)) & 1
        bit = bit.reshape(H, L, -1)[..., :n * width].reshape(H, L, n, width).to(torch.int64)
        return (bit << torch.arange(width, device=dev)).sum(-1)

    code = fields(pt.main[b, :, :L], mb)
    if ab:
        code = code | (fields(pt.aux[b, :, :L], ab) << mb)
    flags = fields(pt.flags[b, :, :L], 1).bool() if pt.flags is not None else None
    return code & ((1 << ib) - 1), code >> ib, flags


def exact_dense(pt, b: int, L: int, x=None) -> torch.Tensor:
    """fp32 (H, L, d_h) decode of sequence b without any rounding to the cache dtype: joint[idx] * (rq * rs / qmax),
    flagged chunks verbatim from x (H, L, d_h), the tensor that was quantized."""
    idx, rq, flags = unpack_planes(pt, b, L)
    H, n = pt.H, pt.n
    J = pt.joint.float()
    cw = torch.stack([J[h][idx[h]] for h in range(H)])                              # (H, L, n, 4)
    rad = rq.float() * pt.scale[b, :, :L].float().unsqueeze(-1) / float(pt.qmax)
    d = cw * rad.unsqueeze(-1)
    if flags is not None:
        assert x is not None
        d = torch.where(flags.unsqueeze(-1), x.float().view(H, L, n, 4), d)
    return d.reshape(H, L, 4 * n)


def gpu_attention_refs(Qb, K_D, V_D, K_x, V_x):
    """One sequence, decode: Qb (H_q, d), dense caches (H_kv, L, d).  Returns (ref over the D-rounded cache, ref over
    the unrounded cache, attention-weighted |V|), fp32 on the GPU (softmax in float64)."""
    Hq, d = Qb.shape
    Hkv = K_D.shape[0]
    g = Hq // Hkv
    q = Qb.double().view(Hkv, g, d)

    def attend(K, V, Vabs=None):
        p = torch.softmax(torch.einsum("hgd,hkd->hgk", q, K.double()) * d ** -0.5, dim=-1)
        o = torch.einsum("hgk,hkd->hgd", p, V.double()).reshape(Hq, d).float()
        if Vabs is None:
            return o
        return o, torch.einsum("hgk,hkd->hgd", p, Vabs.double()).reshape(Hq, d).float()

    ref_d = attend(K_D, V_D)
    ref_x, a_abs = attend(K_x, V_x, V_x.abs())
    return ref_d, ref_x, a_abs


def masked_two_refs(cache, Q, T, mask=None):
    """The two fp32 references of assert_attention_close for a whole batch with an explicit visibility mask
    (bool, broadcastable to (B, H_q, T_q, T); None = everything visible), computed on the cache's device from the
    cache's own planes: attention over the D-rounded dense cache (what the reference attends over) and over the
    unrounded product joint[idx] * (rq * rs / qmax) read by the independent bit reader (flagged chunks verbatim in
    both).  Returns (ref_d, ref_x, attention-weighted |V|), each (B, H_q, T_q, d_h); softmax in float64; rows without a
    visible token give 0."""
    from hqmq_amd import ops
    B, Hq, Tq, d = Q.shape
    Hkv = cache.K.H
    g = Hq // Hkv
    K_D, V_D = ops.dequant_packed(cache.K, T, 0), ops.dequant_packed(cache.V, T, 0)
    outs = ([], [], [])
    for b in range(B):
        K_x, V_x = exact_dense(cache.K, b, T, K_D[b]), exact_dense(cache.V, b, T, V_D[b])
        q = Q[b].double().view(Hkv, g, Tq, d)
        mb = None
        if mask is not None:
            mb = mask.expand(B, Hq, Tq, T)[b].view(Hkv, g, Tq, T)

        def attend(K, V, Vabs=None):
            s = torch.einsum("hgqd,hkd->hgqk", q, K.double()) * d ** -0.5
            if mb is not None:
                s = s.masked_fill(~mb, float("-inf"))
            p = torch.nan_to_num(torch.softmax(s, dim=-1))
            o = torch.einsum("hgqk,hkd->hgqd", p, V.double()).reshape(Hq, Tq, d).float()
            if Vabs is None:
                return o
            return o, torch.einsum("hgqk,hkd->hgqd", p, Vabs.double()).reshape(Hq, Tq, d).float()

        outs[0].append(attend(K_D[b], V_D[b]))
        rx, ab = attend(K_x, V_x, V_x.abs())
        outs[1].append(rx)
        outs[2].append(ab)
    return tuple(torch.stack(o).cpu() for o in outs)
