"""The reference's kernel entry points, on the HIP path.

Signatures follow src/quantizers/hqmq_attention.py:68-75,425-438,
hqmq_kernel.py:102-108, hqmq_attention_hopper.py:35-53,185-198 and
hqmq_attention_blackwell.py:50-66 of the reference.  The Triton tuning knobs
(block_q, block_kv, optimized, num_warps, num_stages) are accepted and ignored:
there is one kernel, written for gfx950.  use_fp8_codebook=True rounds the joint
tables to float8_e4m3fn, as the reference's Hopper path does (there the fp8
values are promoted to fp16 inside the kernel; here they are kept as fp16 in
LDS, which is the same arithmetic).  Extra keyword arguments (kv_lens,
causal_offset, n_splits) are additions.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F

from . import _lib as L
from . import ops
from .packed import PackedKV, PackedTensor


def decode_dequant(idx: torch.Tensor, radius_q: torch.Tensor, radius_scale: torch.Tensor, joint: torch.Tensor,
                   r_qmax: int) -> torch.Tensor:
    """(B, H, T, n) codes -> dense (B, H, T, 4n) in joint.dtype."""
    return ops.dequant(idx, radius_q, radius_scale, joint, r_qmax)


def _bits_for(r_qmax: int) -> int:
    b = max(1, int(r_qmax).bit_length())
    if b > 8:
        raise L.HqmqError(f"r_qmax={r_qmax} needs more than 8 radius bits")
    return b


def _pack_unpacked(idx, rq, rs, joint, r_qmax: int) -> PackedTensor:
    """The reference's unpacked representation -> a PackedTensor (codes packed on the GPU)."""
    B, H, T, n = idx.shape
    K = joint.shape[1]
    if joint.stride(-1) != 1 or joint.stride(1) != 4:
        joint = joint.contiguous()
    # a table of K rows is addressed like one of ceil(K/24) secondaries; the radius field holds r_qmax
    S_eff = max(1, -(-K // 24))
    rb = _bits_for(r_qmax)
    ib, mb, ab = L.layout_bits(S_eff, rb)
    if mb == 12 and (n // 4) % 2:      # a lane's share of a 12-bit row must be whole bytes: use 16-bit codes
        mb, ab = 16, max(0, ib + rb - 16)
    pt = PackedTensor(B, H, T, 4 * n, S_eff, rb, joint.dtype, idx.device, joint=joint, layout=(ib, mb, ab))
    pt.qmax = int(r_qmax)
    ops.pack_codes(idx, rq, pt)
    pt.scale[:, :, :T] = rs            # into the padded plane: rows up to the capacity stay readable
    if pt.scale_max is not None:       # the range guard of bf16 / fp32 caches: the largest finite scale, as fp32 bits
        pt.scale_max = torch.nan_to_num(rs.detach().float().abs(), nan=0.0, posinf=0.0).amax().reshape(1).view(torch.int32)
        if pt.dtype == torch.bfloat16 and not torch.cuda.is_current_stream_capturing():
            pt.refresh_range()         # one device read: bf16 scales of 2^15 and more take the guarded kernel
    pt.length = T
    return pt


def _through_fp8(joint: torch.Tensor) -> torch.Tensor:
    """The table with every entry rounded to float8_e4m3fn, in its own dtype (every e4m3 number is exact in
    fp16, bf16 and fp32)."""
    return encode_joint_fp8(joint).to(joint.dtype)


def fused_attention(
    Q: torch.Tensor,
    K_idx: torch.Tensor, K_radius_q: torch.Tensor, K_radius_scale: torch.Tensor, joint_K: torch.Tensor,
    V_idx: torch.Tensor, V_radius_q: torch.Tensor, V_radius_scale: torch.Tensor, joint_V: torch.Tensor,
    r_qmax: int,
    causal: bool = True,
    softmax_scale: Optional[float] = None,
    block_q: Optional[int] = None,
    block_kv: Optional[int] = None,
    optimized: bool = True,
    num_warps: Optional[int] = None,
    num_stages: Optional[int] = None,
    use_fp8_codebook: bool = False,
    *,
    kv_lens: Optional[torch.Tensor] = None,
    causal_offset: int = 0,
    n_splits: int = 0,
) -> torch.Tensor:
    """Fused HQMQ attention on unpacked codes; K and V are never materialised densely.

    Q (B, H_q, T_q, d_h); idx/radius_q (B, H_kv, T_kv, n) ints; radius_scale (B, H_kv, T_kv);
    joint (H_kv, K, 4).  Returns O like Q.  `causal` uses the reference's top-left alignment.
    """
    L.require_gpu(Q, "Q")
    B, H_q, T_q, d_h = Q.shape
    H_kv, T_kv, n_chunks = K_idx.shape[1], K_idx.shape[2], K_idx.shape[3]
    assert d_h == n_chunks * 4, f"d_h={d_h} != n_chunks*4={n_chunks * 4}"
    assert H_q % H_kv == 0, f"H_q={H_q} must be divisible by H_kv={H_kv}"
    if joint_K.shape[1] != joint_V.shape[1]:
        raise L.HqmqError("joint_K and joint_V must hold the same number of codewords")
    dt = joint_K.dtype
    if use_fp8_codebook:
        joint_K, joint_V = _through_fp8(joint_K), _through_fp8(joint_V)
    Qc = Q if Q.dtype == dt else Q.to(dt)
    Kc = _pack_unpacked(K_idx, K_radius_q, K_radius_scale, joint_K, r_qmax)
    Vc = _pack_unpacked(V_idx, V_radius_q, V_radius_scale, joint_V.to(dt), r_qmax)
    O = ops.attn_fwd(Qc, Kc, Vc, T_kv, kv_lens=kv_lens, causal=causal, causal_offset=causal_offset,
                     softmax_scale=softmax_scale, n_splits=n_splits)
    return O if O.dtype == Q.dtype else O.to(Q.dtype)


def fused_attention_packed(Q: torch.Tensor, cache: PackedKV, *, causal: bool = False, softmax_scale: Optional[float] = None,
                           kv_lens: Optional[torch.Tensor] = None, causal_offset: int = 0, n_splits: int = 0,
                           T_kv: Optional[int] = None, out: Optional[torch.Tensor] = None,
                           force_generic: bool = False, use_fp8_codebook: bool = False,
                           kv_starts: Optional[torch.Tensor] = None,
                           batch_order: Optional[torch.Tensor] = None,
                           fp8_table_storage: bool = False) -> torch.Tensor:
    """Fused attention straight from the bit-packed cache (the fast path).

    Decode: T_q = 1, causal=False.  Chunked prefill: causal=True with causal_offset = number of
    cached tokens before the chunk (bottom-right alignment).  Ragged batches pass kv_lens (int32 [B]);
    left-padded batches pass kv_starts (int32 [B], the first real token of every sequence).  batch_order (int32 [B],
    e.g. ops.longest_first(kv_lens)) starts the sequences' blocks in that order: scheduling only, same result.
    force_generic (True or 1) runs the layout-generic kernel where a specialised one exists (a second implementation
    of the same arithmetic, used by the tests); 2 keeps the specialised kernels that hold their tiles in registers
    where the one that lands its loads in LDS would run (plain 16+0 caches at d_h 128; same results bit for bit).  use_fp8_codebook decodes with the joint tables rounded to
    float8_e4m3fn (an accuracy/footprint experiment of the reference; the rounded tables are kept per cache);
    with fp8_table_storage=True the kernel also keeps them as float8 in LDS (half the table footprint, two
    conversions per gathered codeword; same results, 6-12 % slower on MI355X, where the decode is bound by
    vector-ALU issue and not by LDS space).
    """
    if fp8_table_storage and not use_fp8_codebook:
        raise L.HqmqError("fp8_table_storage needs use_fp8_codebook=True: only tables rounded to e4m3 can be kept as float8")
    if use_fp8_codebook:
        cache = PackedKV(cache.K.with_fp8_table(), cache.V.with_fp8_table())
    if T_kv is None:
        T_kv = cache.K.t_cap if kv_lens is not None else cache.K.length
    d, d_store = Q.shape[-1], cache.K.d_head
    if d < d_store and d == cache.K.d_head_orig:
        # a cache of zero-padded heads (PaddedHQMQ): pad Q the same way, keep the scale of the real head size
        if softmax_scale is None:
            softmax_scale = d ** -0.5
        O = ops.attn_fwd(torch.nn.functional.pad(Q, (0, d_store - d)), cache.K, cache.V, T_kv, kv_lens=kv_lens,
                         kv_starts=kv_starts, batch_order=batch_order, causal=causal,
                         causal_offset=causal_offset, softmax_scale=softmax_scale, n_splits=n_splits,
                         force_generic=force_generic)[..., :d]
        if out is not None:
            out.copy_(O)
            return out
        return O.contiguous()
    return ops.attn_fwd(Q, cache.K, cache.V, T_kv, kv_lens=kv_lens, kv_starts=kv_starts, batch_order=batch_order, causal=causal,
                        causal_offset=causal_offset, softmax_scale=softmax_scale, n_splits=n_splits, out=out,
                        force_generic=force_generic, fp8_table_storage=fp8_table_storage)


def fused_attention_reference(
    Q: torch.Tensor,
    K_idx: torch.Tensor, K_radius_q: torch.Tensor, K_radius_scale: torch.Tensor, joint_K: torch.Tensor,
    V_idx: torch.Tensor, V_radius_q: torch.Tensor, V_radius_scale: torch.Tensor, joint_V: torch.Tensor,
    r_qmax: int,
    causal: bool = True,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    """The unfused pipeline: dense decode of K and V (HIP kernel), GQA broadcast, torch SDPA on the GPU."""
    B, H_q, T_q, d_h = Q.shape
    H_kv = K_idx.shape[1]
    assert H_q % H_kv == 0, f"H_q={H_q} must be divisible by H_kv={H_kv}"
    g = H_q // H_kv
    K = decode_dequant(K_idx, K_radius_q, K_radius_scale, joint_K, r_qmax)
    V = decode_dequant(V_idx, V_radius_q, V_radius_scale, joint_V, r_qmax)
    if g > 1:
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d_h)
    return F.scaled_dot_product_attention(Q, K, V, attn_mask=None, is_causal=causal, scale=softmax_scale)


def fused_attention_hopper(Q, K_idx, K_radius_q, K_radius_scale, joint_K, V_idx, V_radius_q, V_radius_scale, joint_V,
                           r_qmax, causal=True, softmax_scale=None, block_q=256, block_kv=128, num_warps=8,
                           num_stages=3, use_fp8_codebook=True):
    """Name kept for callers of the reference; runs the one gfx950 kernel (fp8 table by default, as there)."""
    return fused_attention(Q, K_idx, K_radius_q, K_radius_scale, joint_K, V_idx, V_radius_q, V_radius_scale, joint_V,
                           r_qmax, causal=causal, softmax_scale=softmax_scale, use_fp8_codebook=use_fp8_codebook)


def fused_attention_blackwell(Q, K_idx, K_radius_q, K_radius_scale, joint_K, V_idx, V_radius_q, V_radius_scale, joint_V,
                              r_qmax, causal=True, softmax_scale=None, block_q=256, block_kv=256, num_warps=8,
                              num_stages=4, use_fp8_codebook=True):
    """Name kept for callers of the reference; runs the one gfx950 kernel (fp8 table by default, as there)."""
    return fused_attention(Q, K_idx, K_radius_q, K_radius_scale, joint_K, V_idx, V_radius_q, V_radius_scale, joint_V,
                           r_qmax, causal=causal, softmax_scale=softmax_scale, use_fp8_codebook=use_fp8_codebook)


def encode_joint_fp8(joint_fp16: torch.Tensor) -> torch.Tensor:
    """(H, K, 4) joint codebook -> float8_e4m3fn."""
    return joint_fp16.to(torch.float8_e4m3fn)


def hopper_available() -> bool:
    """False: this build targets CDNA4 (gfx950) only."""
    return False


def blackwell_available() -> bool:
    """False: this build targets CDNA4 (gfx950) only."""
    return False


def device_info() -> dict:
    """Which device the kernels will run on; same keys in the GPU and the no-GPU case."""
    if not torch.cuda.is_available():
        return {"gpu": None, "compute_capability": None, "variant": "cpu", "variant_auto_dispatched": "cpu",
                "fp8_codebook": False, "fp8_codebook_supported": False}
    cap = torch.cuda.get_device_capability()
    props = torch.cuda.get_device_properties(0)
    arch = getattr(props, "gcnArchName", "").split(":")[0]
    return {"gpu": torch.cuda.get_device_name(), "compute_capability": f"{cap[0]}.{cap[1]}", "arch": arch,
            "variant": "cdna4", "variant_auto_dispatched": "cdna4", "fp8_codebook": False,
            "fp8_codebook_supported": True}
