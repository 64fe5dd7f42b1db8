"""Shared test helpers: bit-exact comparison, fixture decoding, seeded inputs."""
import numpy as np
import torch

DT = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}
EPS = {torch.float32: 2.0 ** -11, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


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
    plus two units of the compute precision relative to the reference value (the kernels multiply in fp16;
    a bf16 result cannot be closer than its own rounding)."""
    return base + 2.0 * EPS[dtype] * ref.abs()


def read_bits(row: np.ndarray, bitpos: int, nbits: int) -> int:
    """Python reader of the packed little-endian bit stream (independent of the C and HIP packers)."""
    v = 0
    for i in range(nbits):
        p = bitpos + i
        v |= ((int(row[p >> 3]) >> (p & 7)) & 1) << i
    return v
