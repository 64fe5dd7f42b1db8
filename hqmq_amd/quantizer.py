"""The reference's quantizer classes, backed by the HIP kernels.

Class names, constructor signatures, attributes and error behaviour follow
src/quantizers/{base,hqmq,outlier_aware,outlier_generic,hqmq_padded}.py of the
reference.  `quantize_K` / `quantize_V` keep the fake-quant contract (same
shape and dtype out); the additions (`encode_*`, `new_cache`, `append`) expose
the integer codes and the bit-packed cache the reference never materialises.

Only the production branch is implemented in kernels: unit magnitude, linear
radius, jl_dim = 0, evaluation mode, 1 <= radius_bits <= 8.  The ablation
switches are accepted by the constructors and raise NotImplementedError when a
quantize call would need them.  Tensors must live on the GPU: there is no CPU path.
"""
from __future__ import annotations

import math
from abc import ABC, abstractmethod
from typing import Optional

import torch
import torch.nn as nn

from . import _lib as L
from . import ops
from .codebook import _make_24cell_codebook
from .packed import PackedKV, PackedTensor


class KVQuantizer(ABC):
    """Plug-in interface: (B, n_kv_heads, T, d_head) in, same shape and dtype out."""

    @abstractmethod
    def quantize_K(self, k: torch.Tensor, layer_idx: int) -> torch.Tensor: ...

    @abstractmethod
    def quantize_V(self, v: torch.Tensor, layer_idx: int) -> torch.Tensor: ...

    @abstractmethod
    def bits_per_value(self) -> float: ...

    @property
    def name(self) -> str:
        return type(self).__name__


class HQMQQuantizer(KVQuantizer):
    """Hurwitz quaternion multiplicative quantizer (direction = q_p * q_s, per-token max radius scale)."""

    def __init__(self, n_layers: int, n_heads: int, secondary_size: int = 24, radius_bits: int = 4, jl_dim: int = 0,
                 magnitude_mode: str = "unit", robust_radius_scale: bool = False, log_radius: bool = False,
                 device: str = "cuda", init: str = "random", seed: int = 42):
        self.chunk_dim = 4
        self.n_layers, self.n_heads = n_layers, n_heads
        self.secondary_size, self.radius_bits, self.jl_dim = secondary_size, radius_bits, jl_dim
        self.magnitude_mode = magnitude_mode
        self.robust_radius_scale, self.log_radius = robust_radius_scale, log_radius
        if magnitude_mode not in ("unit", "free"):
            raise ValueError(f"magnitude_mode={magnitude_mode}")
        self.training = False
        self.tau = 1.0
        self._primary = _make_24cell_codebook()
        self._R = None
        gen = torch.Generator().manual_seed(seed)
        if init == "random":
            raw = torch.randn(n_layers, n_heads, 2, secondary_size, 4, generator=gen)
        elif init == "hurwitz_perturbed":
            reps = (secondary_size + 23) // 24
            base = self._primary.repeat(reps, 1)[:secondary_size].view(1, 1, 1, secondary_size, 4)
            raw = base.expand(n_layers, n_heads, 2, secondary_size, 4).clone()
            raw = raw + 0.1 * torch.randn_like(raw)
        else:
            raise ValueError(init)
        self.secondary_raw = nn.Parameter(raw.to(device=device, dtype=torch.float32))
        self._joint_cache: dict = {}

    # ---- hooks the reference's calibration glue looks for ----
    def trainable_parameters(self):
        return [self.secondary_raw]

    def set_training(self, training: bool, tau: Optional[float] = None):
        self.training = training
        if tau is not None:
            self.tau = tau
        self.invalidate_codebooks()

    def _refresh_rotations(self):
        self.invalidate_codebooks()

    def invalidate_codebooks(self):
        """Forget the cached joint tables.  They are rebuilt on the next call; needed after an in-place write
        through secondary_raw.data (which leaves no trace on the parameter), not after assignments or ordinary
        in-place ops, which the cache detects itself.  Packed caches made earlier keep the table they were created
        with: codes stay decodable with the table they were encoded against."""
        self._joint_cache.clear()

    # ---- codebook ----
    def _check_supported(self):
        if (self.magnitude_mode != "unit" or self.jl_dim != 0 or self.robust_radius_scale or self.log_radius
                or self.training or not 1 <= self.radius_bits <= 8):
            raise NotImplementedError(
                "the HIP path implements the production branch only: magnitude_mode='unit', jl_dim=0, linear radius "
                "with 1..8 bits, evaluation mode")

    def _joint_and_slack(self, layer_idx: int, kv: int, ref: torch.Tensor):
        L.require_gpu(ref, "tensor")
        raw = self.secondary_raw
        if raw.device != ref.device:
            raise L.HqmqError(f"quantizer parameters are on {raw.device}, the tensor is on {ref.device}")
        key = (layer_idx, kv, ref.dtype)
        stamp = (id(raw), raw.data_ptr(), raw._version)     # a new parameter, new storage (.data = w) or an in-place op
        hit = self._joint_cache.get(key)
        if hit is not None and hit[0] == stamp:
            return hit[1], hit[2]
        joint, slack = ops.build_joint(raw.detach()[layer_idx, :, kv], ref.dtype)
        self._joint_cache[key] = (stamp, joint, slack)
        return joint, slack

    def _get_codebook(self, layer_idx: int, kv: int, ref: torch.Tensor) -> torch.Tensor:
        """(n_heads, 24*S, 4) joint codebook q_p * q_s in ref.dtype, index k = p*S + s."""
        return self._joint_and_slack(layer_idx, kv, ref)[0]

    # ---- fake-quant contract ----
    def _qdq(self, x: torch.Tensor, layer_idx: int, kv: int) -> torch.Tensor:
        if x.shape[-1] % 4 != 0:
            raise ValueError(f"d_head={x.shape[-1]} not divisible by 4")
        self._check_supported()
        joint, slack = self._joint_and_slack(layer_idx, kv, x)
        return ops.quantize(x, joint, slack, self.radius_bits, want_codes=False, want_dense=True)["out"]

    def quantize_K(self, k, layer_idx):
        return self._qdq(k, layer_idx, kv=0)

    def quantize_V(self, v, layer_idx):
        return self._qdq(v, layer_idx, kv=1)

    def bits_per_value(self):
        bits_dir = math.log2(24 * self.secondary_size)
        radius = 0 if self.magnitude_mode == "free" else self.radius_bits
        return (bits_dir + radius + self.jl_dim) / 4.0

    @property
    def name(self) -> str:
        parts = [f"HQMQ_s{self.secondary_size}_r{self.radius_bits}"]
        if self.jl_dim > 0:
            parts.append(f"jl{self.jl_dim}")
        if self.magnitude_mode != "unit":
            parts.append(self.magnitude_mode)
        if self.log_radius:
            parts.append("logr")
        if self.robust_radius_scale:
            parts.append("robust")
        return "_".join(parts)

    # ---- real codes (additive API) ----
    def encode(self, x: torch.Tensor, layer_idx: int, kv: int) -> dict:
        """Integer codes of x: idx (int32, in [0, 24S)), rq (int32, in [0, qmax]), r_max (x.dtype),
        joint (the table idx refers to).  These are the fused kernel's unpacked inputs."""
        if x.shape[-1] % 4 != 0:
            raise ValueError(f"d_head={x.shape[-1]} not divisible by 4")
        self._check_supported()
        joint, slack = self._joint_and_slack(layer_idx, kv, x)
        out = ops.quantize(x, joint, slack, self.radius_bits, want_codes=True)
        out["joint"] = joint
        return out

    def encode_K(self, k, layer_idx):
        return self.encode(k, layer_idx, 0)

    def encode_V(self, v, layer_idx):
        return self.encode(v, layer_idx, 1)

    def new_cache(self, batch: int, max_tokens: int, d_head: int, dtype: torch.dtype, layer_idx: int,
                  outliers: bool = False, sideband_frac: float = 0.125) -> PackedKV:
        """An empty bit-packed cache for one layer (K and V planes, codebooks attached)."""
        self._check_supported()
        dev = self.secondary_raw.device
        ref = torch.empty(0, dtype=dtype, device=dev)
        mk = lambda kv: PackedTensor(batch, self.n_heads, max_tokens, d_head, self.secondary_size, self.radius_bits,
                                     dtype, dev, joint=self._joint_and_slack(layer_idx, kv, ref)[0], outliers=outliers,
                                     sideband_frac=sideband_frac)
        return PackedKV(mk(0), mk(1))

    def _append_one(self, cache: PackedTensor, x: torch.Tensor, layer_idx: int, kv: int, pos, median_mult=None):
        joint, slack = self._joint_and_slack(layer_idx, kv, x)
        T = x.shape[2]
        t_off = 0 if pos is not None else cache.length
        if pos is None and t_off + T > cache.t_cap:
            raise L.HqmqError(f"cache capacity {cache.t_cap} exceeded by append of {T} rows at {t_off}")
        thr = count = None
        if median_mult is not None:
            if not cache.has_outliers:
                raise L.HqmqError("this cache was allocated without an outlier sideband")
            _, thr, count = ops.med3x_threshold(x, median_mult)
        ops.quantize(x, joint, slack, self.radius_bits, want_codes=False, thr=thr, cache=cache, t_off=t_off, pos=pos)
        if thr is not None:
            ops.outlier_compact(x, cache, t_off=t_off, pos=pos)
        if pos is None:
            cache.length = t_off + T
        cache.note_append(T)
        return count

    def append(self, cache: PackedKV, k: torch.Tensor, v: torch.Tensor, layer_idx: int,
               pos: Optional[torch.Tensor] = None) -> None:
        """Quantize the new tokens k, v (B, H, T_new, d_h) and write them behind the rows already in `cache`.
        pos (int32 [B]) gives each sequence's current length for ragged batches; the caller advances it."""
        self._check_supported()
        self._append_both(cache, k, v, layer_idx, pos)

    def _append_both(self, cache: PackedKV, k: torch.Tensor, v: torch.Tensor, layer_idx: int, pos, median_mult=None):
        """K and V through one call of the library (shared launches); returns the flagged-chunk counts per head."""
        if k.shape[2] != v.shape[2]:
            raise ValueError("k and v must bring the same number of new tokens")
        T = k.shape[2]
        for pt in (cache.K, cache.V):
            if pos is None and pt.length + T > pt.t_cap:
                raise L.HqmqError(f"cache capacity {pt.t_cap} exceeded by append of {T} rows at {pt.length}")
            if median_mult is not None and not pt.has_outliers:
                raise L.HqmqError("this cache was allocated without an outlier sideband")
        if pos is None and cache.K.length != cache.V.length:      # never the case for caches filled through append()
            return (self._append_one(cache.K, k, layer_idx, 0, pos, median_mult),
                    self._append_one(cache.V, v, layer_idx, 1, pos, median_mult))
        kj, ks = self._joint_and_slack(layer_idx, 0, k)
        vj, vs = self._joint_and_slack(layer_idx, 1, v)
        t_off = 0 if pos is not None else cache.K.length
        counts = ops.append_kv(k, v, cache.K, cache.V, kj, ks, vj, vs, self.radius_bits, t_off=t_off, pos=pos,
                               median_mult=median_mult)
        if pos is None:
            cache.K.length = cache.V.length = t_off + T
        cache.K.note_append(T)
        cache.V.note_append(T)
        return counts


class _OutlierStats:
    """Running mean of the per-call outlier rate, read back from the device lazily."""

    def __init__(self):
        self._observed_outlier_rate = 0.0
        self._n_observations = 0
        self._pending = []

    def _note(self, count: torch.Tensor, total: int):
        self._pending.append((count, total))
        if len(self._pending) > 4096:
            self._fold()

    def _fold(self):
        for count, total in self._pending:
            rate = float(count.sum().item()) / max(total, 1)
            self._observed_outlier_rate = (self._observed_outlier_rate * self._n_observations + rate) / (self._n_observations + 1)
            self._n_observations += 1
        self._pending = []


class OutlierAwareHQMQQuantizer(KVQuantizer, _OutlierStats):
    """Med-C outlier extraction around HQMQ: chunks with norm > C * per-head median stay verbatim."""

    def __init__(self, inner: HQMQQuantizer, outlier_fraction: float = 0.01, threshold_mode: str = "fraction",
                 median_mult: float = 20.0):
        assert isinstance(inner, HQMQQuantizer), "wrapper expects HQMQQuantizer"
        _OutlierStats.__init__(self)
        self.inner = inner
        # The reference's median is torch.quantile, which raises above 2^24 chunks per head in one call
        # (src/quantizers/outlier_aware.py:68).  The radix select here has no such bound; set this to True to get
        # the reference's RuntimeError from quantize_K / quantize_V / encode instead of the extension.
        self.strict_quantile_limit = False
        self.outlier_fraction, self.threshold_mode, self.median_mult = outlier_fraction, threshold_mode, median_mult
        self.chunk_dim = inner.chunk_dim

    def trainable_parameters(self):
        return self.inner.trainable_parameters()

    def set_training(self, training, tau=None):
        self.inner.set_training(training, tau=tau)

    def _refresh_rotations(self):
        self.inner._refresh_rotations()

    def _require_median_mode(self):
        if self.threshold_mode == "fraction":
            raise NotImplementedError("threshold_mode='fraction' is not implemented in the HIP path; use 'median_mult'")
        if self.threshold_mode != "median_mult":
            raise ValueError(self.threshold_mode)

    def _qdq(self, x: torch.Tensor, layer_idx: int, kv: int) -> torch.Tensor:
        self._require_median_mode()
        if x.shape[-1] % 4 != 0:
            raise ValueError(f"d_head={x.shape[-1]} not divisible by 4")
        self.inner._check_supported()
        joint, slack = self.inner._joint_and_slack(layer_idx, kv, x)
        _, thr, count = ops.med3x_threshold(x, self.median_mult, strict_quantile_limit=self.strict_quantile_limit)
        self._note(count, x.numel() // 4)
        return ops.quantize(x, joint, slack, self.inner.radius_bits, want_codes=False, want_dense=True, thr=thr)["out"]

    def quantize_K(self, k, layer_idx):
        return self._qdq(k, layer_idx, kv=0)

    def quantize_V(self, v, layer_idx):
        return self._qdq(v, layer_idx, kv=1)

    def bits_per_value(self):
        self._fold()
        if self._n_observations > 0:
            p = self._observed_outlier_rate
        else:
            p = self.outlier_fraction if self.threshold_mode == "fraction" else 0.03
        return (1 - p) * self.inner.bits_per_value() + p * 16 + 1 / self.chunk_dim

    @property
    def name(self):
        if self.threshold_mode == "fraction":
            return f"Outlier{int(self.outlier_fraction * 100)}p_{self.inner.name}"
        return f"OutlierMed{self.median_mult:.0f}_{self.inner.name}"

    # ---- real codes (additive API) ----
    def encode(self, x: torch.Tensor, layer_idx: int, kv: int) -> dict:
        """idx, rq, r_max as the inner quantizer gives them, plus mask (bool, flagged chunks),
        median (fp32 per head) and threshold (x.dtype per head)."""
        self._require_median_mode()
        self.inner._check_supported()
        joint, slack = self.inner._joint_and_slack(layer_idx, kv, x)
        med, thr, count = ops.med3x_threshold(x, self.median_mult, strict_quantile_limit=self.strict_quantile_limit)
        self._note(count, x.numel() // 4)
        out = ops.quantize(x, joint, slack, self.inner.radius_bits, want_codes=True, thr=thr, want_mask=True)
        out.update(joint=joint, median=med, threshold=thr)
        return out

    def encode_K(self, k, layer_idx):
        return self.encode(k, layer_idx, 0)

    def encode_V(self, v, layer_idx):
        return self.encode(v, layer_idx, 1)

    def new_cache(self, batch, max_tokens, d_head, dtype, layer_idx, sideband_frac: float = 0.125) -> PackedKV:
        return self.inner.new_cache(batch, max_tokens, d_head, dtype, layer_idx, outliers=True, sideband_frac=sideband_frac)

    def append(self, cache: PackedKV, k, v, layer_idx, pos=None) -> None:
        """Quantize-and-append with Med-C extraction; the median is over the chunks of this call, per head."""
        self._require_median_mode()
        self.inner._check_supported()
        counts = self.inner._append_both(cache, k, v, layer_idx, pos, median_mult=self.median_mult)
        for count, x in zip(counts, (k, v)):
            if count is not None:
                self._note(count, x.numel() // 4)


class OutlierAwareGenericQuantizer(KVQuantizer, _OutlierStats):
    """Med-C outlier extraction around any KVQuantizer (fake-quant only: the inner has no packed form)."""

    def __init__(self, inner: KVQuantizer, chunk_dim: int = 4, outlier_fraction: float = 0.03,
                 threshold_mode: str = "median_mult", median_mult: float = 3.0):
        _OutlierStats.__init__(self)
        self.inner, self.chunk_dim = inner, chunk_dim
        self.outlier_fraction, self.threshold_mode, self.median_mult = outlier_fraction, threshold_mode, median_mult

    def trainable_parameters(self):
        return self.inner.trainable_parameters() if hasattr(self.inner, "trainable_parameters") else []

    def set_training(self, training, tau=None):
        if hasattr(self.inner, "set_training"):
            self.inner.set_training(training, tau=tau)

    def _qdq(self, x: torch.Tensor, layer_idx: int, kv: int) -> torch.Tensor:
        if self.threshold_mode == "fraction":
            raise NotImplementedError("threshold_mode='fraction' is not implemented in the HIP path; use 'median_mult'")
        if self.threshold_mode != "median_mult":
            raise ValueError(self.threshold_mode)
        if self.chunk_dim != 4:
            raise NotImplementedError("the Med-C kernels work on 4-element chunks")
        B, H, T, d = x.shape
        _, thr, count = ops.med3x_threshold(x, self.median_mult)
        self._note(count, x.numel() // 4)
        mask = ops.outlier_mask(x, thr)
        inner = self.inner.quantize_K(x, layer_idx) if kv == 0 else self.inner.quantize_V(x, layer_idx)
        n = d // 4
        return torch.where(mask.unsqueeze(-1), x.reshape(B, H, T, n, 4), inner.reshape(B, H, T, n, 4)).reshape(B, H, T, d)

    def quantize_K(self, k, layer_idx):
        return self._qdq(k, layer_idx, kv=0)

    def quantize_V(self, v, layer_idx):
        return self._qdq(v, layer_idx, kv=1)

    def bits_per_value(self):
        self._fold()
        if self._n_observations > 0:
            p = self._observed_outlier_rate
        else:
            p = self.outlier_fraction if self.threshold_mode == "fraction" else 0.03
        return (1 - p) * self.inner.bits_per_value() + p * 16.0 + 1.0 / self.chunk_dim

    @property
    def name(self):
        if self.threshold_mode == "fraction":
            return f"Outlier{int(self.outlier_fraction * 100)}p_{self.inner.__class__.__name__}"
        return f"OutlierMed{self.median_mult:.0f}_{self.inner.__class__.__name__}"


class PaddedHQMQQuantizer(KVQuantizer):
    """HQMQ for head dims that are not a multiple of 4: zero-pad, quantize, truncate."""

    def __init__(self, n_layers: int, n_heads: int, d_head: int, secondary_size: int = 24, radius_bits: int = 4,
                 device: str = "cuda", init: str = "random", seed: int = 42):
        self.d_head_orig = d_head
        self.d_head_padded = (d_head + 3) // 4 * 4
        self.pad_count = self.d_head_padded - d_head
        self.chunk_dim = 4
        self.radius_bits, self.secondary_size = radius_bits, secondary_size
        self.inner = HQMQQuantizer(n_layers=n_layers, n_heads=n_heads, secondary_size=secondary_size,
                                   radius_bits=radius_bits, device=device, init=init, seed=seed)

    def trainable_parameters(self):
        return self.inner.trainable_parameters()

    def set_training(self, training, tau=None):
        self.inner.set_training(training, tau=tau)

    def _qdq(self, x: torch.Tensor, layer_idx: int, kv: int) -> torch.Tensor:
        d = x.shape[-1]
        if d != self.d_head_padded:
            assert d == self.d_head_orig, f"Expected d_head={self.d_head_orig}, got {d}"
            x = torch.nn.functional.pad(x, (0, self.pad_count))
        xq = self.inner.quantize_K(x, layer_idx) if kv == 0 else self.inner.quantize_V(x, layer_idx)
        return xq[..., :self.d_head_orig]

    def quantize_K(self, k, layer_idx):
        return self._qdq(k, layer_idx, kv=0)

    def quantize_V(self, v, layer_idx):
        return self._qdq(v, layer_idx, kv=1)

    def bits_per_value(self):
        return self.inner.bits_per_value() * self.d_head_padded / self.d_head_orig

    @property
    def name(self):
        return f"PaddedHQMQ_d{self.d_head_orig}to{self.d_head_padded}_{self.inner.name}"

    # ---- packed cache: the head is zero-padded to a size the attention kernels take ----
    _ATTN_DIMS = (16, 32, 64, 80, 128, 160, 256)

    @property
    def d_head_stored(self) -> int:
        """Head size of the packed planes: the smallest the attention kernels support that holds d_head.
        The extra chunks are all-zero, quantize to radius code 0 and decode to exactly 0."""
        for d in self._ATTN_DIMS:
            if d >= self.d_head_padded:
                return d
        raise L.HqmqError(f"d_head={self.d_head_orig} is beyond the attention kernels' 256")

    def _pad(self, x: torch.Tensor) -> torch.Tensor:
        d = x.shape[-1]
        if d == self.d_head_stored:
            return x
        assert d in (self.d_head_orig, self.d_head_padded), f"Expected d_head={self.d_head_orig}, got {d}"
        return torch.nn.functional.pad(x, (0, self.d_head_stored - d))

    def new_cache(self, batch: int, max_tokens: int, dtype: torch.dtype, layer_idx: int) -> PackedKV:
        """An empty bit-packed cache of d_head_stored-wide heads (12-bit code rows need an even number of chunks
        per lane; where the head does not give that, codes are stored 16 bits wide)."""
        inner, d = self.inner, self.d_head_stored
        inner._check_supported()
        idx_bits, main_bits, aux_bits = L.layout_bits(inner.secondary_size, inner.radius_bits)
        layout = None
        if main_bits == 12 and (d // 16) % 2:
            layout = (idx_bits, 16, max(0, idx_bits + inner.radius_bits - 16))
        dev = inner.secondary_raw.device
        ref = torch.empty(0, dtype=dtype, device=dev)
        mk = lambda kv: PackedTensor(batch, inner.n_heads, max_tokens, d, inner.secondary_size, inner.radius_bits, dtype, dev,
                                     joint=inner._joint_and_slack(layer_idx, kv, ref)[0], layout=layout)
        kv = PackedKV(mk(0), mk(1))
        kv.K.d_head_orig = kv.V.d_head_orig = self.d_head_orig
        return kv

    def append(self, cache: PackedKV, k: torch.Tensor, v: torch.Tensor, layer_idx: int, pos=None) -> None:
        self.inner.append(cache, self._pad(k), self._pad(v), layer_idx, pos=pos)
