"""Hugging Face `transformers` caches over the HQMQ path.

QuantizedCache
    The reference's cache hook (src/model_utils.py:22-32 of the reference): every K, V that is appended goes
    through `quantize_K` / `quantize_V` (fake quantization on the GPU kernels) into an ordinary DynamicCache.

PackedQuantizedCache  +  attn_implementation="hqmq_packed"
    What the reference describes but does not have: each layer keeps the bit-packed planes (`PackedKV`), an
    append quantizes the new tokens straight into them, and attention reads the compressed cache with the fused
    kernel.  `update` returns only the new tokens' K, V (nothing dense is kept); the tensors it returns carry a
    reference to their layer, which is how the attention function finds the planes.

    model.set_attn_implementation("hqmq_packed")
    cache = PackedQuantizedCache(quantizer, max_tokens=4096)
    out = model(input_ids, past_key_values=cache, use_cache=True)

Limits: the mask is causal, optionally with left padding (the usual batched-generation layout; pad tokens are
quantized and stored like any other, and never attended to); no beam reordering (cropping is supported).  This module imports `transformers`; nothing else in the package does.
"""
from __future__ import annotations

from typing import Optional

import warnings

import torch
from transformers import AttentionInterface, DynamicCache
from transformers.cache_utils import DynamicLayer

from ._lib import HqmqError
from .attention import fused_attention_packed
from .quantizer import KVQuantizer

ATTN_NAME = "hqmq_packed"


class QuantizedCache(DynamicCache):
    """DynamicCache that fake-quantizes K, V on every update (same class as the reference's)."""

    def __init__(self, quantizer: KVQuantizer):
        super().__init__()
        self.quantizer = quantizer

    def update(self, key_states, value_states, layer_idx, *args, **kwargs):
        k_q = self.quantizer.quantize_K(key_states, layer_idx)
        v_q = self.quantizer.quantize_V(value_states, layer_idx)
        return super().update(k_q, v_q, layer_idx, *args, **kwargs)


class PackedLayer(DynamicLayer):
    """One layer's compressed K and V."""

    def __init__(self, quantizer, layer_idx: int, max_tokens: int, sideband_frac: float, overflow_check_every: int = 256):
        super().__init__()
        self.quantizer, self.layer_idx, self.max_tokens, self.sideband_frac = quantizer, layer_idx, max_tokens, sideband_frac
        self.packed = None
        self.n_tokens = 0
        # a sideband that runs full stores further outlier chunks as plain HQMQ chunks: the flag the kernels set is
        # read back after the first append (the prefill) and then once every `overflow_check_every` appends (one
        # device read for K and V together, never under stream capture; 0 = never, call check_overflow() yourself),
        # and a warning is issued once
        self.overflow_check_every = overflow_check_every
        self._appends = 0
        self._warned = False

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, *args, **kwargs):
        if self.packed is None:
            B, _, _, d_h = key_states.shape
            kw = {"sideband_frac": self.sideband_frac} if hasattr(self.quantizer, "median_mult") else {}
            self.packed = self.quantizer.new_cache(B, self.max_tokens, d_h, key_states.dtype, self.layer_idx, **kw)
            self.dtype, self.device = key_states.dtype, key_states.device
            self.keys = self.values = torch.empty(0, dtype=self.dtype, device=self.device)
            self.is_initialized = True
        if self.n_tokens + key_states.shape[2] > self.packed.K.t_cap:
            raise HqmqError(f"PackedQuantizedCache holds {self.packed.K.t_cap} tokens per sequence; raise max_tokens")
        self.quantizer.append(self.packed, key_states, value_states, self.layer_idx)
        self.n_tokens += key_states.shape[2]
        self._appends += 1
        if self.packed.K.has_outliers and self.overflow_check_every and not self._warned and (
                self._appends == 1 or self._appends % self.overflow_check_every == 0) and not torch.cuda.is_current_stream_capturing():
            if int((self.packed.K.sb_overflow | self.packed.V.sb_overflow).item()):          # K and V in one read
                self._warned = True
                warnings.warn(f"layer {self.layer_idx}: the outlier sideband is full; further outlier chunks are stored as plain "
                              f"HQMQ chunks (accuracy of those chunks, not data, is lost). Raise sideband_frac ({self.sideband_frac}).")
        key_states.hqmq_layer = self          # how hqmq_packed_attention finds the planes
        return key_states, value_states

    def get_seq_length(self) -> int:
        return self.n_tokens

    def get_max_length(self) -> int:
        return self.max_tokens

    def crop(self, tokens_to_remove: int) -> None:
        """Drops the last -tokens_to_remove tokens (DynamicLayer.crop; a positive value is its older meaning: the
        length to keep)."""
        if self.packed is None or tokens_to_remove == 0:
            return
        keep = tokens_to_remove if tokens_to_remove > 0 else max(self.n_tokens + tokens_to_remove, 0)
        if keep >= self.n_tokens:
            return
        self.packed.crop_(keep)
        self.n_tokens = keep

    def batch_repeat_interleave(self, repeats: int) -> None:
        raise NotImplementedError("a packed cache cannot be repeated along the batch")

    def batch_select_indices(self, indices: torch.Tensor) -> None:
        raise NotImplementedError("a packed cache cannot be re-indexed along the batch")


class PackedQuantizedCache(DynamicCache):
    """Keeps every layer bit-packed; use with attn_implementation="hqmq_packed"."""

    def __init__(self, quantizer, max_tokens: int, sideband_frac: float = 0.125, overflow_check_every: int = 256):
        super().__init__()
        if not hasattr(quantizer, "append") or not hasattr(quantizer, "new_cache"):
            raise TypeError("PackedQuantizedCache needs an HQMQ quantizer (HQMQ(...) or with_outlier_extraction(HQMQ(...)))")
        self.quantizer, self.max_tokens, self.sideband_frac = quantizer, int(max_tokens), sideband_frac
        self.overflow_check_every = overflow_check_every

    def update(self, key_states, value_states, layer_idx, *args, **kwargs):
        while len(self.layers) <= layer_idx:
            self.layers.append(PackedLayer(self.quantizer, len(self.layers), self.max_tokens, self.sideband_frac,
                                           self.overflow_check_every))
        return self.layers[layer_idx].update(key_states, value_states, *args, **kwargs)

    def check_overflow(self) -> None:
        """Raises if any layer ran out of outlier sideband room (one device read per tensor): allocate with a
        larger sideband_frac for data with many flagged chunks."""
        for layer in self.layers:
            if layer.packed is not None:
                layer.packed.K.check_overflow()
                layer.packed.V.check_overflow()

    def nbytes(self) -> int:
        """Compressed bytes held (all layers, rows written so far)."""
        return sum(layer.packed.nbytes(layer.n_tokens) for layer in self.layers if layer.packed is not None)


def hqmq_packed_attention(module, query, key, value, attention_mask, dropout: float = 0.0,
                          scaling: Optional[float] = None, **kwargs):
    """attention_interface function: causal attention of `query` over the packed cache of `key`'s layer."""
    layer = getattr(key, "hqmq_layer", None)
    if layer is None:
        raise HqmqError('attn_implementation="hqmq_packed" needs past_key_values=PackedQuantizedCache(...)')
    if dropout:
        raise NotImplementedError("attention dropout is not supported on the packed path")
    t_q = query.shape[2]
    out = fused_attention_packed(query, layer.packed, causal=True, causal_offset=layer.n_tokens - t_q,
                                 softmax_scale=scaling, T_kv=layer.n_tokens,
                                 kv_starts=_first_visible(attention_mask, layer.n_tokens))
    return out.transpose(1, 2).contiguous(), None


def _first_visible(attention_mask, t_kv: int):
    """Left padding from the 4-D mask the model built (bool, or additive with 0 = visible): the first key the
    last query row may see, per sequence.  Everything else about the mask is taken to be causal."""
    if attention_mask is None:
        return None
    row = attention_mask[:, 0, -1, :t_kv]
    visible = row if row.dtype == torch.bool else row > -1.0
    return visible.to(torch.int32).argmax(-1).to(torch.int32)


def register() -> str:
    """Registers the attention function (and the mask builder it shares with sdpa) under ATTN_NAME."""
    AttentionInterface.register(ATTN_NAME, hqmq_packed_attention)
    try:
        from transformers.masking_utils import AttentionMaskInterface, sdpa_mask
        AttentionMaskInterface.register(ATTN_NAME, sdpa_mask)
    except ImportError:          # older transformers build the mask without a per-implementation table
        pass
    return ATTN_NAME


register()
