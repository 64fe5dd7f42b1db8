"""HQMQ: Hurwitz Quaternion Multiplicative Quantization for KV cache — MI355X build.

Same public names as the reference package (hqmq/__init__.py:53-125 there):

    import hqmq
    q = hqmq.HQMQ(n_layers=32, n_heads=8, secondary_size=192, radius_bits=6)
    q = hqmq.with_outlier_extraction(q, C=3.0)
    K_q = q.quantize_K(K, layer_idx=0)            # fake-quant, same shape and dtype
    O = hqmq.fused_attention(Q, K_idx, K_rq, K_rs, joint_K, V_idx, V_rq, V_rs, joint_V, r_qmax=63)

plus the packed path the reference lacks:

    cache = q.new_cache(batch, max_tokens, d_head, torch.float16, layer_idx=0)
    q.append(cache, K, V, layer_idx=0)
    O = hqmq.fused_attention_packed(Q, cache)
"""
from hqmq_amd import (HQMQ, PaddedHQMQ, OutlierAwareHQMQQuantizer, OutlierAwareGenericQuantizer, fused_attention,
                      fused_attention_reference, fused_attention_packed, with_outlier_extraction, device_info,
                      PackedKV, PackedTensor, HqmqError, __version__)
from hqmq_amd import attention as kernels_ada        # noqa: F401  one kernel module serves all three names
from hqmq_amd import attention as kernels_hopper     # noqa: F401
from hqmq_amd import attention as kernels_blackwell  # noqa: F401

__all__ = [
    "HQMQ", "PaddedHQMQ", "OutlierAwareHQMQQuantizer", "OutlierAwareGenericQuantizer",
    "fused_attention", "fused_attention_reference", "fused_attention_packed",
    "with_outlier_extraction", "device_info", "PackedKV", "PackedTensor",
    "kernels_ada", "kernels_hopper", "kernels_blackwell",
]
