"""Kernel entry points under the reference's names (hqmq/kernels.py:6-36 there).

The three hardware-variant names all run the single gfx950 kernel.
"""
from hqmq_amd.attention import (fused_attention as fused_attention_ada, fused_attention_reference, fused_attention_hopper,
                                fused_attention_blackwell, fused_attention_packed, decode_dequant, encode_joint_fp8,
                                hopper_available, blackwell_available)

__all__ = [
    "fused_attention_ada", "fused_attention_hopper", "fused_attention_blackwell", "fused_attention_reference",
    "fused_attention_packed", "decode_dequant", "encode_joint_fp8", "hopper_available", "blackwell_available",
]
