"""hqmq_amd — the HQMQ KV-cache path on MI355X (gfx950): HIP kernels behind a C ABI.

The public names of the reference's `hqmq` package are re-exported from here;
`import hqmq` (the façade at the repository root) gives the same objects.
"""
from .codebook import _make_24cell_codebook, quat_mul
from .quantizer import (KVQuantizer, HQMQQuantizer, OutlierAwareHQMQQuantizer, OutlierAwareGenericQuantizer,
                        PaddedHQMQQuantizer)
from .attention import (fused_attention, fused_attention_packed, fused_attention_reference, fused_attention_hopper,
                        fused_attention_blackwell, decode_dequant, encode_joint_fp8, hopper_available,
                        blackwell_available, device_info)
from .packed import PackedKV, PackedTensor
from ._lib import HqmqError, library_path

HQMQ = HQMQQuantizer
PaddedHQMQ = PaddedHQMQQuantizer


def with_outlier_extraction(quantizer, C: float = 3.0, *, generic: bool = False):
    """Wrap a quantizer with median-multiplier outlier extraction (chunks with norm > C * median stay verbatim).

    generic=False: the HQMQ wrapper (packed cache and sideband available); generic=True: the
    wrapper that accepts any KVQuantizer (fake-quant only).
    """
    if generic:
        return OutlierAwareGenericQuantizer(quantizer, chunk_dim=4, threshold_mode="median_mult", median_mult=C)
    return OutlierAwareHQMQQuantizer(quantizer, threshold_mode="median_mult", median_mult=C)


__version__ = "0.1.0"
