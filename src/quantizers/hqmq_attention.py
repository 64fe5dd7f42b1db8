from hqmq_amd.attention import fused_attention as fused_hqmq_attention_triton  # noqa: F401
from hqmq_amd.attention import fused_attention_reference as fused_hqmq_attention_torch  # noqa: F401
