from hqmq_amd.attention import fused_attention_blackwell as fused_hqmq_attention_blackwell  # noqa: F401
from hqmq_amd.attention import blackwell_available  # noqa: F401
