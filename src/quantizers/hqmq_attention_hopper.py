from hqmq_amd.attention import fused_attention_hopper as fused_hqmq_attention_hopper  # noqa: F401
from hqmq_amd.attention import encode_joint_fp8, hopper_available  # noqa: F401
