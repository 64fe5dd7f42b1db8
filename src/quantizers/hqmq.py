from hqmq_amd.codebook import quat_mul  # noqa: F401
from hqmq_amd.quantizer import HQMQQuantizer  # noqa: F401
