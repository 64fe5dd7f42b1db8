from hqmq_amd.quantizer import PaddedHQMQQuantizer  # noqa: F401
