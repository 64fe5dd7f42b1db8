from hqmq_amd.quantizer import OutlierAwareHQMQQuantizer  # noqa: F401
