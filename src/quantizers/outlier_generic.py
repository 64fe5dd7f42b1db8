from hqmq_amd.quantizer import OutlierAwareGenericQuantizer  # noqa: F401
