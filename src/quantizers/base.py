from hqmq_amd.quantizer import KVQuantizer  # noqa: F401
