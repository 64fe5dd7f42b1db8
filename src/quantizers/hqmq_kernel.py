from hqmq_amd.attention import decode_dequant as hqmq_decode_triton  # noqa: F401
