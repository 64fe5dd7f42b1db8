from hqmq_amd.codebook import _make_24cell_codebook  # noqa: F401
