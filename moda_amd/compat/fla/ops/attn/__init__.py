from moda_amd import parallel_attn, parallel_attn_bwd, parallel_attn_fwd  # noqa: F401
