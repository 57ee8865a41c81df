"""CPU restatement of the reference's torch MoDA definition.

TEST INFRASTRUCTURE ONLY.  Nothing under ``moda_amd/`` imports this package;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may call it, and only as the checker / the reported CPU baseline.
"""
from .moda_oracle import (  # noqa: F401
    MODES,
    visible_mask,
    moda_rows,
    moda_dense,
    moda_dense_fwd_bwd,
    moda_rows_subset,
    moda_blockwise_fwd_bwd,
    plain_gqa_dense,
    depth_cache_ref,
    depth_cache_grad_ref,
    compact_depth,
    scatter_depth_grad,
    packed_visible_mask,
    moda_packed_fwd_bwd,
    make_inputs,
    error_metrics,
    passes_reference_rule,
    flops_fwd,
)
