"""Same export list as libs/moda_triton/fla/ops/moda/__init__.py:5-29 (minus the torch reference loops)."""
from moda_amd import (  # noqa: F401
    parallel_moda,
    parallel_moda_bwd,
    parallel_moda_fwd,
    parallel_moda_chunk_visible,
    parallel_moda_chunk_visible_bwd,
    parallel_moda_chunk_visible_fwd,
    parallel_fda,
    parallel_fda_bwd,
    parallel_fda_fwd,
)

__all__ = [
    "parallel_moda",
    "parallel_moda_fwd",
    "parallel_moda_bwd",
    "parallel_moda_chunk_visible",
    "parallel_moda_chunk_visible_fwd",
    "parallel_moda_chunk_visible_bwd",
    "parallel_fda",
    "parallel_fda_fwd",
    "parallel_fda_bwd",
]
