"""Same export list as libs/moda_triton/fla/ops/moda/__init__.py:5-29, minus the three torch reference loops
(``naive_*_ref``): this package ships kernels only, asking for one of those names raises an ImportError that
says where a restatement of them lives."""
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


_REFERENCE_LOOPS = (
    "naive_mixture_of_depth_causal_ref",
    "naive_mixture_of_depth_causal_ref_vis",
    "naive_mixture_of_depth_causal_chunk_visible_ref",
)


def __getattr__(name):
    if name in _REFERENCE_LOOPS:
        raise ImportError(
            f"fla.ops.moda.{name} is one of the reference's torch loops (moda_v14.py:1900-1991, "
            "moda_v16.py:2487-2582); moda_amd ships the device kernels only.  A CPU restatement of the loops, "
            "kept as test infrastructure, is oracle/moda_oracle.py (moda_rows) at the root of the moda_amd "
            "source tree."
        )
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
