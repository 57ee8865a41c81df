"""moda_amd -- MI355X (gfx950) implementation of MoDA's fused sequence+depth attention.

Public names follow the reference's ``fla.ops.moda`` package
(libs/moda_triton/fla/ops/moda/__init__.py:5-29) plus the depth-only and plain
attention entry points that the reference keeps in sibling modules.
"""
from .ops import (  # noqa: F401
    parallel_moda,
    parallel_moda_fwd,
    parallel_moda_bwd,
    parallel_moda_chunk_visible,
    parallel_moda_chunk_visible_fwd,
    parallel_moda_chunk_visible_bwd,
    parallel_fda,
    parallel_fda_fwd,
    parallel_fda_bwd,
    parallel_attn,
    parallel_attn_fwd,
    parallel_attn_bwd,
    ParallelMixtureOfDepthAttentionFunction,
    ParallelMixtureOfDepthAttentionChunkVisibleFunction,
    ParallelFlashDepthAttentionFunction,
    ParallelAttentionFunction,
    fold_gqa_heads,
    unfold_gqa_heads,
    set_fp32_compute,
)
from .depth_cache import build_depth_cache, stack_depth, DepthCache  # noqa: F401
from .modules import DepthStream, MoDAAttention, MoDAStack  # noqa: F401

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
    "parallel_attn",
    "parallel_attn_fwd",
    "parallel_attn_bwd",
    "fold_gqa_heads",
    "unfold_gqa_heads",
    "set_fp32_compute",
    "build_depth_cache",
    "stack_depth",
    "DepthCache",
    "DepthStream",
    "MoDAAttention",
    "MoDAStack",
]
