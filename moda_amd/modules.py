"""Caller-side pieces around the attention operator: the attention module of the reference's vision
model and a manager for the depth stream it feeds.

``MoDAAttention`` has the constructor, parameter names (``q``, ``kv``, ``proj``) and return value of the
reference's module (vision_tasks/deit/models.py:215-267), so its ``state_dict`` loads unchanged; it
hands the strided ``k``/``v`` views of the fused projection to the kernels as they are (the reference's
operator copies them first) and can take a partially filled depth cache (``depth_valid``).

``DepthStream`` replaces the model-side loop of vision_tasks/deit/models.py:383-387, which re-stacks the
K/V of all previous layers for every layer:
  * with gradients enabled it keeps the per-layer K/V and builds the token-major cache with the HIP
    reorganisation kernel (differentiable, ``stack_depth``);
  * without gradients it appends each layer in place to one preallocated cache and exposes the number
    of filled slots -- nothing is rebuilt.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch
from torch import nn

from .depth_cache import DepthCache, stack_depth
from .ops import parallel_moda


class DepthStream:
    """Depth K/V of the layers seen so far, in the layout the kernels read.

    ``context()`` -> ``(cached_k, cached_v, depth_valid)`` for the next layer (``(None, None, None)``
    before the first ``push``); ``push(k, v)`` adds one layer's ``[B, T, H, D]`` tensors.
    ``max_layers`` sizes the in-place cache of the no-grad path; ``inplace=False`` forces the rebuilding
    path also without gradients (what the reference does), ``None`` decides by whether gradients flow."""

    def __init__(self, max_layers: int, inplace: Optional[bool] = None):
        self.max_layers = int(max_layers)
        self._layers: List[Tuple[torch.Tensor, torch.Tensor]] = []
        self._cache: Optional[DepthCache] = None
        self._inplace: Optional[bool] = inplace

    def __len__(self):
        if self._inplace:
            return self._cache.n if self._cache is not None else 0
        return len(self._layers)

    def push(self, k: torch.Tensor, v: torch.Tensor):
        if self._inplace is None:
            self._inplace = not (torch.is_grad_enabled() and (k.requires_grad or v.requires_grad))
        if self._inplace:
            if self._cache is None:
                B, T, H, D = k.shape
                self._cache = DepthCache(B, T, self.max_layers, H, D, k.dtype, k.device)
            self._cache.append(k.detach(), v.detach())
        else:
            assert len(self._layers) < self.max_layers, "depth stream is full"
            self._layers.append((k, v))

    def context(self):
        if len(self) == 0:
            return None, None, None
        if self._inplace:
            return self._cache.filled()
        return stack_depth([kv[0] for kv in self._layers]), stack_depth([kv[1] for kv in self._layers]), None


class MoDAAttention(nn.Module):
    """Attention over the sequence and over the depth stream; GQA groups are folded into the query
    rows (``q [B, N*G, num_kv_heads, head_dim]``, ``moda_group_num = G``) exactly as in
    vision_tasks/deit/models.py:244-267.  ``is_causal`` defaults to the vision model's ``False``.

    ``ffn_kv=True`` adds a second projection ``kv_ffn`` and the method ``project_depth_kv`` that maps
    another hidden state (e.g. the block's FFN output) to depth K/V, for callers that also feed the
    depth stream from their feed-forward layers."""

    def __init__(self, dim, num_heads=8, num_kv_heads=1, qkv_bias=False, attn_drop=0., proj_drop=0.,
                 is_causal=False, ffn_kv=False):
        super().__init__()
        if dim % num_heads != 0:
            raise ValueError(f"dim ({dim}) must be divisible by num_heads ({num_heads})")
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads ({num_heads}) must be divisible by num_kv_heads ({num_kv_heads})")
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.moda_group_num = num_heads // num_kv_heads
        self.head_dim = dim // num_heads
        self.scale = self.head_dim ** -0.5
        self.is_causal = is_causal
        self.q = nn.Linear(dim, dim, bias=qkv_bias)
        self.kv = nn.Linear(dim, 2 * num_kv_heads * self.head_dim, bias=qkv_bias)
        self.proj = nn.Linear(dim, dim)
        self.proj_drop = nn.Dropout(proj_drop)
        self.kv_ffn = nn.Linear(dim, 2 * num_kv_heads * self.head_dim, bias=qkv_bias) if ffn_kv else None

    def _split_kv(self, kv: torch.Tensor):
        B, N, _ = kv.shape
        kv = kv.reshape(B, N, 2, self.num_kv_heads, self.head_dim)
        return kv[:, :, 0], kv[:, :, 1]

    def project_depth_kv(self, h: torch.Tensor):
        """Depth K/V ``[B, N, num_kv_heads, head_dim]`` of a hidden state other than the attention input."""
        assert self.kv_ffn is not None, "constructed without ffn_kv=True"
        return self._split_kv(self.kv_ffn(h))

    def forward(self, x, depth_k=None, depth_v=None, depth_valid=None):
        B, N, C = x.shape
        G = self.moda_group_num
        q = self.q(x).reshape(B, N * G, self.num_kv_heads, self.head_dim)
        k, v = self._split_kv(self.kv(x))
        o = parallel_moda(q=q, k=k, v=v, g=None, scale=self.scale, cu_seqlens=None, cached_k=depth_k,
                          cached_v=depth_v, moda_group_num=G, is_causal=self.is_causal, head_first=False,
                          warn_shape=False, depth_valid=depth_valid)
        x = self.proj_drop(self.proj(o.reshape(B, N, C)))
        return x, k, v


class MoDAStack(nn.Module):
    """``depth`` pre-norm blocks (attention + MLP) chained through one ``DepthStream``: the body of
    ``MoDAVisionTransformer.forward_features`` (vision_tasks/deit/models.py:376-390) without the patch
    embedding and the classifier, for timing and testing whole-model steps."""

    def __init__(self, dim, depth, num_heads, num_kv_heads, mlp_ratio=4., qkv_bias=True, is_causal=False):
        super().__init__()
        self.blocks = nn.ModuleList()
        for _ in range(depth):
            blk = nn.Module()
            blk.norm1 = nn.LayerNorm(dim, eps=1e-6)
            blk.attn = MoDAAttention(dim, num_heads, num_kv_heads, qkv_bias=qkv_bias, is_causal=is_causal)
            blk.norm2 = nn.LayerNorm(dim, eps=1e-6)
            hidden = int(dim * mlp_ratio)
            blk.mlp = nn.Sequential(nn.Linear(dim, hidden), nn.GELU(), nn.Linear(hidden, dim))
            self.blocks.append(blk)

    def forward(self, x, inplace_cache: Optional[bool] = None):
        stream = DepthStream(len(self.blocks), inplace=inplace_cache)
        for blk in self.blocks:
            dk, dv, n = stream.context()
            a, k, v = blk.attn(blk.norm1(x), depth_k=dk, depth_v=dv, depth_valid=n)
            x = x + a
            x = x + blk.mlp(blk.norm2(x))
            stream.push(k, v)
        return x
