"""Depth-KV cache in the token-major layout the attention kernels read.

``build_depth_cache`` replaces the caller-side
``torch.stack(dim=2).reshape(B, N*L, H, K).contiguous()`` of
vision_tasks/deit/models.py:361-375 with one HBM-bound HIP copy kernel per
tensor (and its transpose in backward).  ``DepthCache`` goes one step further:
a preallocated ``[B, T, L_max, H, D]`` buffer to which each layer's K/V is
appended in place, so the cache is never rebuilt.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from .ops import _DTYPES, _check_device, _stream


def _ptr_array(tensors: Sequence[torch.Tensor]):
    arr = (ctypes.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr()
    return arr


def _reorg_fwd(layers: Sequence[torch.Tensor], cache: torch.Tensor, slot0: int, L_total: int):
    B, T, H, D = layers[0].shape
    # the C ABI sees bare pointers: every extent it will touch is checked here
    assert tuple(cache.shape) == (B, T * L_total, H, D) and cache.is_contiguous(), \
        f"cache must be a contiguous {(B, T * L_total, H, D)} tensor, got {tuple(cache.shape)}"
    assert 0 <= slot0 and slot0 + len(layers) <= L_total, "slots out of range"
    for x in layers:
        assert tuple(x.shape) == (B, T, H, D) and x.is_contiguous(), "every layer must be a contiguous [B, T, H, D] tensor"
        assert x.dtype == cache.dtype and x.device == cache.device, "layers and cache must share dtype and device"
    _check_device(cache)
    with torch.cuda.device(cache.device):
        rc = _lib.load().moda_hip_depth_reorg_fwd(_ptr_array(layers), len(layers), slot0, L_total, B, T, H, D,
                                                  _DTYPES[cache.dtype], ctypes.c_void_p(cache.data_ptr()),
                                                  _stream(cache))
    _lib.check(rc, "moda_hip_depth_reorg_fwd")


def _reorg_bwd(d_cache: torch.Tensor, n_layers: int, slot0: int, L_total: int, shape) -> List[torch.Tensor]:
    B, T, H, D = shape
    assert tuple(d_cache.shape) == (B, T * L_total, H, D) and d_cache.is_contiguous(), \
        f"d_cache must be a contiguous {(B, T * L_total, H, D)} tensor, got {tuple(d_cache.shape)}"
    assert 0 <= slot0 and slot0 + n_layers <= L_total, "slots out of range"
    _check_device(d_cache)
    outs = [torch.empty(B, T, H, D, dtype=d_cache.dtype, device=d_cache.device) for _ in range(n_layers)]
    with torch.cuda.device(d_cache.device):
        rc = _lib.load().moda_hip_depth_reorg_bwd(ctypes.c_void_p(d_cache.data_ptr()), n_layers, slot0, L_total, B, T,
                                                  H, D, _DTYPES[d_cache.dtype], _ptr_array(outs), _stream(d_cache))
    _lib.check(rc, "moda_hip_depth_reorg_bwd")
    return outs


class _StackDepth(torch.autograd.Function):
    @staticmethod
    def forward(ctx, *layers):
        _check_device(layers[0])
        layers = [x.contiguous() for x in layers]
        B, T, H, D = layers[0].shape
        L = len(layers)
        for x in layers:
            assert x.shape == (B, T, H, D) and x.dtype == layers[0].dtype, "all layers must share shape and dtype"
        cache = torch.empty(B, T * L, H, D, dtype=layers[0].dtype, device=layers[0].device)
        _reorg_fwd(layers, cache, 0, L)
        ctx.shape = (B, T, H, D)
        ctx.L = L
        return cache

    @staticmethod
    def backward(ctx, d_cache):
        return tuple(_reorg_bwd(d_cache.contiguous(), ctx.L, 0, ctx.L, ctx.shape))


def stack_depth(layers: Sequence[torch.Tensor]) -> torch.Tensor:
    """``L`` tensors ``[B,T,H,D]`` -> ``[B, T*L, H, D]`` with row ``t*L + l`` = layer ``l`` of token ``t``."""
    return _StackDepth.apply(*layers)


def build_depth_cache(kv_list: Sequence[Tuple[torch.Tensor, torch.Tensor]]):
    """Drop-in for ``MoDAVisionTransformer._build_depth_cache`` (deit/models.py:361-375)."""
    if not kv_list:
        return None, None
    return stack_depth([kv[0] for kv in kv_list]), stack_depth([kv[1] for kv in kv_list])


class DepthCache:
    """Preallocated depth stream: ``append`` writes one layer's K and V into its
    slot of the token-major buffers.  ``filled()`` returns ``(k, v, n)``: the whole
    ``[B, T*L_max, H, D]`` buffers and the number of slots written so far, to be
    passed as ``cached_k, cached_v, depth_valid=n`` -- nothing is copied or rebuilt
    between layers (the reference re-stacks all previous layers for every layer,
    vision_tasks/deit/models.py:383-387).  The buffers are not initialised: the kernels
    never read a slot that has not been written.  Inference/no-grad use only: ``append``
    writes in place."""

    def __init__(self, B: int, T: int, L_max: int, H: int, D: int, dtype, device):
        self.shape = (B, T, H, D)
        self.L_max = L_max
        self.k = torch.empty(B, T * L_max, H, D, dtype=dtype, device=device)
        self.v = torch.empty(B, T * L_max, H, D, dtype=dtype, device=device)
        self.n = 0

    def append(self, k: torch.Tensor, v: torch.Tensor):
        assert self.n < self.L_max, "depth cache is full"
        for name, x in (("k", k), ("v", v)):
            assert tuple(x.shape) == self.shape, f"{name} must be {self.shape} like the cache, got {tuple(x.shape)}"
            assert x.dtype == self.k.dtype and x.device == self.k.device, \
                f"{name} must have the cache's dtype ({self.k.dtype}) and device"
        _reorg_fwd([k.contiguous()], self.k, self.n, self.L_max)
        _reorg_fwd([v.contiguous()], self.v, self.n, self.L_max)
        self.n += 1

    def filled(self):
        assert self.n > 0, "depth cache is empty"
        return self.k, self.v, self.n

    def full(self):
        assert self.n == self.L_max
        return self.k, self.v
