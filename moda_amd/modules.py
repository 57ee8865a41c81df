"""Caller-side pieces around the attention operator: the attention module of the reference's vision
model and a manager for the depth stream it feeds.

``MoDAAttention`` has the constructor, parameter names (``q``, ``kv``, ``proj``) and return value of the
reference's module (vision_tasks/deit/models.py:215-267), so its ``state_dict`` loads unchanged; it
hands the strided ``k``/``v`` views of the fused projection to the kernels as they are (the reference's
operator copies them first) and can take a partially filled depth cache (``depth_valid``).

``DepthStream`` replaces the model-side loop of vision_tasks/deit/models.py:383-387, which re-stacks the
K/V of all previous layers for every layer (and lets autograd scatter the gradient of every such stack
back): one token-major cache is preallocated per forward pass and each layer's K/V is written into its
slot once.
  * With gradients flowing, a second buffer of the same shape collects the depth gradients: the backward
    of the attention that saw ``n`` slots adds its share to slots ``< n`` (the kernels' accumulate mode),
    and the gradient of a layer's K/V is the slice of that buffer for its slot, read when autograd
    reaches the layer.  Neither direction touches a slot more than once per consumer.
  * Without gradients only the cache is kept.
  * ``inplace=False`` keeps the reference's behaviour (rebuild per layer, differentiable ``stack_depth``).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch
from torch import nn

from . import _lib
from .depth_cache import DepthCache, _reorg_bwd, _reorg_fwd, stack_depth
from .ops import _chunk_tokens, _raw_bwd, _raw_fwd, parallel_moda, parallel_moda_chunk_visible


class _TrainBuffers:
    """Cache and gradient accumulators of one forward/backward pass, ``[B, T*L_max, H, D]`` each.  The
    accumulators start as zeros; the cache needs no initialisation (the kernels never read a slot that has not
    been written: ``depth_valid``)."""

    def __init__(self, B, T, L_max, H, D, dtype, device):
        self.shape, self.L_max = (B, T, H, D), L_max
        self.k = torch.empty(B, T * L_max, H, D, dtype=dtype, device=device)
        self.v = torch.empty_like(self.k)
        self.gk = torch.zeros_like(self.k)
        self.gv = torch.zeros_like(self.k)


class _StreamAttention(torch.autograd.Function):
    """parallel_moda over the sequence and the first ``n`` slots of the stream's cache.  The cache is not an
    autograd input: its gradient goes to the stream's accumulators, from where ``_StreamPush.backward`` of the
    layer that owns a slot hands it on.  ``token`` chains the stream's operations so that autograd runs
    their backward passes in reverse order whatever else connects the layers."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, q, k, v, token, buf, n, scale, G, mode, chunk_tokens):
        o, lse = _raw_fwd(mode, q, k, v, buf.k if n else None, buf.v if n else None, scale, G, chunk_tokens,
                          depth_valid=n if n else None)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.buf, ctx.n, ctx.scale, ctx.G, ctx.mode, ctx.chunk_tokens = buf, n, scale, G, mode, chunk_tokens
        ctx.set_materialize_grads(False)
        ctx.mark_non_differentiable(lse)
        return o, lse, token.new_zeros(())

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, do, _dlse, _dtoken):
        q, k, v, o, lse = ctx.saved_tensors
        buf, n = ctx.buf, ctx.n
        do = torch.zeros_like(o) if do is None else do.to(o.dtype)
        mode, cb = ctx.mode, ctx.chunk_tokens
        dq, dk, dv = torch.empty_like(q), torch.empty(k.shape, dtype=k.dtype, device=k.device), \
            torch.empty(v.shape, dtype=v.dtype, device=v.device)
        if n:
            _raw_bwd(mode, q, k, v, buf.k, buf.v, o, lse, do, ctx.scale, ctx.G, cb, out=(dq, dk, dv, buf.gk, buf.gv),
                     depth_valid=n, accumulate_depth=True)
        else:
            _raw_bwd(mode, q, k, v, None, None, o, lse, do, ctx.scale, ctx.G, cb, out=(dq, dk, dv, None, None))
        return dq, dk, dv, None, None, None, None, None, None, None


class _StreamPush(torch.autograd.Function):
    """Writes one layer's K/V into slot ``slot`` of the cache; its backward returns what the attention calls
    that saw the slot have added to the gradient accumulators (all of them ran before: see ``token``)."""

    @staticmethod
    def forward(ctx, k, v, token, buf, slot):
        _reorg_fwd([k.contiguous()], buf.k, slot, buf.L_max)
        _reorg_fwd([v.contiguous()], buf.v, slot, buf.L_max)
        ctx.buf, ctx.slot = buf, slot
        ctx.set_materialize_grads(False)
        return token.new_zeros(())

    @staticmethod
    def backward(ctx, _dtoken):
        buf = ctx.buf
        (gk,) = _reorg_bwd(buf.gk, 1, ctx.slot, buf.L_max, buf.shape)
        (gv,) = _reorg_bwd(buf.gv, 1, ctx.slot, buf.L_max, buf.shape)
        return gk, gv, None, None, None


class DepthStream:
    """Depth K/V of the layers seen so far, in the layout the kernels read.

    Per layer: ``o = stream.attend(q, k, v, scale=..., moda_group_num=..., is_causal=...)`` (attention over
    the sequence and over everything pushed so far), then ``stream.push(k, v)`` with the layer's
    ``[B, T, H, D]`` tensors (any number of pushes per layer, e.g. K/V projected from the FFN output as
    well).  ``max_layers`` sizes the cache.  ``inplace=None`` keeps one cache in place (with gradient
    accumulators when gradients flow), ``inplace=False`` rebuilds the cache per layer as the reference does.

    ``context()`` -> ``(cached_k, cached_v, depth_valid)`` is the lower-level access for callers that
    invoke ``parallel_moda`` themselves; with gradients flowing it uses the rebuilding path (the in-place
    gradient path needs ``attend``).  One backward pass per forward pass: the accumulators are consumed by it."""

    def __init__(self, max_layers: int, inplace: Optional[bool] = None):
        self.max_layers = int(max_layers)
        self._layers: List[Tuple[torch.Tensor, torch.Tensor]] = []
        self._cache: Optional[DepthCache] = None
        self._train: Optional[_TrainBuffers] = None
        self._token: Optional[torch.Tensor] = None
        self._n = 0
        self._inplace: Optional[bool] = inplace
        self._mode: Optional[str] = None  # 'train' | 'infer' | 'rebuild', fixed by the first push
        self._used_context = False

    def __len__(self):
        return self._n

    def _decide(self, k, v):
        if self._mode is not None:
            return
        grads = torch.is_grad_enabled() and (k.requires_grad or v.requires_grad)
        if self._inplace is False or (grads and self._used_context):
            self._mode = "rebuild"
        else:
            self._mode = "train" if grads else "infer"

    def push(self, k: torch.Tensor, v: torch.Tensor):
        assert self._n < self.max_layers, "depth stream is full"
        self._decide(k, v)
        B, T, H, D = k.shape
        if self._mode == "train":
            if self._train is None:
                self._train = _TrainBuffers(B, T, self.max_layers, H, D, k.dtype, k.device)
                self._token = torch.zeros((), device=k.device)
            self._token = _StreamPush.apply(k, v, self._token, self._train, self._n)
        elif self._mode == "infer":
            if self._cache is None:
                self._cache = DepthCache(B, T, self.max_layers, H, D, k.dtype, k.device)
            self._cache.append(k.detach(), v.detach())
        else:
            self._layers.append((k, v))
        self._n += 1

    def context(self):
        self._used_context = True
        if self._n == 0:
            return None, None, None
        if self._mode == "infer":
            return self._cache.filled()
        assert self._mode == "rebuild", \
            "with gradients flowing through an in-place depth stream use attend(): the depth gradients are " \
            "collected by the stream, not by autograd"
        return stack_depth([kv[0] for kv in self._layers]), stack_depth([kv[1] for kv in self._layers]), None

    def attend(self, q, k, v, scale=None, moda_group_num=1, is_causal=True, chunk_rows=None):
        """``parallel_moda(q, k, v, cached_k, cached_v, ...)`` over what has been pushed so far; with ``chunk_rows``
        (query rows per chunk, the reference's 64) ``parallel_moda_chunk_visible`` instead: a token also sees the
        depth slots of the earlier tokens of its chunk (causal by definition)."""
        chunk_visible = chunk_rows is not None
        assert not chunk_visible or is_causal, "chunk-visible attention is causal"
        if self._mode == "train" or (self._mode is None and self._inplace is not False and not self._used_context
                                     and torch.is_grad_enabled() and (q.requires_grad or k.requires_grad)):
            # the same argument contract as parallel_moda, which is bypassed here
            assert q.shape[2] == k.shape[2] and q.shape[1] == k.shape[1] * moda_group_num, \
                "q must be [B, T*moda_group_num, H, D] for k [B, T, H, D]"
            assert 128 % moda_group_num == 0, \
                "To keep depth alignment consistent with backward, BT % moda_group_num must be 0"
            if scale is None:
                scale = q.shape[-1] ** -0.5
            if self._token is None:
                self._token = torch.zeros((), device=q.device)
            buf = self._train if self._n else None
            mode = _lib.CHUNK_VISIBLE if chunk_visible else _lib.CAUSAL if is_causal else _lib.NONCAUSAL
            cb = _chunk_tokens(moda_group_num, chunk_rows) if chunk_visible else 0
            o, _, self._token = _StreamAttention.apply(q, k, v, self._token, buf, self._n, scale, moda_group_num,
                                                       mode, cb)
            return o
        if self._n == 0:
            dk = dv = n = None
        elif self._mode == "infer":
            dk, dv, n = self._cache.filled()
        else:
            dk, dv = stack_depth([kv[0] for kv in self._layers]), stack_depth([kv[1] for kv in self._layers])
            n = None
        if chunk_visible:
            return parallel_moda_chunk_visible(q=q, k=k, v=v, g=None, scale=scale, cu_seqlens=None, cached_k=dk,
                                               cached_v=dv, moda_group_num=moda_group_num, head_first=False,
                                               warn_shape=False, chunk_rows=chunk_rows, depth_valid=n)
        return parallel_moda(q=q, k=k, v=v, g=None, scale=scale, cu_seqlens=None, cached_k=dk, cached_v=dv,
                             moda_group_num=moda_group_num, is_causal=is_causal, head_first=False, warn_shape=False,
                             depth_valid=n)


class MoDAAttention(nn.Module):
    """Attention over the sequence and over the depth stream; GQA groups are folded into the query
    rows (``q [B, N*G, num_kv_heads, head_dim]``, ``moda_group_num = G``) exactly as in
    vision_tasks/deit/models.py:244-267.  ``is_causal`` defaults to the vision model's ``False``.

    ``forward(x, depth_k, depth_v)`` is the reference's call; ``forward(x, stream=DepthStream)`` attends
    over the stream instead.  Either way the layer's own ``k, v`` are returned for the caller to push.

    ``ffn_kv=True`` adds a second projection ``kv_ffn`` and the method ``project_depth_kv`` that maps
    another hidden state (e.g. the block's FFN output) to depth K/V, for callers that also feed the
    depth stream from their feed-forward layers."""

    def __init__(self, dim, num_heads=8, num_kv_heads=1, qkv_bias=False, attn_drop=0., proj_drop=0.,
                 is_causal=False, ffn_kv=False, chunk_rows=None):
        super().__init__()
        self.chunk_rows = chunk_rows  # not None: chunk-visible attention with chunks of that many query rows
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

    def forward(self, x, depth_k=None, depth_v=None, depth_valid=None, stream: Optional[DepthStream] = None):
        B, N, C = x.shape
        G = self.moda_group_num
        q = self.q(x).reshape(B, N * G, self.num_kv_heads, self.head_dim)
        k, v = self._split_kv(self.kv(x))
        if stream is not None:
            assert depth_k is None and depth_v is None, "pass either a stream or explicit depth tensors"
            o = stream.attend(q, k, v, scale=self.scale, moda_group_num=G, is_causal=self.is_causal,
                              chunk_rows=self.chunk_rows)
        elif self.chunk_rows is not None:
            o = parallel_moda_chunk_visible(q=q, k=k, v=v, g=None, scale=self.scale, cu_seqlens=None, cached_k=depth_k,
                                            cached_v=depth_v, moda_group_num=G, head_first=False, warn_shape=False,
                                            chunk_rows=self.chunk_rows, depth_valid=depth_valid)
        else:
            o = parallel_moda(q=q, k=k, v=v, g=None, scale=self.scale, cu_seqlens=None, cached_k=depth_k,
                              cached_v=depth_v, moda_group_num=G, is_causal=self.is_causal, head_first=False,
                              warn_shape=False, depth_valid=depth_valid)
        x = self.proj_drop(self.proj(o.reshape(B, N, C)))
        return x, k, v


class MoDAStack(nn.Module):
    """``depth`` blocks (attention + MLP) chained through one ``DepthStream``: the body of
    ``MoDAVisionTransformer.forward_features`` (vision_tasks/deit/models.py:376-390) without the patch
    embedding and the classifier, for timing and testing whole-model steps.  Pre-norm blocks as in the
    reference (``x + f(norm(x))``, deit/models.py:288-292) or, with ``post_norm=True``, ``norm(x + f(x))``;
    ``ffn_kv=True`` also pushes K/V projected from every block's output into the stream (two slots per
    block)."""

    def __init__(self, dim, depth, num_heads, num_kv_heads, mlp_ratio=4., qkv_bias=True, is_causal=False,
                 post_norm=False, ffn_kv=False, chunk_rows=None):
        super().__init__()
        self.post_norm, self.ffn_kv = post_norm, ffn_kv
        self.blocks = nn.ModuleList()
        for _ in range(depth):
            blk = nn.Module()
            blk.norm1 = nn.LayerNorm(dim, eps=1e-6)
            blk.attn = MoDAAttention(dim, num_heads, num_kv_heads, qkv_bias=qkv_bias, is_causal=is_causal,
                                     ffn_kv=ffn_kv, chunk_rows=chunk_rows)
            blk.norm2 = nn.LayerNorm(dim, eps=1e-6)
            hidden = int(dim * mlp_ratio)
            blk.mlp = nn.Sequential(nn.Linear(dim, hidden), nn.GELU(), nn.Linear(hidden, dim))
            self.blocks.append(blk)

    def forward(self, x, inplace_cache: Optional[bool] = None):
        stream = DepthStream(len(self.blocks) * (2 if self.ffn_kv else 1), inplace=inplace_cache)
        for blk in self.blocks:
            if self.post_norm:
                a, k, v = blk.attn(x, stream=stream)
                x = blk.norm1(x + a)
                x = blk.norm2(x + blk.mlp(x))
            else:
                a, k, v = blk.attn(blk.norm1(x), stream=stream)
                x = x + a
                x = x + blk.mlp(blk.norm2(x))
            stream.push(k, v)
            if self.ffn_kv:
                stream.push(*blk.attn.project_depth_kv(x))
        return x
