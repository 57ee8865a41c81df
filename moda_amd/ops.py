"""Host side of the fused sequence+depth attention operators.

Mirrors the reference's Python operator interface -- same function names,
argument meaning, assertions and return conventions -- on top of the C ABI of
``libmoda_hip.so``:

  * ``parallel_moda`` / ``parallel_moda_fwd`` / ``parallel_moda_bwd``
    (libs/moda_triton/fla/ops/moda/moda_v14.py:2792-2893, 381-522, 1470-1842)
  * ``parallel_moda_chunk_visible`` / ``_fwd`` / ``_bwd``
    (moda_v16.py:3614-3651, 498-633, 2099-2343)
  * ``parallel_fda`` / ``_fwd`` / ``_bwd`` (fda_v12.py:1346-1449, 261-400, 881-1135)
  * ``parallel_attn`` (fla/ops/attn/parallel.py:678-730), the plain causal comparator.

Tensors stay torch tensors; torch is used for allocation, streams and autograd
only.  Every compute step is a HIP kernel of the shared library.
"""
from __future__ import annotations

import ctypes
import warnings
from typing import NamedTuple, Optional, Tuple

import torch

from . import _lib
from ._lib import Desc, Strides

_DTYPES = {torch.bfloat16: _lib.BF16, torch.float16: _lib.FP16, torch.float32: _lib.FP32}

# How fp32 tensors are computed.  "fp32": in fp32 on the vector-ALU kernels (exact to fp32 rounding, two orders of
# magnitude slower than the matrix kernels).  "fp16" / "bf16": the inputs are rounded to that type, the matrix
# kernels run, the results are widened again.  "fp16" is what the reference's own fp32 path amounts to: its
# tl.dot calls (moda_v14.py:188, 209, 699-712) take the default input precision, which rounds fp32 operands to a
# 10-bit mantissa (TF32) and accumulates in fp32 -- fp16 has the same mantissa; its range (6e-8 .. 65504) is the
# caller's responsibility, "bf16" trades three mantissa bits for the fp32 range.
_FP32_COMPUTE = "fp32"
_FP32_COMPUTE_TYPES = {"fp16": torch.float16, "bf16": torch.bfloat16}


def set_fp32_compute(mode: str) -> str:
    """Choose how fp32 tensors are computed ("fp32", "fp16" or "bf16", see above); returns the previous setting."""
    global _FP32_COMPUTE
    assert mode in ("fp32", "fp16", "bf16"), f"unknown fp32 compute mode {mode!r}"
    previous, _FP32_COMPUTE = _FP32_COMPUTE, mode
    return previous


def _narrowed(*xs):
    """fp32 tensors -> the 16-bit compute type chosen with set_fp32_compute (None stays None)."""
    t = _FP32_COMPUTE_TYPES[_FP32_COMPUTE]
    return tuple(None if x is None else x.to(t) for x in xs)


# Query rows per chunk of the chunk-visible variant when the caller does not
# say: the value the reference hard-wires in its launchers (moda_v16.py:581-585).
DEFAULT_CHUNK_ROWS = 64


class PackedBatch(NamedTuple):
    """A variable-length batch on one packed token axis, as the kernels take it."""
    cu: torch.Tensor  # int32 [n + 1] on the device: first base token of each sequence, then the total
    n: int            # sequences
    max_len: int      # base tokens of the longest sequence
    total: int        # base tokens in the packed axis
    host: object = None  # ctypes int32 array [n + 1]: the offsets again, in host memory (the library checks them and
                         # can launch per sequence where it has no packed kernel)


def _packed(cu_seqlens, q: torch.Tensor, rows_per_token: int) -> Optional[PackedBatch]:
    """``cu_seqlens`` as a caller passes it (fla's convention: cumulative sequence lengths, first entry 0,
    tensors of batch size 1 holding all sequences back to back) -> PackedBatch.  The offsets count BASE
    TOKENS, i.e. rows of k/v; sequence i owns query rows ``cu[i]*G .. cu[i+1]*G`` and depth rows
    ``cu[i]*L .. cu[i+1]*L``.  The reference carries the argument but asserts it away
    (moda_v14.py:2672-2673); its dormant kernel code reads the offsets in query rows (moda_v14.py:83-101),
    which is the same thing for ``moda_group_num == 1``.  Costs one device-to-host copy of the offsets
    (the longest sequence sizes the launch); pass the returned PackedBatch instead of the tensor to reuse it."""
    if cu_seqlens is None or isinstance(cu_seqlens, PackedBatch):
        return cu_seqlens
    assert q.shape[0] == 1, "with cu_seqlens all sequences share one packed row axis: batch size must be 1"
    assert cu_seqlens.dim() == 1 and cu_seqlens.numel() >= 1, "cu_seqlens must be a vector of n+1 offsets"
    host = cu_seqlens.detach().to("cpu", torch.int64)
    lens = host[1:] - host[:-1]
    assert int(host[0]) == 0 and bool((lens >= 0).all()), "cu_seqlens must start at 0 and not decrease"
    total = int(host[-1])
    assert total * rows_per_token == q.shape[1], (
        f"cu_seqlens ends at {total} base tokens but q holds {q.shape[1]} rows "
        f"({rows_per_token} per token)")
    cu = cu_seqlens.detach().to(device=q.device, dtype=torch.int32).contiguous()
    host_arr = (ctypes.c_int32 * host.numel())(*host.tolist())
    return PackedBatch(cu, int(lens.numel()), int(lens.max()) if lens.numel() else 0, total, host_arr)


def _ptr(x: Optional[torch.Tensor]):
    return ctypes.c_void_p(x.data_ptr()) if x is not None else ctypes.c_void_p(0)


def _stream(x: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)


def _usable(x: Optional[torch.Tensor], vec16: bool = True) -> Optional[torch.Tensor]:
    """Return ``x`` if the kernels can read it in place (unit inner stride, 16-byte
    aligned rows), else a contiguous copy -- the reference's ``@contiguous``
    (fla/utils.py:130-164) made a copy of every non-contiguous input.  ``vec16=False``: the
    vector-ALU kernels, which load element by element and take any non-negative strides."""
    if x is None:
        return None
    if not vec16:
        ok = x.dim() == 4 and (x.stride(3) == 1 or x.shape[3] == 1) and all(x.stride(i) >= 0 for i in range(3))
        return x if ok else x.contiguous()
    m = 16 // x.element_size()
    ok = (
        x.dim() == 4
        and (x.stride(3) == 1 or x.shape[3] == 1)
        and all(x.stride(i) % m == 0 for i in range(3))
        and x.data_ptr() % 16 == 0
        and all(x.stride(i) >= 0 for i in range(3))
        and x.stride(1) * x.element_size() < (1 << 24)  # row offsets inside a tile are 32-bit
    )
    return x if ok else x.contiguous()


def _matrix_core_path(q: torch.Tensor, val: torch.Tensor, packed: Optional["PackedBatch"] = None) -> bool:
    """Whether the call runs on the matrix-core kernels, whose rows must be 16-byte aligned.  The rule is the
    library's own (``moda_hip_uses_matrix_cores``): it is asked with a descriptor that carries what the rule reads
    -- dtype, head dims, whether the batch is packed and has host offsets."""
    if q.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {q.dtype}; expected bf16, fp16 or fp32")
    d = Desc()
    d.struct_size = ctypes.sizeof(Desc)
    d.dtype = _DTYPES[q.dtype]
    d.mode = _lib.NONCAUSAL
    d.B = d.T = d.H = d.G = 1
    d.D, d.Dv = q.shape[3], val.shape[3]
    d.scale = 1.0
    if packed is not None:
        d.B, d.T, d.total_tokens = packed.n, packed.max_len, packed.total
        d.cu_seqlens = packed.cu.data_ptr()
        if packed.host is not None:
            d.cu_seqlens_host = ctypes.cast(packed.host, ctypes.c_void_p)
    rc = _lib.load().moda_hip_uses_matrix_cores(ctypes.byref(d))
    if rc < 0:  # a head dim the library rejects: the launch itself will report it
        return False
    return rc == 1


def _strides(x: Optional[torch.Tensor]) -> Strides:
    if x is None:
        return Strides(0, 0, 0)
    return Strides(x.stride(0), x.stride(1), x.stride(2))


def _check_device(x: torch.Tensor):
    if not x.is_cuda:
        raise RuntimeError(
            "moda_amd operators run only on an MI355X (gfx950) device tensor; there is no CPU path"
        )


def _desc(mode, q, k, v, kd, vd, G, L, chunk_tokens, scale, o=None, do=None, dq=None, dk=None, dv=None, dkd=None,
          dvd=None, depth_valid=None, packed: Optional[PackedBatch] = None, accumulate_depth=False) -> Desc:
    d = Desc()
    d.struct_size = ctypes.sizeof(Desc)
    if q.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {q.dtype}; expected bf16, fp16 or fp32")
    d.dtype = _DTYPES[q.dtype]
    d.mode = mode
    src = kd if mode == _lib.DEPTH_ONLY else k
    d.B = q.shape[0]
    d.H = src.shape[2]
    d.G = G
    d.D = q.shape[3]
    val = vd if mode == _lib.DEPTH_ONLY else v
    d.Dv = val.shape[3]
    d.L = L
    if depth_valid is not None and L > 0:
        assert 1 <= depth_valid <= L, f"depth_valid must be in [1, {L}], got {depth_valid}"
        d.L_valid = int(depth_valid)
    if mode == _lib.DEPTH_ONLY:
        d.T = q.shape[1] // G
    else:
        d.T = k.shape[1]
    if packed is not None:
        d.B, d.T = packed.n, packed.max_len
        d.cu_seqlens = packed.cu.data_ptr()
        d.total_tokens = packed.total
        if packed.host is not None:
            d.cu_seqlens_host = ctypes.cast(packed.host, ctypes.c_void_p)
    d.chunk_tokens = chunk_tokens
    d.flags = _lib.FLAG_ACCUMULATE_DEPTH_GRADS if accumulate_depth else 0
    d.scale = float(scale)
    d.q, d.k, d.v, d.kd, d.vd = _strides(q), _strides(k), _strides(v), _strides(kd), _strides(vd)
    d.o, d.d_o = _strides(o), _strides(do)
    d.dq, d.dk, d.dv, d.dkd, d.dvd = _strides(dq), _strides(dk), _strides(dv), _strides(dkd), _strides(dvd)
    return d


def _same_dtype(*xs):
    dt = None
    for x in xs:
        if x is None:
            continue
        if dt is None:
            dt = x.dtype
        elif x.dtype != dt:
            raise TypeError(f"all tensors must share one dtype, got {dt} and {x.dtype}")


def _check_shapes(mode, q, k, v, kd, vd, G, o=None, do=None, lse=None):
    """The C ABI takes bare pointers: it derives every extent from ``k`` (or ``q``), ``G`` and the depth
    row count and cannot see what the buffers really hold.  A mismatch would be an out-of-bounds access
    on the device, so every extent is checked here, before any launch.  Returns ``(T, L)``."""
    assert q.dim() == 4, "q must be [B, rows, heads, D]"
    B = q.shape[0]
    assert G >= 1, "moda_group_num must be positive"
    if mode == _lib.DEPTH_ONLY:
        assert k is None and v is None, "depth-only attention takes no sequence k/v"
        assert kd is not None and vd is not None, "depth-only attention needs the depth k/v"
        assert q.shape[1] % G == 0, "query rows must be a multiple of moda_group_num"
        T, H = q.shape[1] // G, kd.shape[2]
        assert q.shape[2] == H, "q and depth k/v must have the same number of heads"
    else:
        assert k is not None and v is not None and k.dim() == 4 and v.dim() == 4, "k, v must be [B, T, H, D]"
        T, H = k.shape[1], k.shape[2]
        assert k.shape[0] == B and v.shape[0] == B, "batch sizes of q, k, v differ"
        assert v.shape[1] == T and v.shape[2] == H, "k and v must agree in tokens and heads"
        assert k.shape[3] == q.shape[3], "q and k must share the head dim"
        if mode == _lib.PLAIN_GQA:
            assert q.shape[1] == T and q.shape[2] == H * G, "plain GQA: q must be [B, T, H*G, D]"
        else:
            assert q.shape[2] == H, "folded layout: q and k must have the same number of heads"
            assert q.shape[1] == T * G, f"q holds {q.shape[1]} rows, expected T*moda_group_num = {T * G}"
    L = 0
    if kd is not None or vd is not None:
        assert kd is not None and vd is not None, "depth k and v must be given together"
        assert kd.dim() == 4 and vd.dim() == 4, "depth k/v must be [B, T*L, H, D]"
        assert kd.shape[0] == B and vd.shape[0] == B, "depth k/v batch size differs from q"
        assert kd.shape[2] == H and vd.shape[2] == H, "depth k/v head count mismatch"
        assert kd.shape[3] == q.shape[3], "depth k must share q's head dim"
        assert vd.shape[1] == kd.shape[1], "depth k and v must have the same number of rows"
        if T > 0:
            assert kd.shape[1] % T == 0, "depth rows must be T * L"
            L = kd.shape[1] // T
        else:
            assert kd.shape[1] == 0, "depth rows must be T * L"
        if v is not None:
            assert vd.shape[3] == v.shape[3], "v and depth v must share the value head dim"
    Dv = (vd if mode == _lib.DEPTH_ONLY else v).shape[3]
    for name, x in (("o", o), ("do", do)):
        if x is not None:
            assert tuple(x.shape) == (B, q.shape[1], q.shape[2], Dv), f"{name} must be {(B, q.shape[1], q.shape[2], Dv)}"
    if lse is not None:
        assert tuple(lse.shape) == (B, q.shape[1], q.shape[2]) and lse.dtype == torch.float32, \
            "lse must be fp32 [B, rows, heads]"
    return T, L


def _raw_fwd(mode, q, k, v, kd, vd, scale, G, chunk_tokens=0, depth_valid=None, packed=None):
    """Launch the forward kernels. Returns (o, lse)."""
    if q.dtype == torch.float32 and _FP32_COMPUTE != "fp32":
        o, lse = _raw_fwd(mode, *_narrowed(q, k, v, kd, vd), scale, G, chunk_tokens, depth_valid, packed)
        return o.float(), lse
    _check_shapes(mode, q, k, v, kd, vd, G)
    _check_device(q)
    _same_dtype(q, k, v, kd, vd)
    vec16 = _matrix_core_path(q, vd if mode == _lib.DEPTH_ONLY else v, packed)
    q, k, v, kd, vd = (_usable(x, vec16) for x in (q, k, v, kd, vd))
    src = kd if mode == _lib.DEPTH_ONLY else k
    T = q.shape[1] // G if mode == _lib.DEPTH_ONLY else k.shape[1]
    L = (kd.shape[1] // T) if (kd is not None and T > 0) else 0
    if kd is not None and T == 0:
        L = 0
    val = vd if mode == _lib.DEPTH_ONLY else v
    o = torch.empty(q.shape[0], q.shape[1], q.shape[2], val.shape[-1], dtype=val.dtype, device=q.device)
    lse = torch.empty(q.shape[0], q.shape[1], q.shape[2], dtype=torch.float32, device=q.device)
    if L == 0:
        kd = vd = None
    d = _desc(mode, q, k, v, kd, vd, G, L, chunk_tokens, scale, o=o, depth_valid=depth_valid, packed=packed)
    with torch.cuda.device(q.device):
        rc = _lib.load().moda_hip_fwd(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(kd), _ptr(vd), _ptr(o),
                                      _ptr(lse), _stream(q))
    _lib.check(rc, "moda_hip_fwd")
    return o, lse


def _raw_bwd(mode, q, k, v, kd, vd, o, lse, do, scale, G, chunk_tokens=0, stages=_lib.STAGE_ALL, out=None, ws=None,
             depth_valid=None, packed=None, accumulate_depth=False):
    """Launch the backward kernels. Returns (dq, dk, dv, dkd, dvd).

    ``stages`` selects a subset of {delta, dq, dk/dv}; ``out`` (a previous return
    value) and ``ws`` (a workspace tensor) let the caller reuse buffers across calls.
    ``accumulate_depth``: the depth gradients are ADDED to the ``dkd, dvd`` given in ``out`` (slots
    ``>= depth_valid`` untouched) instead of overwriting them."""
    assert not accumulate_depth or (out is not None and out[3] is not None and out[4] is not None), \
        "accumulate_depth needs the gradient buffers to add to"
    if q.dtype == torch.float32 and _FP32_COMPUTE != "fp32":
        # 16-bit gradients from the matrix kernels (without the accumulate flag: the slots without data come back
        # as zeros), widened into the caller's fp32 buffers or added to them
        got = _raw_bwd(mode, *_narrowed(q, k, v, kd, vd, o), lse, *_narrowed(do), scale, G, chunk_tokens, stages,
                       None, None, depth_valid, packed, False)
        if out is None:
            return tuple(None if g_ is None else g_.float() for g_ in got)
        for i, (dst, g_) in enumerate(zip(out, got)):
            if dst is not None:
                dst.add_(g_) if (accumulate_depth and i >= 3) else dst.copy_(g_)
        return tuple(out)
    _check_shapes(mode, q, k, v, kd, vd, G, o=o, do=do, lse=lse)
    _check_device(q)
    _same_dtype(q, k, v, kd, vd, o, do)
    vec16 = _matrix_core_path(q, vd if mode == _lib.DEPTH_ONLY else v, packed)
    q, k, v, kd, vd, o, do = (_usable(x, vec16) for x in (q, k, v, kd, vd, o, do))
    lse = lse.contiguous()
    T = q.shape[1] // G if mode == _lib.DEPTH_ONLY else k.shape[1]
    L = (kd.shape[1] // T) if (kd is not None and T > 0) else 0
    if out is not None:
        dq, dk, dv, dkd, dvd = out
        for g_, x_ in ((dq, q), (dk, k), (dv, v), (dkd, kd), (dvd, vd)):
            assert (g_ is None) == (x_ is None) and (g_ is None or (g_.shape == x_.shape and g_.dtype == x_.dtype)), \
                "reused gradient buffers must match their inputs in shape and dtype"
    else:
        dq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        dk = torch.empty(k.shape, dtype=k.dtype, device=q.device) if k is not None else None
        dv = torch.empty(v.shape, dtype=v.dtype, device=q.device) if v is not None else None
        dkd = torch.empty(kd.shape, dtype=kd.dtype, device=q.device) if kd is not None else None
        dvd = torch.empty(vd.shape, dtype=vd.dtype, device=q.device) if vd is not None else None
    kd_a, vd_a, dkd_a, dvd_a = (kd, vd, dkd, dvd) if L > 0 else (None, None, None, None)
    d = _desc(mode, q, k, v, kd_a, vd_a, G, L, chunk_tokens, scale, o=o, do=do, dq=dq, dk=dk, dv=dv, dkd=dkd_a,
              dvd=dvd_a, depth_valid=depth_valid, packed=packed, accumulate_depth=accumulate_depth and L > 0)
    lib = _lib.load()
    nbytes = lib.moda_hip_bwd_workspace_bytes(ctypes.byref(d))
    if ws is None:
        ws = torch.empty(max(int(nbytes), 4), dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        rc = lib.moda_hip_bwd_stages(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(kd_a), _ptr(vd_a), _ptr(o),
                                     _ptr(lse), _ptr(do), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(dkd_a), _ptr(dvd_a),
                                     _ptr(ws), ctypes.c_size_t(ws.numel() * ws.element_size()), int(stages),
                                     _stream(q))
    _lib.check(rc, "moda_hip_bwd")
    return dq, dk, dv, dkd, dvd


def bwd_workspace(mode, q, k, v, kd, vd, G, chunk_tokens=0, packed=None) -> torch.Tensor:
    """A workspace tensor of the size the backward asks for, for callers that reuse one across calls (``ws=``)."""
    T, L = _check_shapes(mode, q, k, v, kd, vd, G)
    kd_a, vd_a = (kd, vd) if L > 0 else (None, None)
    d = _desc(mode, q, k, v, kd_a, vd_a, G, L, chunk_tokens, 1.0, packed=packed)
    nbytes = _lib.load().moda_hip_bwd_workspace_bytes(ctypes.byref(d))
    return torch.empty(max(int(nbytes), 4), dtype=torch.uint8, device=q.device)


# ---------------------------------------------------------------------------
# MoDA (causal / non-causal)  -- moda_v14.py
# ---------------------------------------------------------------------------
def _assert_group_tile(moda_group_num: int, rows: int = 128):
    assert (
        rows % moda_group_num == 0
    ), "To keep depth alignment consistent with backward, BT % moda_group_num must be 0"


def parallel_moda_fwd(q, k, v, g_cumsum, scale, cu_seqlens=None, cached_k=None, cached_v=None, moda_group_num=1,
                      is_causal=True, customized_BT=None, customized_BS=None, customized_BK=None, customized_BV=None,
                      customized_num_warps=None, depth_valid=None):
    """moda_v14.py:381-522.  Returns ``(o, lse)``; tile-size knobs are accepted and ignored.
    ``depth_valid`` (not in the reference): only the first ``depth_valid`` of the ``L`` slots per token
    of ``cached_k/v`` are visible."""
    assert g_cumsum is None, "g_cumsum is not supported in this version"
    assert q.shape[2] == k.shape[2], (
        "Implicit head-dimension GQA is not allowed. "
        "Please fold grouping only into `moda_group_num`: "
        "use q.shape[2] == k.shape[2] and set T_q = T_kv * moda_group_num."
    )
    _assert_group_tile(moda_group_num)
    mode = _lib.CAUSAL if is_causal else _lib.NONCAUSAL
    return _raw_fwd(mode, q, k, v, cached_k, cached_v, scale, moda_group_num, depth_valid=depth_valid,
                    packed=_packed(cu_seqlens, q, moda_group_num))


def parallel_moda_bwd(q, k, v, o, g_cumsum, lse, do, scale=None, chunk_size=128, cu_seqlens=None, cached_k=None,
                      cached_v=None, moda_group_num=1, is_causal=True, customized_BT=None, customized_BS=None,
                      customized_BK=None, customized_BV=None, customized_num_warps=None, group_bs=None,
                      group_warps=None, depth_bs=None, depth_warps=None, depth_valid=None):
    """moda_v14.py:1470-1842.  Returns ``(dq, dk, dv, dg_cumsum=None, d_cached_k, d_cached_v)``."""
    assert g_cumsum is None, "g_cumsum is not supported in this version"
    assert q.shape[2] == k.shape[2], (
        "Implicit head-dimension GQA is not allowed. "
        "Please fold grouping only into `moda_group_num`: "
        "use q.shape[2] == k.shape[2] and set T_q = T_kv * moda_group_num."
    )
    if scale is None:
        scale = q.shape[-1] ** -0.5
    _assert_group_tile(moda_group_num)
    mode = _lib.CAUSAL if is_causal else _lib.NONCAUSAL
    dq, dk, dv, dkd, dvd = _raw_bwd(mode, q, k, v, cached_k, cached_v, o, lse, do, scale, moda_group_num,
                                    depth_valid=depth_valid, packed=_packed(cu_seqlens, q, moda_group_num))
    return dq, dk, dv, None, dkd, dvd


def _autograd_forward(ctx, fwd_impl, q, k, v, g, scale, cu_seqlens, cached_k, cached_v, moda_group_num, **kw):
    assert g is None, "g is not supported in this version"
    packed = _packed(cu_seqlens, q, moda_group_num)
    has_depth = cached_k is not None and cached_v is not None
    if not has_depth:
        cached_k = cached_v = None
    o, lse = fwd_impl(q=q, k=k, v=v, g_cumsum=None, scale=scale, cu_seqlens=packed, cached_k=cached_k,
                      cached_v=cached_v, moda_group_num=moda_group_num, **kw)
    ctx.packed = packed
    ctx.save_for_backward(q, k, v, o, lse, *([cached_k, cached_v] if has_depth else []))
    ctx.has_depth = has_depth
    ctx.scale = scale
    ctx.moda_group_num = moda_group_num
    ctx.kw = kw
    return o.to(q.dtype), lse


def _autograd_backward(ctx, bwd_impl, do):
    if ctx.has_depth:
        q, k, v, o, lse, cached_k, cached_v = ctx.saved_tensors
    else:
        q, k, v, o, lse = ctx.saved_tensors
        cached_k = cached_v = None
    dq, dk, dv, _, dkd, dvd = bwd_impl(q=q, k=k, v=v, o=o, g_cumsum=None, lse=lse, do=do.to(o.dtype), scale=ctx.scale,
                                       cu_seqlens=ctx.packed, cached_k=cached_k, cached_v=cached_v,
                                       moda_group_num=ctx.moda_group_num, **ctx.kw)
    if not ctx.has_depth:
        dkd = dvd = None
    return dq.to(q), dk.to(k), dv.to(v), dkd, dvd


class ParallelMixtureOfDepthAttentionFunction(torch.autograd.Function):
    """moda_v14.py:2649-2789: 14 inputs, 14 gradients, gradient into ``lse`` ignored."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, q, k, v, g, scale, cu_seqlens, cached_k=None, cached_v=None, moda_group_num=1, is_causal=True,
                group_bs=None, group_warps=None, depth_bs=None, depth_warps=None, depth_valid=None):
        o, lse = _autograd_forward(ctx, parallel_moda_fwd, q, k, v, g, scale, cu_seqlens, cached_k, cached_v,
                                   moda_group_num, is_causal=is_causal, depth_valid=depth_valid)
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, do, dlse_unused):
        dq, dk, dv, dkd, dvd = _autograd_backward(ctx, parallel_moda_bwd, do)
        return dq, dk, dv, None, None, None, dkd, dvd, None, None, None, None, None, None, None


def _prepare_inputs(api_name, q, k, v, g, cached_k, cached_v, scale, moda_group_num, head_first,
                    return_depth_grads, warn_shape):
    """Shared argument contract of parallel_moda (moda_v14.py:2817-2871) and
    parallel_moda_chunk_visible (moda_v16.py:3496-3565)."""
    if head_first:
        q = q.transpose(1, 2)
        k = k.transpose(1, 2)
        v = v.transpose(1, 2)
        if g is not None:
            g = g.transpose(1, 2)
        if cached_k is not None and cached_v is not None:
            cached_k = cached_k.transpose(1, 2)
            cached_v = cached_v.transpose(1, 2)
    elif warn_shape and q.shape[1] < q.shape[2]:
        warnings.warn(
            f"[{api_name}] detected seq_len({q.shape[1]}) < num_heads({q.shape[2]}). "
            "input may be in head_first format while head_first=True is not set."
        )
    B, T_q, HQ, Kdim = q.shape
    T_kv = k.shape[1]
    H = k.shape[2]
    assert HQ == H, (
        "Implicit head-dimension GQA is not allowed. "
        "Please fold grouping only into `moda_group_num`: "
        "use q.shape[2] == k.shape[2] and set T_q = T_kv * moda_group_num."
    )
    if scale is None:
        scale = Kdim ** -0.5
    if moda_group_num > 1:
        assert T_q == T_kv * moda_group_num, "When moda_group_num > 1, T_q must equal T_kv * moda_group_num"
    else:
        assert T_q == T_kv, "When moda_group_num=1, T_q must equal T_kv"
    if cached_k is not None and cached_v is not None:
        assert cached_k.shape[0] == B and cached_v.shape[0] == B
        assert cached_k.shape[2] == H and cached_v.shape[2] == H, "cached_k/v head count mismatch"
        assert cached_k.shape[1] % T_kv == 0, "cached_k time dimension must be T_kv * L"
        L = cached_k.shape[1] // T_kv
        assert cached_v.shape[1] == T_kv * L, "cached_v shape mismatch"
        if (cached_k.requires_grad or cached_v.requires_grad) and not return_depth_grads:
            warnings.warn(
                "cached_k/v requires gradients, but return_depth_grads=False. "
                "Gradients are still computed and returned."
            )
    if g is not None:
        assert g.shape[:3] == (B, T_q, HQ), "g must be [B,T_q,HQ]"
    return q, k, v, g, cached_k, cached_v, scale


def parallel_moda(q, k, v, g=None, cached_k=None, cached_v=None, scale=None, cu_seqlens=None, moda_group_num=1,
                  is_causal=True, head_first=False, need_lse=False, return_depth_grads=True, warn_shape=True,
                  customized_BT=None, customized_BS=None, customized_BT_backward=None, customized_BS_backward=None,
                  group_bs=None, group_warps=None, depth_bs=None, depth_warps=None, depth_valid=None):
    """Fused sequence+depth attention; signature of moda_v14.py:2792-2815, plus ``depth_valid``.

    q ``[B, T*G, H, D]``; k, v ``[B, T, H, D]``; cached_k/v ``[B, T*L, H, D]`` or
    None.  Returns ``o`` (q.dtype) or ``(o, lse)`` with ``lse`` fp32 in base-2
    units.  The ``customized_*``, ``group_*`` and ``depth_*`` knobs tune the
    reference's Triton launches and have no meaning here; they are accepted and
    ignored.  ``depth_valid`` (an extension): ``cached_k/v`` keep ``L`` slots per token
    but only the first ``depth_valid`` are visible -- the result equals that for the
    compacted ``[B, T*depth_valid, H, D]`` tensors, the gradients of the other slots are
    zero, and a preallocated cache (``DepthCache``) need not be rebuilt per layer.  The other slots are
    never read: they may hold anything (an uninitialised ``torch.empty`` buffer included).
    """
    q, k, v, g, cached_k, cached_v, scale = _prepare_inputs(
        "parallel_moda", q, k, v, g, cached_k, cached_v, scale, moda_group_num, head_first, return_depth_grads,
        warn_shape)
    o, lse = ParallelMixtureOfDepthAttentionFunction.apply(
        q, k, v, g, scale, cu_seqlens, cached_k, cached_v, moda_group_num, is_causal, group_bs, group_warps, depth_bs,
        depth_warps, depth_valid)
    return (o, lse) if need_lse else o


# ---------------------------------------------------------------------------
# chunk-visible MoDA -- moda_v16.py
# ---------------------------------------------------------------------------
def _chunk_tokens(moda_group_num: int, chunk_rows: Optional[int]) -> int:
    """Base tokens per chunk.  The reference's launchers take ``customized_BT`` but overwrite it with 64 rows on
    every device (moda_v16.py:545-584), so a chunk is always 64 query rows there; ``chunk_rows`` (an argument
    the reference does not have) is the way to ask for another chunk size here."""
    rows = chunk_rows if chunk_rows is not None else DEFAULT_CHUNK_ROWS
    assert (
        rows % moda_group_num == 0
    ), "BT must be divisible by moda_group_num to keep chunk-visible base_t aligned"
    return rows // moda_group_num


def parallel_moda_chunk_visible_fwd(q, k, v, g_cumsum, scale, cu_seqlens=None, cached_k=None, cached_v=None,
                                    moda_group_num=1, customized_BT=None, customized_BS=None, customized_BK=None,
                                    customized_BV=None, customized_num_warps=None, chunk_rows=None, depth_valid=None):
    """moda_v16.py:498-633.  The tile-size knobs are accepted and ignored, ``customized_BT`` included (the
    reference overwrites it with 64, moda_v16.py:581-585); ``chunk_rows`` sets the chunk size in query rows,
    ``depth_valid`` is that of ``parallel_moda``."""
    assert g_cumsum is None, "g_cumsum is not supported in this version"
    assert q.shape[2] == k.shape[2], "Implicit head-dimension GQA is not allowed."
    cb = _chunk_tokens(moda_group_num, chunk_rows)
    return _raw_fwd(_lib.CHUNK_VISIBLE, q, k, v, cached_k, cached_v, scale, moda_group_num, cb,
                    depth_valid=depth_valid, packed=_packed(cu_seqlens, q, moda_group_num))


def parallel_moda_chunk_visible_bwd(q, k, v, o, g_cumsum, lse, do, scale=None, chunk_size=128, cu_seqlens=None,
                                    cached_k=None, cached_v=None, moda_group_num=1, customized_BT=None,
                                    customized_BS=None, customized_BK=None, customized_BV=None,
                                    customized_num_warps=None, chunk_rows=None, depth_valid=None):
    """moda_v16.py:2099-2343 (``customized_BT`` ignored as there, ``chunk_rows``, ``depth_valid`` as in the forward)."""
    assert g_cumsum is None, "g_cumsum is not supported in this version"
    if scale is None:
        scale = q.shape[-1] ** -0.5
    cb = _chunk_tokens(moda_group_num, chunk_rows)
    dq, dk, dv, dkd, dvd = _raw_bwd(_lib.CHUNK_VISIBLE, q, k, v, cached_k, cached_v, o, lse, do, scale,
                                    moda_group_num, cb, depth_valid=depth_valid,
                                    packed=_packed(cu_seqlens, q, moda_group_num))
    return dq, dk, dv, None, dkd, dvd


class ParallelMixtureOfDepthAttentionChunkVisibleFunction(torch.autograd.Function):
    """moda_v16.py:3456-3493 (9 inputs)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, q, k, v, g, scale, cu_seqlens, cached_k=None, cached_v=None, moda_group_num=1,
                chunk_rows=None, depth_valid=None):
        o, lse = _autograd_forward(ctx, parallel_moda_chunk_visible_fwd, q, k, v, g, scale, cu_seqlens, cached_k,
                                   cached_v, moda_group_num, chunk_rows=chunk_rows, depth_valid=depth_valid)
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, do, dlse_unused):
        dq, dk, dv, dkd, dvd = _autograd_backward(ctx, parallel_moda_chunk_visible_bwd, do)
        return dq, dk, dv, None, None, None, dkd, dvd, None, None, None


def parallel_moda_chunk_visible(q, k, v, g=None, cached_k=None, cached_v=None, scale=None, cu_seqlens=None,
                                moda_group_num=1, head_first=False, need_lse=False, return_depth_grads=True,
                                warn_shape=True, customized_BT=None, customized_BS=None, customized_BT_backward=None,
                                customized_BS_backward=None, chunk_rows=None, depth_valid=None):
    """Chunk-visible MoDA; signature of moda_v16.py:3614-3632 plus ``chunk_rows`` and ``depth_valid`` (the latter
    as in ``parallel_moda``: only the first ``depth_valid`` slots of every token hold data).  A query of base
    token ``t`` additionally sees the depth slots of tokens ``floor(t/Cb)*Cb .. t`` with
    ``Cb = 64 // moda_group_num``.  The four ``customized_*`` arguments are accepted and dropped exactly as the
    reference's wrapper drops them (moda_v16.py:3646-3650: a chunk is 64 query rows whatever they say);
    ``chunk_rows``, which the reference does not have, selects another chunk size in query rows."""
    q, k, v, g, cached_k, cached_v, scale = _prepare_inputs(
        "parallel_moda_chunk_visible", q, k, v, g, cached_k, cached_v, scale, moda_group_num, head_first,
        return_depth_grads, warn_shape)
    o, lse = ParallelMixtureOfDepthAttentionChunkVisibleFunction.apply(
        q, k, v, g, scale, cu_seqlens, cached_k, cached_v, moda_group_num, chunk_rows, depth_valid)
    return (o, lse) if need_lse else o


# ---------------------------------------------------------------------------
# FDA (depth-only) -- fda_v12.py
# ---------------------------------------------------------------------------
def parallel_fda_fwd(q, g_cumsum, scale, cu_seqlens=None, cached_k=None, cached_v=None, moda_group_num=1,
                     customized_BT=None, customized_BS=None, customized_BK=None, customized_BV=None,
                     customized_num_warps=None):
    """fda_v12.py:261-400.  Returns ``(o, lse)``."""
    assert g_cumsum is None, "g_cumsum is not supported in this version"
    assert cached_k is not None and cached_v is not None, "Flash Depth Attention requires cached_k/cached_v"
    _assert_group_tile(moda_group_num)
    return _raw_fwd(_lib.DEPTH_ONLY, q, None, None, cached_k, cached_v, scale, moda_group_num,
                    packed=_packed(cu_seqlens, q, moda_group_num))


def parallel_fda_bwd(q, o, g_cumsum, lse, do, scale=None, chunk_size=128, cu_seqlens=None, cached_k=None,
                     cached_v=None, moda_group_num=1, customized_BT=None, customized_BS=None, customized_BK=None,
                     customized_BV=None, customized_num_warps=None, group_bs=None, group_warps=None, depth_bs=None,
                     depth_warps=None):
    """fda_v12.py:881-1135.  Returns ``(dq, dg_cumsum=None, d_cached_k, d_cached_v)``."""
    assert g_cumsum is None, "g_cumsum is not supported in this version"
    if scale is None:
        scale = q.shape[-1] ** -0.5
    dq, _, _, dkd, dvd = _raw_bwd(_lib.DEPTH_ONLY, q, None, None, cached_k, cached_v, o, lse, do, scale,
                                  moda_group_num, packed=_packed(cu_seqlens, q, moda_group_num))
    return dq, None, dkd, dvd


class ParallelFlashDepthAttentionFunction(torch.autograd.Function):
    """fda_v12.py:1207-1338 (13 inputs; the k, v slots must be None)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, q, k, v, g, scale, cu_seqlens, cached_k=None, cached_v=None, moda_group_num=1, group_bs=None,
                group_warps=None, depth_bs=None, depth_warps=None):
        assert g is None, "g is not supported in this version"
        assert k is None and v is None, "Flash Depth Attention does not accept legacy k/v; pass None"
        ctx.packed = _packed(cu_seqlens, q, moda_group_num)
        o, lse = parallel_fda_fwd(q, None, scale, ctx.packed, cached_k, cached_v, moda_group_num)
        ctx.save_for_backward(q, o, lse, cached_k, cached_v)
        ctx.scale = scale
        ctx.moda_group_num = moda_group_num
        ctx.mark_non_differentiable(lse)
        return o.to(q.dtype), lse

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, do, dlse_unused):
        q, o, lse, cached_k, cached_v = ctx.saved_tensors
        dq, _, dkd, dvd = parallel_fda_bwd(q, o, None, lse, do.to(o.dtype), ctx.scale, cu_seqlens=ctx.packed,
                                           cached_k=cached_k, cached_v=cached_v, moda_group_num=ctx.moda_group_num)
        return dq.to(q), None, None, None, None, None, dkd, dvd, None, None, None, None, None


def parallel_fda(q, k=None, v=None, g=None, cached_k=None, cached_v=None, scale=None, cu_seqlens=None,
                 moda_group_num=1, head_first=False, need_lse=False, return_depth_grads=True, warn_shape=True,
                 customized_BT=None, customized_BS=None, customized_BT_backward=None, customized_BS_backward=None,
                 group_bs=None, group_warps=None, depth_bs=None, depth_warps=None):
    """Depth-only attention; signature of fda_v12.py:1346-1368."""
    assert k is None and v is None, "Flash Depth Attention does not accept legacy k/v; pass None"
    if head_first:
        q = q.transpose(1, 2)
        if g is not None:
            g = g.transpose(1, 2)
        if cached_k is not None and cached_v is not None:
            cached_k = cached_k.transpose(1, 2)
            cached_v = cached_v.transpose(1, 2)
    elif warn_shape and q.shape[1] < q.shape[2]:
        warnings.warn(
            f"[parallel_fda] detected seq_len({q.shape[1]}) < num_heads({q.shape[2]}). "
            "input may be in head_first format while head_first=True is not set."
        )
    B, T_q, HQ, Kdim = q.shape
    assert cached_k is not None and cached_v is not None, "Flash Depth Attention requires cached_k/cached_v"
    assert moda_group_num > 0
    assert T_q % moda_group_num == 0, "T_q must be divisible by moda_group_num"
    T_kv = T_q // moda_group_num
    H = cached_k.shape[2]
    assert HQ == H, (
        "Implicit head-dimension GQA is not allowed. "
        "Please fold grouping only into `moda_group_num`: "
        "use q.shape[2] == cached_k.shape[2] and set T_q = T_kv * moda_group_num."
    )
    if scale is None:
        scale = Kdim ** -0.5
    assert cached_k.shape[0] == B and cached_v.shape[0] == B
    assert cached_k.shape[2] == H and cached_v.shape[2] == H, "cached_k/v head count mismatch"
    assert cached_k.shape[1] % T_kv == 0, "cached_k time dimension must be T_kv * L"
    L = cached_k.shape[1] // T_kv
    assert L > 0
    assert cached_v.shape[1] == T_kv * L, "cached_v shape mismatch"
    if (cached_k.requires_grad or cached_v.requires_grad) and not return_depth_grads:
        warnings.warn(
            "cached_k/v requires gradients, but return_depth_grads=False. "
            "Gradients are still computed and returned."
        )
    if g is not None:
        assert g.shape[:3] == (B, T_q, HQ), "g must be [B,T_q,HQ]"
    o, lse = ParallelFlashDepthAttentionFunction.apply(q, k, v, g, scale, cu_seqlens, cached_k, cached_v,
                                                       moda_group_num, group_bs, group_warps, depth_bs, depth_warps)
    return (o, lse) if need_lse else o


# ---------------------------------------------------------------------------
# head-dim GQA <-> the folded layout of the depth modes
# ---------------------------------------------------------------------------
def fold_gqa_heads(x: torch.Tensor, num_kv_heads: int, head_order: str = "group_major") -> torch.Tensor:
    """``[B, T, Hq, D]`` (one query head per head-dim slot) -> the folded ``[B, T*G, Hkv, D]`` that
    ``parallel_moda`` / ``parallel_moda_chunk_visible`` / ``parallel_fda`` take with ``moda_group_num = G``,
    ``G = Hq // Hkv``: the G query heads that share a kv head become G consecutive rows of the token.

    Which query heads share a kv head is a convention of the model, so it is an explicit argument:
    ``"group_major"`` -- query head ``g*Hkv + hkv`` reads kv head ``hkv`` (the fold of the reference's vision
    model, vision_tasks/deit/models.py:248-250); a free view of a contiguous ``x``.
    ``"kv_major"`` -- query head ``hkv*G + g`` reads kv head ``hkv`` (``repeat_interleave`` models and the plain
    comparator, fla/ops/attn/parallel.py:48-49); needs one copy."""
    B, T, Hq, D = x.shape
    assert Hq % num_kv_heads == 0, "query heads must be a multiple of kv heads"
    G = Hq // num_kv_heads
    if head_order == "group_major":
        return x.reshape(B, T, G, num_kv_heads, D).reshape(B, T * G, num_kv_heads, D)
    assert head_order == "kv_major", "head_order must be 'group_major' or 'kv_major'"
    return x.reshape(B, T, num_kv_heads, G, D).transpose(2, 3).reshape(B, T * G, num_kv_heads, D)


def unfold_gqa_heads(x: torch.Tensor, moda_group_num: int, head_order: str = "group_major") -> torch.Tensor:
    """Inverse of :func:`fold_gqa_heads`: ``[B, T*G, Hkv, D]`` -> ``[B, T, G*Hkv, D]``."""
    B, TG, Hkv, D = x.shape
    G = moda_group_num
    assert TG % G == 0, "rows must be a multiple of moda_group_num"
    if head_order == "group_major":
        return x.reshape(B, TG // G, G * Hkv, D)
    assert head_order == "kv_major", "head_order must be 'group_major' or 'kv_major'"
    return x.reshape(B, TG // G, G, Hkv, D).transpose(2, 3).reshape(B, TG // G, Hkv * G, D)


# ---------------------------------------------------------------------------
# plain causal attention with head-dim GQA -- fla/ops/attn/parallel.py
# ---------------------------------------------------------------------------
def parallel_attn_fwd(q, k, v, g_cumsum=None, scale=None, cu_seqlens=None):
    """fla/ops/attn/parallel.py:443-503.  q ``[B,T,HQ,D]``, k/v ``[B,T,H,D]``; returns ``(o, lse)``."""
    assert g_cumsum is None
    assert q.shape[2] % k.shape[2] == 0, "HQ must be a multiple of H"
    assert q.shape[1] == k.shape[1]
    if scale is None:
        scale = k.shape[-1] ** -0.5
    return _raw_fwd(_lib.PLAIN_GQA, q, k, v, None, None, scale, q.shape[2] // k.shape[2],
                    packed=_packed(cu_seqlens, q, 1))


def parallel_attn_bwd(q, k, v, o, g_cumsum, lse, do, scale=None, chunk_size=128, cu_seqlens=None):
    """fla/ops/attn/parallel.py:522-629.  Returns ``(dq, dk, dv, dg=None)``."""
    assert g_cumsum is None
    if scale is None:
        scale = k.shape[-1] ** -0.5
    dq, dk, dv, _, _ = _raw_bwd(_lib.PLAIN_GQA, q, k, v, None, None, o, lse, do, scale, q.shape[2] // k.shape[2],
                                packed=_packed(cu_seqlens, q, 1))
    return dq, dk, dv, None


class ParallelAttentionFunction(torch.autograd.Function):
    """fla/ops/attn/parallel.py:632-675."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, q, k, v, g, scale, cu_seqlens):
        assert g is None, "g is not supported"
        ctx.packed = _packed(cu_seqlens, q, 1)
        o, lse = parallel_attn_fwd(q, k, v, None, scale, ctx.packed)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.scale = scale
        return o.to(q.dtype)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, do):
        q, k, v, o, lse = ctx.saved_tensors
        dq, dk, dv, _ = parallel_attn_bwd(q, k, v, o, None, lse, do.to(o.dtype), ctx.scale, cu_seqlens=ctx.packed)
        return dq.to(q), dk.to(k), dv.to(v), None, None, None


def parallel_attn(q, k, v, g=None, scale=None, cu_seqlens=None, head_first=False):
    """Plain causal attention with head-dim GQA; signature of fla/ops/attn/parallel.py:678-686."""
    if head_first:
        raise DeprecationWarning(
            "head_first is deprecated and will be removed in a future version. "
            "Please use head_first=False for now instead."
        )
    if q.shape[1] < q.shape[2]:
        warnings.warn(
            f"Input tensor shape suggests potential format mismatch: seq_len ({q.shape[1]}) < num_heads ({q.shape[2]}). "
        )
    if scale is None:
        scale = k.shape[-1] ** -0.5
    return ParallelAttentionFunction.apply(q, k, v, g, scale, cu_seqlens)
