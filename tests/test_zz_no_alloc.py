"""The allocation-free backward entry point ``moda_hip_bwd_static`` against ``moda_hip_bwd``.

Both are called straight through the C ABI (ctypes on the shared library, device pointers from torch
tensors).  ``moda_hip_bwd_static`` keeps the row sums of o * do in a workspace inside the library's device
image instead of a caller-provided buffer; it runs the same kernels, so its gradients must equal those of
``moda_hip_bwd`` bit for bit.  ``moda_hip_bwd``'s own output is held to the parity bar against the oracle
(bf16 ``|err| <= 2e-2 + 2^-7 |ref|``, fp16 ``4e-3 + 2^-9 |ref|``).  Two calls in a row, the second one on
a smaller problem, show that what an earlier call left in the shared workspace does not leak into a later one.
"""
import ctypes
import sys

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: (2e-2, 2.0 ** -7), torch.float16: (4e-3, 2.0 ** -9)}
MODE_ID = {"causal": 0, "noncausal": 1, "chunk_visible": 2, "depth_only": 3}


def say(msg):
    sys.stdout.write(msg + "\n")
    sys.stdout.flush()


def _ptr(x):
    return ctypes.c_void_p(x.data_ptr() if x is not None else 0)


def _both_backwards(dev, B, T, H, D, L, G, mode, dtype, cb=0, seed=0):
    from moda_amd import _lib, ops

    lib = _lib.load()
    say(f"no-alloc backward: B={B} T={T} H={H} D={D} L={L} G={G} {mode} {dtype}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=seed, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
    sc = D ** -0.5
    ref = oracle.moda_dense_fwd_bwd(inp, sc, G, mode, cb)
    g = {k: (None if v is None else v.to(dev)) for k, v in inp.items()}
    q, k, v, kd, vd, do = g["q"], g["k"], g["v"], g["kd"], g["vd"], g["do"]
    m = MODE_ID[mode]
    o, lse = ops._raw_fwd(m, q, k, v, kd, vd, sc, G, cb)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    def outputs(fill):
        mk = lambda x: None if x is None else torch.full_like(x, fill)
        return mk(q), mk(k), mk(v), mk(kd), mk(vd)

    # the existing entry point, with a workspace the caller allocates
    a = outputs(float("nan"))
    d = ops._desc(m, q, k, v, kd, vd, G, L, cb, sc, o=o, do=do, dq=a[0], dk=a[1], dv=a[2], dkd=a[3], dvd=a[4])
    nbytes = lib.moda_hip_bwd_workspace_bytes(ctypes.byref(d))
    assert 0 < nbytes <= _lib.STATIC_WORKSPACE_BYTES
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    rc = lib.moda_hip_bwd(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(kd), _ptr(vd), _ptr(o), _ptr(lse), _ptr(do),
                          _ptr(a[0]), _ptr(a[1]), _ptr(a[2]), _ptr(a[3]), _ptr(a[4]), _ptr(ws),
                          ctypes.c_size_t(nbytes), stream)
    assert rc == 0, lib.moda_hip_strerror(rc)
    # the allocation-free one: no workspace argument; free device memory must not move across the call
    b = outputs(float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    rc = lib.moda_hip_bwd_static(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(kd), _ptr(vd), _ptr(o), _ptr(lse),
                                 _ptr(do), _ptr(b[0]), _ptr(b[1]), _ptr(b[2]), _ptr(b[3]), _ptr(b[4]), stream)
    assert rc == 0, lib.moda_hip_strerror(rc)
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info(dev)[0]
    atol, rtol = TOL[dtype]
    for name, x, y in zip(("dq", "dk", "dv", "dkd", "dvd"), a, b):
        if x is None:
            assert ref[name] is None
            continue
        assert torch.isfinite(x.float()).all(), f"moda_hip_bwd {name}: non-finite values"
        r = ref[name].float()
        err = (x.float().cpu() - r).abs()
        assert bool((err <= atol + rtol * r.abs()).all()), f"moda_hip_bwd {name}: max |err| {err.max():.3e}"
        assert torch.equal(x.view(torch.int16), y.view(torch.int16)), f"moda_hip_bwd_static {name} differs from moda_hip_bwd"
    return free_before, free_after


def test_static_workspace_backward_matches_and_survives_a_smaller_second_call(gpu_device):
    dev = gpu_device
    # first call fills most of the rows a later call could see stale values in
    _both_backwards(dev, 2, 300, 2, 128, 6, 4, "causal", torch.bfloat16)
    # second call, smaller in every extent (and other modes): must not be affected by what the first left behind
    fb, fa = _both_backwards(dev, 1, 77, 2, 128, 5, 2, "causal", torch.bfloat16, seed=1)
    assert fa == fb, f"free device memory moved across moda_hip_bwd_static: {fb} -> {fa}"
    _both_backwards(dev, 1, 50, 1, 64, 3, 4, "depth_only", torch.float16, seed=2)
    _both_backwards(dev, 1, 96, 2, 64, 2, 4, "chunk_visible", torch.float16, cb=16, seed=3)


def test_static_workspace_with_fewer_row_segments(gpu_device):
    """A shape for which moda_hip_bwd asks for more workspace than the built-in one holds (fp32 partial sums of
    dk, dv per row segment): the allocation-free entry point then sums over fewer segments, which may move the
    last bit of dk, dv and nothing else."""
    from moda_amd import _lib, ops

    lib = _lib.load()
    dev = gpu_device
    B, T, H, D, L, G = 2, 2048, 4, 128, 1, 4
    say(f"no-alloc backward, fewer row segments: B={B} T={T} H={H} D={D} L={L} G={G}")
    gen = torch.Generator(device=dev).manual_seed(3)
    rn = lambda *s: (0.5 * torch.randn(*s, generator=gen, device=dev)).bfloat16()
    q, k, v, kd, vd, do = rn(B, T * G, H, D), rn(B, T, H, D), rn(B, T, H, D), rn(B, T * L, H, D), rn(B, T * L, H, D), \
        rn(B, T * G, H, D)
    sc = D ** -0.5
    o, lse = ops._raw_fwd(_lib.CAUSAL, q, k, v, kd, vd, sc, G)
    ws = ops.bwd_workspace(_lib.CAUSAL, q, k, v, kd, vd, G)
    assert ws.numel() > _lib.STATIC_WORKSPACE_BYTES
    a = ops._raw_bwd(_lib.CAUSAL, q, k, v, kd, vd, o, lse, do, sc, G, ws=ws)
    b = tuple(torch.full_like(x, float("nan")) for x in a)
    d = ops._desc(_lib.CAUSAL, q, k, v, kd, vd, G, L, 0, sc, o=o, do=do, dq=b[0], dk=b[1], dv=b[2], dkd=b[3], dvd=b[4])
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    rc = lib.moda_hip_bwd_static(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(kd), _ptr(vd), _ptr(o), _ptr(lse),
                                 _ptr(do), _ptr(b[0]), _ptr(b[1]), _ptr(b[2]), _ptr(b[3]), _ptr(b[4]), stream)
    assert rc == 0, lib.moda_hip_strerror(rc)
    for i in (0, 3, 4):  # dq, dkd, dvd: untouched by the split
        assert torch.equal(a[i].view(torch.int16), b[i].view(torch.int16))
    for i in (1, 2):     # dk, dv: same sums in another order
        x, y = a[i].float(), b[i].float()
        assert torch.isfinite(y).all()
        assert bool(((x - y).abs() <= 2e-2 + 2.0 ** -7 * x.abs()).all())
        assert ((x - y).norm() / x.norm()).item() <= 4e-3


def test_static_workspace_rejects_oversized_problems(gpu_device):
    from moda_amd import _lib

    lib = _lib.load()
    d = _lib.Desc()
    d.struct_size = ctypes.sizeof(_lib.Desc)
    d.dtype, d.mode = _lib.BF16, _lib.CAUSAL
    d.B, d.T, d.H, d.G, d.D, d.L = 1, 1 << 20, 4, 4, 128, 0   # 16 Mi rows x 4 bytes = 64 MiB of row sums
    d.scale = 1.0
    need = lib.moda_hip_bwd_workspace_bytes(ctypes.byref(d))
    assert need > _lib.STATIC_WORKSPACE_BYTES
    z = ctypes.c_void_p(0)
    rc = lib.moda_hip_bwd_static(ctypes.byref(d), z, z, z, z, z, z, z, z, z, z, z, z, z, z)
    assert rc == _lib.ESTATIC
    assert b"STATIC_WORKSPACE" in lib.moda_hip_strerror(rc)
