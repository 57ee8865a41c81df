"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports
every symbol the header declares, the ctypes mirror of the descriptor matches,
and the host functions keep the reference's argument contract
(moda_v14.py:2834-2871, fda_v12.py:1370-1437).  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_functions():
    text = open(os.path.join(ROOT, "include", "moda_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moda_hip_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from moda_amd import _lib

    lib = _lib.load()
    names = _header_functions()
    assert set(names) == set(_lib.EXPORTS)
    for n in names:
        assert getattr(lib, n) is not None


def test_descriptor_layout_and_version():
    from moda_amd import _lib

    lib = _lib.load()
    assert lib.moda_hip_version() == 105
    assert ctypes.sizeof(_lib.Desc) == 16 + 7 * 8 + 8 + 12 * 24 + 24 + 8
    assert _lib.Desc.cu_seqlens.offset == 80 + 12 * 24
    assert _lib.Desc.q.offset == 80
    # a descriptor with the wrong struct_size is rejected without touching any device
    d = _lib.Desc()
    d.struct_size = 12
    assert lib.moda_hip_bwd_workspace_bytes(ctypes.byref(d)) == 0
    assert lib.moda_hip_fwd(ctypes.byref(d), None, None, None, None, None, None, None, None) == -1
    assert b"invalid" in lib.moda_hip_strerror(-1)


def test_descriptor_validation_codes():
    from moda_amd import _lib

    lib = _lib.load()

    def desc(**kw):
        d = _lib.Desc()
        d.struct_size = ctypes.sizeof(_lib.Desc)
        d.dtype, d.mode = _lib.BF16, _lib.CAUSAL
        d.B, d.T, d.H, d.G, d.D, d.L = 1, 8, 1, 1, 64, 0
        d.scale = 1.0
        for k, v in kw.items():
            setattr(d, k, v)
        return d

    assert lib.moda_hip_bwd_workspace_bytes(ctypes.byref(desc())) == 8 * 4
    assert lib.moda_hip_bwd_workspace_bytes(ctypes.byref(desc(G=4, H=2, B=3))) == 3 * 2 * 32 * 4
    assert lib.moda_hip_bwd_workspace_bytes(ctypes.byref(desc(mode=_lib.PLAIN_GQA, G=4, H=2))) == 8 * 8 * 4
    # packed variable-length batch: the workspace covers the packed row axis once, not B x longest sequence
    assert lib.moda_hip_bwd_workspace_bytes(
        ctypes.byref(desc(B=3, T=8, G=2, H=2, cu_seqlens=0x1000, total_tokens=13))) == 2 * 13 * 2 * 4
    # ... the longest sequence cannot exceed the packed axis; the offsets must be 4-byte aligned
    assert lib.moda_hip_bwd_workspace_bytes(ctypes.byref(desc(B=3, T=8, cu_seqlens=0x1000, total_tokens=7))) == 0
    assert lib.moda_hip_bwd_workspace_bytes(ctypes.byref(desc(B=3, T=8, cu_seqlens=0x1002, total_tokens=9))) == 0
    null = None
    # missing q pointer
    assert lib.moda_hip_fwd(ctypes.byref(desc()), null, null, null, null, null, null, null, null) == -1
    # unsupported head dim
    assert lib.moda_hip_fwd(ctypes.byref(desc(D=512)), null, null, null, null, null, null, null, null) == -2
    # depth-only without depth slots, plain GQA with depth slots, chunk-visible without chunk size
    assert lib.moda_hip_fwd(ctypes.byref(desc(mode=_lib.DEPTH_ONLY)), null, null, null, null, null, null, null, null) == -1
    assert lib.moda_hip_fwd(ctypes.byref(desc(mode=_lib.PLAIN_GQA, L=2)), null, null, null, null, null, null, null, null) == -1
    assert lib.moda_hip_fwd(ctypes.byref(desc(mode=_lib.CHUNK_VISIBLE, L=2)), null, null, null, null, null, null, null, null) == -1
    # value head dim: negative is invalid, beyond 256 or not a multiple of 4 unsupported
    assert lib.moda_hip_fwd(ctypes.byref(desc(Dv=-4)), null, null, null, null, null, null, null, null) == -1
    assert lib.moda_hip_fwd(ctypes.byref(desc(Dv=512)), null, null, null, null, null, null, null, null) == -2
    assert lib.moda_hip_fwd(ctypes.byref(desc(Dv=30)), null, null, null, null, null, null, null, null) == -2
    # empty problem is a successful no-op
    assert lib.moda_hip_fwd(ctypes.byref(desc(T=0)), null, null, null, null, null, null, null, null) == 0
    # misaligned pointer (never dereferenced: alignment is checked first)
    bogus = ctypes.c_void_p(0x1008)
    ok = ctypes.c_void_p(0x1000)
    assert lib.moda_hip_fwd(ctypes.byref(desc()), bogus, ok, ok, null, null, ok, ok, null) == -3
    # reorg argument checks
    arr = (ctypes.c_void_p * 1)(0x1000)
    assert lib.moda_hip_depth_reorg_fwd(arr, 1, 3, 3, 1, 4, 1, 64, _lib.BF16, ok, null) == -1  # slot out of range
    assert lib.moda_hip_depth_reorg_fwd(arr, 0, 0, 3, 1, 4, 1, 64, _lib.BF16, ok, null) == 0   # nothing to do


def test_matrix_core_routing_rule_is_the_librarys():
    """The host wrapper asks the library which kernels a call runs on (rows must be 16-byte aligned for the
    matrix kernels): every combination of dtype, head dims and packing, against the rule stated in the header."""
    from moda_amd import _lib, ops

    lib = _lib.load()
    host = (ctypes.c_int32 * 3)(0, 5, 13)
    for dtype, tdt in ((_lib.BF16, torch.bfloat16), (_lib.FP16, torch.float16), (_lib.FP32, torch.float32)):
        for D in (8, 36, 64, 100, 128, 136, 192, 256):
            for Dv in (D, 64 if D != 64 else 32):
                for packed in (None, "device_only", "with_host"):
                    d = _lib.Desc()
                    d.struct_size = ctypes.sizeof(_lib.Desc)
                    d.dtype, d.mode = dtype, _lib.CAUSAL
                    d.B, d.T, d.H, d.G, d.D, d.Dv, d.L = 1, 8, 1, 1, D, Dv, 0
                    d.scale = 1.0
                    pb = None
                    if packed:
                        d.B, d.T, d.total_tokens, d.cu_seqlens = 2, 8, 13, 0x1000
                        cu = torch.tensor([0, 5, 13], dtype=torch.int32)
                        pb = ops.PackedBatch(cu, 2, 8, 13, host if packed == "with_host" else None)
                        if packed == "with_host":
                            d.cu_seqlens_host = ctypes.cast(host, ctypes.c_void_p)
                    want = (dtype != _lib.FP32 and D % 8 == 0 and Dv % 8 == 0
                            and not (max(D, Dv) > 128 and packed == "device_only"))
                    assert lib.moda_hip_uses_matrix_cores(ctypes.byref(d)) == int(want), (dtype, D, Dv, packed)
                    q, v = torch.zeros(1, 8, 1, D, dtype=tdt), torch.zeros(1, 8, 1, Dv, dtype=tdt)
                    assert ops._matrix_core_path(q, v, pb) == want, (dtype, D, Dv, packed)
    bad = _lib.Desc()
    bad.struct_size = 4
    assert lib.moda_hip_uses_matrix_cores(ctypes.byref(bad)) == -1


def test_host_offsets_are_validated():
    from moda_amd import _lib

    lib = _lib.load()

    def desc(offsets, T, total, with_device=True):
        d = _lib.Desc()
        d.struct_size = ctypes.sizeof(_lib.Desc)
        d.dtype, d.mode = _lib.BF16, _lib.CAUSAL
        d.B, d.T, d.H, d.G, d.D, d.L = len(offsets) - 1, T, 1, 1, 64, 0
        d.scale = 1.0
        d.total_tokens = total
        if with_device:
            d.cu_seqlens = 0x1000
        arr = (ctypes.c_int32 * len(offsets))(*offsets)
        d.cu_seqlens_host = ctypes.cast(arr, ctypes.c_void_p)
        return d, arr

    d, keep = desc([0, 5, 13], 8, 13)
    assert lib.moda_hip_bwd_workspace_bytes(ctypes.byref(d)) == 13 * 4
    for offsets, T, total in (([1, 5, 13], 8, 13),   # does not start at 0
                              ([0, 9, 5, 13], 9, 13),  # decreases
                              ([0, 5, 12], 8, 13),    # does not end at total_tokens
                              ([0, 4, 13], 8, 13)):   # a sequence longer than T
        d, keep = desc(offsets, T, total)
        assert lib.moda_hip_uses_matrix_cores(ctypes.byref(d)) == -1, offsets
    d, keep = desc([0, 5, 13], 8, 13, with_device=False)  # host offsets without the device array
    assert lib.moda_hip_uses_matrix_cores(ctypes.byref(d)) == -1


def test_workspace_alignment_codes():
    from moda_amd import _lib

    lib = _lib.load()
    d = _lib.Desc()
    d.struct_size = ctypes.sizeof(_lib.Desc)
    d.dtype, d.mode = _lib.BF16, _lib.CAUSAL
    d.B, d.T, d.H, d.G, d.D, d.L = 1, 8, 1, 1, 64, 0
    d.scale = 1.0
    for f in ("q", "k", "v", "o", "d_o", "dq", "dk", "dv"):
        getattr(d, f).b, getattr(d, f).t, getattr(d, f).h = 512, 64, 64
    ok = ctypes.c_void_p(0x1000)
    args = [ok] * 3 + [None, None] + [ok] * 6 + [None, None]
    # a workspace pointer that is not 4-byte aligned is refused before anything is launched or dereferenced
    assert lib.moda_hip_bwd(ctypes.byref(d), *args, ctypes.c_void_p(0x1002), 64, None) == -3
    assert lib.moda_hip_bwd(ctypes.byref(d), *args, None, 64, None) == -4
    assert lib.moda_hip_bwd(ctypes.byref(d), *args, ok, 8, None) == -4


def test_import_shim_names_and_reference_loops():
    import os
    import sys

    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "moda_amd", "compat")
    sys.path.insert(0, root)
    try:
        for m in [m for m in sys.modules if m == "fla" or m.startswith("fla.")]:
            del sys.modules[m]
        import fla.ops.moda as shim
        import moda_amd

        assert shim.parallel_moda is moda_amd.parallel_moda
        assert shim.parallel_moda_chunk_visible_bwd is moda_amd.parallel_moda_chunk_visible_bwd
        # the reference package also exports its torch loops; here that is an ImportError that says where to look
        with pytest.raises(ImportError, match="oracle/moda_oracle.py"):
            from fla.ops.moda import naive_mixture_of_depth_causal_ref  # noqa: F401
        with pytest.raises(ImportError, match="reference's torch loops"):
            shim.naive_mixture_of_depth_causal_chunk_visible_ref
        with pytest.raises(AttributeError):
            shim.no_such_name
    finally:
        sys.path.remove(root)
        for m in [m for m in sys.modules if m == "fla" or m.startswith("fla.")]:
            del sys.modules[m]


def test_missing_library_fails_loudly(monkeypatch):
    from moda_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmoda_hip.so")
    with pytest.raises(_lib.MissingLibraryError):
        _lib.load()


def test_cpu_tensors_are_rejected():
    import moda_amd

    q = torch.zeros(1, 8, 1, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        moda_amd.parallel_moda(q, q, q)


def test_argument_contract_matches_reference():
    import moda_amd

    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16)
    # implicit head-dim GQA is refused (moda_v14.py:2839-2843)
    with pytest.raises(AssertionError, match="Implicit head-dimension GQA"):
        moda_amd.parallel_moda(z(1, 8, 4, 64), z(1, 8, 2, 64), z(1, 8, 2, 64))
    # T_q must be T_kv * G (moda_v14.py:2847-2852)
    with pytest.raises(AssertionError, match="T_q must equal T_kv"):
        moda_amd.parallel_moda(z(1, 8, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64), moda_group_num=2)
    with pytest.raises(AssertionError, match="moda_group_num=1"):
        moda_amd.parallel_moda(z(1, 16, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64))
    # depth cache shape checks (moda_v14.py:2856-2862)
    with pytest.raises(AssertionError, match="T_kv \\* L"):
        moda_amd.parallel_moda(z(1, 8, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64), cached_k=z(1, 12, 2, 64),
                               cached_v=z(1, 12, 2, 64))
    with pytest.raises(AssertionError, match="head count"):
        moda_amd.parallel_moda(z(1, 8, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64), cached_k=z(1, 16, 1, 64),
                               cached_v=z(1, 16, 1, 64))
    # g is unsupported (moda_v14.py:2672); cu_seqlens, which the reference asserts away in the next line,
    # is accepted here and validated on the host
    with pytest.raises(AssertionError, match="g is not supported"):
        moda_amd.parallel_moda(z(1, 8, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64), g=torch.zeros(1, 8, 2))
    with pytest.raises(AssertionError, match="batch size must be 1"):
        moda_amd.parallel_moda(z(2, 8, 2, 64), z(2, 8, 2, 64), z(2, 8, 2, 64), cu_seqlens=torch.tensor([0, 8]))
    with pytest.raises(AssertionError, match="start at 0 and not decrease"):
        moda_amd.parallel_moda(z(1, 8, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64), cu_seqlens=torch.tensor([0, 5, 3, 8]))
    with pytest.raises(AssertionError, match="ends at 7 base tokens"):
        moda_amd.parallel_moda(z(1, 16, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64), moda_group_num=2,
                               cu_seqlens=torch.tensor([0, 3, 7]))
    with pytest.raises(RuntimeError, match="no CPU path"):
        moda_amd.parallel_moda(z(1, 8, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64), cu_seqlens=torch.tensor([0, 3, 8]))
    # group size must divide the query tile (moda_v14.py:476-478)
    with pytest.raises(AssertionError, match="BT % moda_group_num"):
        moda_amd.parallel_moda(z(1, 24, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64), moda_group_num=3)
    # FDA (fda_v12.py:1370-1372, 1391-1393)
    with pytest.raises(AssertionError, match="does not accept legacy k/v"):
        moda_amd.parallel_fda(z(1, 8, 2, 64), k=z(1, 8, 2, 64), v=z(1, 8, 2, 64), cached_k=z(1, 16, 2, 64),
                              cached_v=z(1, 16, 2, 64))
    with pytest.raises(AssertionError, match="requires cached_k/cached_v"):
        moda_amd.parallel_fda(z(1, 8, 2, 64))
    # seq_len < num_heads warning (moda_v14.py:2828-2832)
    with pytest.warns(UserWarning, match="head_first"):
        with pytest.raises(RuntimeError):
            moda_amd.parallel_moda(z(1, 2, 4, 64), z(1, 2, 4, 64), z(1, 2, 4, 64))


def test_low_level_entry_points_check_every_extent_before_launching():
    """The C ABI takes bare pointers and derives all extents from k, G and the depth row count; a tensor that
    does not match would be read or written out of bounds on the device.  The host refuses such calls before
    anything is launched (these run on CPU tensors: the shape check comes before the device check)."""
    import moda_amd
    from moda_amd import _lib, ops

    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16)
    q, k, v = z(1, 16, 2, 64), z(1, 8, 2, 64), z(1, 8, 2, 64)
    kd, vd = z(1, 24, 2, 64), z(1, 24, 2, 64)
    lse, o, do = torch.zeros(1, 16, 2), z(1, 16, 2, 64), z(1, 16, 2, 64)
    # a wrong moda_group_num: q rows != T * G
    with pytest.raises(AssertionError, match="expected T\\*moda_group_num"):
        moda_amd.parallel_moda_fwd(q, k, v, None, 0.125, cached_k=kd, cached_v=vd, moda_group_num=1)
    with pytest.raises(AssertionError, match="expected T\\*moda_group_num"):
        moda_amd.parallel_moda_bwd(q, k, v, o, None, lse, do, 0.125, cached_k=kd, cached_v=vd, moda_group_num=4)
    with pytest.raises(AssertionError, match="expected T\\*moda_group_num"):
        moda_amd.parallel_moda_chunk_visible_fwd(q, k, v, None, 0.125, cached_k=kd, cached_v=vd, moda_group_num=1)
    # depth rows that are not T * L, depth v shorter than depth k
    with pytest.raises(AssertionError, match="depth rows must be T \\* L"):
        moda_amd.parallel_moda_fwd(q, k, v, None, 0.125, cached_k=z(1, 20, 2, 64), cached_v=z(1, 20, 2, 64),
                                   moda_group_num=2)
    with pytest.raises(AssertionError, match="same number of rows"):
        moda_amd.parallel_moda_fwd(q, k, v, None, 0.125, cached_k=kd, cached_v=z(1, 16, 2, 64), moda_group_num=2)
    with pytest.raises(AssertionError, match="k and v must agree"):
        moda_amd.parallel_moda_fwd(q, k, z(1, 4, 2, 64), None, 0.125, moda_group_num=2)
    # backward: o / do / lse of the wrong size
    with pytest.raises(AssertionError, match="do must be"):
        moda_amd.parallel_moda_bwd(q, k, v, o, None, lse, z(1, 8, 2, 64), 0.125, moda_group_num=2)
    with pytest.raises(AssertionError, match="lse must be"):
        moda_amd.parallel_moda_bwd(q, k, v, o, None, torch.zeros(1, 8, 2), do, 0.125, moda_group_num=2)
    # depth-only: rows not a multiple of G, depth rows not T * L
    with pytest.raises(AssertionError, match="multiple of moda_group_num"):
        moda_amd.parallel_fda_fwd(z(1, 15, 2, 64), None, 0.125, cached_k=kd, cached_v=vd, moda_group_num=2)
    with pytest.raises(AssertionError, match="depth rows must be T \\* L"):
        moda_amd.parallel_fda_fwd(q, None, 0.125, cached_k=z(1, 20, 2, 64), cached_v=z(1, 20, 2, 64), moda_group_num=2)
    # a consistent call gets as far as the device check
    with pytest.raises(RuntimeError, match="no CPU path"):
        moda_amd.parallel_moda_fwd(q, k, v, None, 0.125, cached_k=kd, cached_v=vd, moda_group_num=2)
    assert ops._check_shapes(_lib.CAUSAL, q, k, v, kd, vd, 2, o=o, do=do, lse=lse) == (8, 3)


def test_depth_cache_append_checks_the_layer_against_the_cache():
    import moda_amd

    cache = moda_amd.DepthCache(2, 8, 3, 2, 64, torch.bfloat16, "cpu")
    z = lambda *s, dt=torch.bfloat16: torch.zeros(*s, dtype=dt)
    with pytest.raises(AssertionError, match="like the cache"):
        cache.append(z(2, 9, 2, 64), z(2, 9, 2, 64))       # more tokens than the cache has
    with pytest.raises(AssertionError, match="like the cache"):
        cache.append(z(2, 8, 2, 128), z(2, 8, 2, 128))     # wider head dim
    with pytest.raises(AssertionError, match="like the cache"):
        cache.append(z(2, 8, 2, 64), z(2, 8, 4, 64))       # v with more heads
    with pytest.raises(AssertionError, match="dtype"):
        cache.append(z(2, 8, 2, 64, dt=torch.float16), z(2, 8, 2, 64, dt=torch.float16))
    assert cache.n == 0
    with pytest.raises(RuntimeError, match="no CPU path"):  # a matching layer reaches the device check
        cache.append(z(2, 8, 2, 64), z(2, 8, 2, 64))
    with pytest.raises(AssertionError, match="cache must be a contiguous"):
        moda_amd.depth_cache._reorg_fwd([z(2, 8, 2, 64)], z(2, 16, 2, 64), 0, 3)


def test_gqa_head_folds_match_the_two_head_conventions():
    """fold_gqa_heads turns head-dim GQA queries into the folded layout of the depth modes.  Pinned on the oracle:
    kv_major folding + the folded operator == the plain comparator (query head hq reads kv head hq // G, the
    repeat_interleave convention); group_major folding == the reference caller's reshape; both invert exactly."""
    import moda_amd
    import oracle

    gen = torch.Generator().manual_seed(3)
    B, T, Hkv, G, D = 2, 9, 2, 3, 8
    q = torch.randn(B, T, Hkv * G, D, generator=gen, dtype=torch.float64)
    k = torch.randn(B, T, Hkv, D, generator=gen, dtype=torch.float64)
    v = torch.randn(B, T, Hkv, D, generator=gen, dtype=torch.float64)
    ref, _ = oracle.plain_gqa_dense(q, k, v, dtype=torch.float64)
    qf = moda_amd.fold_gqa_heads(q, Hkv, "kv_major")
    o, _ = oracle.moda_dense(qf, k, v, None, None, None, G, "causal", dtype=torch.float64)
    assert torch.allclose(moda_amd.unfold_gqa_heads(o, G, "kv_major"), ref, atol=1e-12)
    # group-major: query head g*Hkv + hkv reads kv head hkv, i.e. the caller's q.reshape(B, N, G, Hkv, D)
    qg = moda_amd.fold_gqa_heads(q, Hkv, "group_major")
    assert torch.equal(qg, q.reshape(B, T, G, Hkv, D).reshape(B, T * G, Hkv, D))
    assert qg.data_ptr() == q.data_ptr()  # a view, no copy
    o, _ = oracle.moda_dense(qg, k, v, None, None, None, G, "causal", dtype=torch.float64)
    kk = torch.cat([k] * G, dim=2)  # kv head of query head g*Hkv + hkv is hkv
    vv = torch.cat([v] * G, dim=2)
    ref_g, _ = oracle.plain_gqa_dense(q, kk, vv, dtype=torch.float64)  # one kv head per query head
    assert torch.allclose(moda_amd.unfold_gqa_heads(o, G, "group_major"), ref_g, atol=1e-12)
    for order in ("group_major", "kv_major"):
        assert torch.equal(moda_amd.unfold_gqa_heads(moda_amd.fold_gqa_heads(q, Hkv, order), G, order), q)


def test_compat_package_reexports():
    import sys

    sys.path.insert(0, os.path.join(ROOT, "moda_amd", "compat"))
    try:
        from fla.ops.moda import parallel_moda, parallel_moda_chunk_visible  # noqa: F401
        import moda_amd

        assert parallel_moda is moda_amd.parallel_moda
    finally:
        sys.path.pop(0)
        for m in [m for m in sys.modules if m == "fla" or m.startswith("fla.")]:
            del sys.modules[m]


def test_attention_module_mirrors_reference_parameters():
    """Parameter names and shapes of vision_tasks/deit/models.py:224-243 (a reference state_dict loads
    unchanged); an empty depth stream yields no cache."""
    import moda_amd

    m = moda_amd.MoDAAttention(384, num_heads=6, num_kv_heads=3, qkv_bias=True)
    shapes = {n: tuple(p.shape) for n, p in m.state_dict().items()}
    assert shapes == {"q.weight": (384, 384), "q.bias": (384,), "kv.weight": (384, 384), "kv.bias": (384,),
                      "proj.weight": (384, 384), "proj.bias": (384,)}
    assert m.moda_group_num == 2 and m.head_dim == 64 and m.scale == 64 ** -0.5
    with pytest.raises(ValueError, match="divisible by num_kv_heads"):
        moda_amd.MoDAAttention(384, num_heads=6, num_kv_heads=4)
    s = moda_amd.DepthStream(4)
    assert s.context() == (None, None, None) and len(s) == 0
    with pytest.raises(RuntimeError, match="no CPU path"):
        m(torch.zeros(1, 8, 384))


def test_fp32_compute_setting():
    import moda_amd

    assert moda_amd.set_fp32_compute("fp16") == "fp32"
    assert moda_amd.set_fp32_compute("fp32") == "fp16"
    with pytest.raises(AssertionError):
        moda_amd.set_fp32_compute("tf32")
    assert moda_amd.set_fp32_compute("fp32") == "fp32"
