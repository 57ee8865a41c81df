"""ctypes binding of ``libmoda_hip.so`` (the C ABI declared in ``include/moda_hip.h``).

The shared library is built in-tree by ``make -C moda_amd/csrc`` (or
``__graft_entry__.build()``).  There is no fallback: if it is missing, every
operator of this package raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoda_hip.so")

BF16, FP16, FP32 = 0, 1, 2
CAUSAL, NONCAUSAL, CHUNK_VISIBLE, DEPTH_ONLY, PLAIN_GQA = 0, 1, 2, 3, 4
STAGE_DELTA, STAGE_DQ, STAGE_DKV, STAGE_ALL = 1, 2, 4, 7
FLAG_ACCUMULATE_DEPTH_GRADS = 1
ESTATIC = -7
STATIC_WORKSPACE_BYTES = 8 << 20  # MODA_HIP_STATIC_WORKSPACE_BYTES

EXPORTS = (
    "moda_hip_fwd",
    "moda_hip_bwd_workspace_bytes",
    "moda_hip_bwd",
    "moda_hip_bwd_stages",
    "moda_hip_bwd_static",
    "moda_hip_depth_reorg_fwd",
    "moda_hip_depth_reorg_bwd",
    "moda_hip_uses_matrix_cores",
    "moda_hip_strerror",
    "moda_hip_version",
)


class Strides(Structure):
    _fields_ = [("b", c_int64), ("t", c_int64), ("h", c_int64)]


class Desc(Structure):
    _fields_ = [
        ("struct_size", c_int32),
        ("dtype", c_int32),
        ("mode", c_int32),
        ("L_valid", c_int32),
        ("B", c_int64),
        ("T", c_int64),
        ("H", c_int64),
        ("G", c_int64),
        ("D", c_int64),
        ("L", c_int64),
        ("chunk_tokens", c_int64),
        ("scale", c_float),
        ("flags", c_int32),
        ("q", Strides),
        ("k", Strides),
        ("v", Strides),
        ("kd", Strides),
        ("vd", Strides),
        ("o", Strides),
        ("d_o", Strides),
        ("dq", Strides),
        ("dk", Strides),
        ("dv", Strides),
        ("dkd", Strides),
        ("dvd", Strides),
        ("cu_seqlens", c_void_p),
        ("total_tokens", c_int64),
        ("Dv", c_int64),
        ("cu_seqlens_host", c_void_p),
    ]


class MissingLibraryError(RuntimeError):
    pass


_lib = None


def load():
    """Load the shared library once and declare its prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MissingLibraryError(
            f"{LIB_PATH} not found: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(hipcc, --offload-arch=gfx950). moda_amd has no CPU or eager fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    vp = c_void_p
    lib.moda_hip_fwd.restype = c_int
    lib.moda_hip_fwd.argtypes = [POINTER(Desc), vp, vp, vp, vp, vp, vp, vp, vp]
    lib.moda_hip_bwd_workspace_bytes.restype = c_size_t
    lib.moda_hip_bwd_workspace_bytes.argtypes = [POINTER(Desc)]
    lib.moda_hip_bwd.restype = c_int
    lib.moda_hip_bwd.argtypes = [POINTER(Desc)] + [vp] * 14 + [c_size_t, vp]
    lib.moda_hip_bwd_stages.restype = c_int
    lib.moda_hip_bwd_stages.argtypes = [POINTER(Desc)] + [vp] * 14 + [c_size_t, c_int, vp]
    lib.moda_hip_bwd_static.restype = c_int
    lib.moda_hip_bwd_static.argtypes = [POINTER(Desc)] + [vp] * 13 + [vp]
    lib.moda_hip_depth_reorg_fwd.restype = c_int
    lib.moda_hip_depth_reorg_fwd.argtypes = [POINTER(vp), c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                             c_int64, c_int32, vp, vp]
    lib.moda_hip_depth_reorg_bwd.restype = c_int
    lib.moda_hip_depth_reorg_bwd.argtypes = [vp, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                             c_int32, POINTER(vp), vp]
    lib.moda_hip_uses_matrix_cores.restype = c_int
    lib.moda_hip_uses_matrix_cores.argtypes = [POINTER(Desc)]
    lib.moda_hip_strerror.restype = c_char_p
    lib.moda_hip_strerror.argtypes = [c_int]
    lib.moda_hip_version.restype = c_int
    lib.moda_hip_version.argtypes = []
    _lib = lib
    return lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().moda_hip_strerror(rc).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {rc})")
