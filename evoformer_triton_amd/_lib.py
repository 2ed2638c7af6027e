"""ctypes binding of libevoattn.so (the C ABI declared in include/evoattn.h).

The library is built in-tree by evoformer_triton_amd.build; loading fails loudly when it
is missing: there is no fallback implementation.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libevoattn.so")

# enums of evoattn.h
EVO_NONE, EVO_BF16, EVO_F16, EVO_F32 = -1, 0, 1, 2
EVO_MASK_NONE, EVO_MASK_BOOL, EVO_MASK_F32, EVO_MASK_BF16, EVO_MASK_F16 = 0, 1, 2, 3, 4
EVO_FLAG_FORCE_GENERIC = 1
EVO_FLAG_PREP_VALID = 2
EVO_FLAG_ONLY_DQ = 4
EVO_FLAG_ONLY_DKDV = 8
EVO_FLAG_PER_PROBLEM = 16
EVO_FLAG_GATE_DOUT_INPLACE = 0x80
EVO_FLAG_DEBUG_OTHER_WIDTH = 0x100
EVO_FLAG_DEBUG_NO_KV_RING = 0x200
EVO_FLAG_DEBUG_FWD_BIAS_TILES = 0x400
EVO_FLAG_DEBUG_BIAS_TILES = 0x800
EVO_FLAG_DEBUG_NO_DQ_WIDE = 0x1000
EVO_FLAG_DEBUG_NO_DQ_SPLIT = 0x2000
EVO_PASS_FWD, EVO_PASS_BWD = 0, 1
EVO_OK, EVO_EINVAL, EVO_EUNSUPPORTED, EVO_EALIGN, EVO_EWORKSPACE, EVO_EOVERFLOW, EVO_EHIP = 0, -1, -2, -3, -4, -5, -100

EXPORTS = ("evoattn_version", "evoattn_strerror", "evoattn_check", "evoattn_prep_bytes", "evoattn_bwd_workspace_bytes",
           "evoattn_fwd", "evoattn_fwd_static", "evoattn_bwd", "evoattn_path", "evoattn_kernels",
           "evoattn_layernorm_fwd", "evoattn_layernorm_bwd_workspace_bytes", "evoattn_layernorm_bwd",
           "evoattn_colsum_workspace_bytes", "evoattn_colsum")
EVOATTN_STATIC_PREP_BYTES = 16 << 20


class EvoAttnParams(ctypes.Structure):
    _fields_ = [
        ("B", ctypes.c_int32), ("S", ctypes.c_int32), ("N", ctypes.c_int32), ("H", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("bias_dtype", ctypes.c_int32), ("mask_kind", ctypes.c_int32),
        ("dbias_dtype", ctypes.c_int32), ("flags", ctypes.c_int32),
        ("scale", ctypes.c_float), ("reserved", ctypes.c_int32),
        ("stride_b", ctypes.c_int64), ("stride_h", ctypes.c_int64), ("stride_s", ctypes.c_int64),
        ("stride_n", ctypes.c_int64),
        ("bias_stride_b", ctypes.c_int64), ("bias_stride_h", ctypes.c_int64), ("bias_stride_row", ctypes.c_int64),
        ("mask_stride_b", ctypes.c_int64), ("mask_stride_s", ctypes.c_int64),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("bias", ctypes.c_void_p), ("mask", ctypes.c_void_p),
        ("o", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("dout", ctypes.c_void_p), ("dq", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p),
        ("dbias", ctypes.c_void_p), ("dmask", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("prep", ctypes.c_void_p), ("prep_bytes", ctypes.c_size_t),
        ("gate", ctypes.c_void_p), ("o_gated", ctypes.c_void_p), ("dgate", ctypes.c_void_p),
    ]


class EvoAttnError(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        super().__init__(f"{where} failed: {strerror(code)} (code {code})")


_LIB = None


def load(path: str | None = None) -> ctypes.CDLL:
    """Load the library once; raise if it has not been built."""
    global _LIB
    if _LIB is not None and path is None:
        return _LIB
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m evoformer_triton_amd.build` "
            "(there is no fallback implementation)")
    lib = ctypes.CDLL(path)
    P = ctypes.POINTER(EvoAttnParams)
    lib.evoattn_version.restype = ctypes.c_int
    lib.evoattn_version.argtypes = []
    lib.evoattn_strerror.restype = ctypes.c_char_p
    lib.evoattn_strerror.argtypes = [ctypes.c_int]
    lib.evoattn_check.restype = ctypes.c_int
    lib.evoattn_check.argtypes = [P, ctypes.c_int]
    lib.evoattn_prep_bytes.restype = ctypes.c_size_t
    lib.evoattn_prep_bytes.argtypes = [P]
    lib.evoattn_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.evoattn_bwd_workspace_bytes.argtypes = [P]
    lib.evoattn_fwd.restype = ctypes.c_int
    lib.evoattn_fwd.argtypes = [P, ctypes.c_void_p]
    lib.evoattn_fwd_static.restype = ctypes.c_int
    lib.evoattn_fwd_static.argtypes = [P, ctypes.c_void_p]
    lib.evoattn_bwd.restype = ctypes.c_int
    lib.evoattn_bwd.argtypes = [P, ctypes.c_void_p]
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32
    lib.evoattn_layernorm_fwd.restype = ctypes.c_int
    lib.evoattn_layernorm_fwd.argtypes = [vp, vp, vp, vp, vp, vp, i64, i32, i32, ctypes.c_float, vp]
    lib.evoattn_layernorm_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.evoattn_layernorm_bwd_workspace_bytes.argtypes = [i64, i32, i32]
    lib.evoattn_layernorm_bwd.restype = ctypes.c_int
    lib.evoattn_layernorm_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, i64, i32, i32, vp]
    lib.evoattn_colsum_workspace_bytes.restype = ctypes.c_size_t
    lib.evoattn_colsum_workspace_bytes.argtypes = [i64, i32, i32]
    lib.evoattn_colsum.restype = ctypes.c_int
    lib.evoattn_colsum.argtypes = [vp, i64, vp, vp, ctypes.c_size_t, i64, i32, i32, vp]
    lib.evoattn_path.restype = ctypes.c_char_p
    lib.evoattn_kernels.restype = ctypes.c_char_p
    lib.evoattn_path.argtypes = [P, ctypes.c_int]
    lib.evoattn_kernels.argtypes = [P, ctypes.c_int]
    _LIB = lib
    return lib


def strerror(code: int) -> str:
    return load().evoattn_strerror(code).decode()


def check(rc: int, where: str) -> None:
    if rc != 0:
        raise EvoAttnError(rc, where)
