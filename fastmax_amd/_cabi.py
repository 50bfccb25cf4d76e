"""ctypes view of the C ABI declared in include/fastmax_amd.h.

Loads the in-tree ``libfastmax_hip.so`` (built by ``fastmax_amd.build``).  There is no
fallback: if the library is missing every call raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfastmax_hip.so")

FASTMAX_F32, FASTMAX_BF16 = 0, 1
PASS_FORWARD, PASS_BACKWARD = 0, 1

ERROR_NAMES = {
    0: "FASTMAX_OK", -1: "FASTMAX_E_NULL", -2: "FASTMAX_E_SHAPE", -3: "FASTMAX_E_DTYPE",
    -4: "FASTMAX_E_PARAM", -5: "FASTMAX_E_WORKSPACE", -6: "FASTMAX_E_LAUNCH", -7: "FASTMAX_E_NO_DEVICE",
}

# every symbol include/fastmax_amd.h declares
EXPORTS = (
    "fastmax_version", "fastmax_last_error", "fastmax_check_desc", "fastmax_workspace_bytes",
    "fastmax_workspace_min_bytes", "fastmax_forward", "fastmax_backward", "fastmax_normalize_inplace",
    "fastmax_profile_begin", "fastmax_profile_end",
    "fastmax_state_bytes", "fastmax_decode_workspace_bytes", "fastmax_state_update", "fastmax_decode_step",
    "fastmax_saved_state_bytes", "fastmax_forward_saving", "fastmax_backward_saved", "fastmax_qkv_rope",
    "fastmax_noalloc_scratch_bytes", "fastmax_forward_noalloc",
    "fastmax_workspace_bytes_strided", "fastmax_workspace_min_bytes_strided", "fastmax_saved_state_bytes_strided",
    "fastmax_forward_strided", "fastmax_backward_strided", "fastmax_uses_dense_tiles",
)

KERNEL_NAMES = ("rowstat", "build", "fwd_apply", "bwd_prep", "bwd_dq", "bwd_dk", "bwd_dv", "norm_fix")


class KernelTimes(C.Structure):
    _fields_ = [("ms", C.c_float * 8), ("launches", C.c_int32 * 8)]


class FastmaxDesc(C.Structure):
    _fields_ = [
        ("bh", C.c_int32), ("bhkv", C.c_int32), ("nq", C.c_int32), ("nk", C.c_int32),
        ("d", C.c_int32), ("dtype", C.c_int32), ("mask", C.c_int32), ("normalize", C.c_int32),
        ("p", C.c_int32), ("lim", C.c_float), ("temperature", C.c_float),
        ("a0", C.c_float), ("a1", C.c_float), ("a2", C.c_float),
    ]


class FastmaxStrides(C.Structure):
    _fields_ = [("batch", C.c_int64), ("group", C.c_int64), ("head", C.c_int64), ("token", C.c_int64)]


class FastmaxLayout(C.Structure):
    _fields_ = [("groups", C.c_int32), ("reserved", C.c_int32)] + [
        (name, FastmaxStrides) for name in ("q", "k", "v", "o", "go", "dq", "dk", "dv")]


class RopeDesc(C.Structure):
    _fields_ = [("b", C.c_int32), ("t", C.c_int32), ("groups", C.c_int32), ("q_per_kv", C.c_int32),
                ("hs", C.c_int32), ("rope_n", C.c_int32), ("dtype", C.c_int32)]


class FastmaxError(RuntimeError):
    def __init__(self, code: int, text: str):
        super().__init__(f"{ERROR_NAMES.get(code, code)}: {text}")
        self.code = code


_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m fastmax_amd.build` "
            "(the Fastmax kernels have no fallback path)")
    lib = C.CDLL(LIB_PATH)
    vp, i64, sz = C.c_void_p, C.c_int64, C.c_size_t
    dp = C.POINTER(FastmaxDesc)
    lib.fastmax_version.restype = C.c_char_p
    lib.fastmax_version.argtypes = []
    lib.fastmax_last_error.restype = C.c_char_p
    lib.fastmax_last_error.argtypes = []
    lib.fastmax_check_desc.restype = C.c_int
    lib.fastmax_check_desc.argtypes = [dp]
    lib.fastmax_uses_dense_tiles.restype = C.c_int
    lib.fastmax_uses_dense_tiles.argtypes = [dp]
    lib.fastmax_workspace_bytes.restype = sz
    lib.fastmax_workspace_bytes.argtypes = [dp, C.c_int]
    lib.fastmax_workspace_min_bytes.restype = sz
    lib.fastmax_workspace_min_bytes.argtypes = [dp, C.c_int]
    lib.fastmax_forward.restype = C.c_int
    lib.fastmax_forward.argtypes = [dp, vp, vp, vp, vp, i64, vp, i64, vp, vp, vp, sz, vp]
    lib.fastmax_backward.restype = C.c_int
    lib.fastmax_backward.argtypes = [dp, vp, vp, vp, vp, i64, vp, i64, vp, vp, vp, vp, vp, vp, vp, sz, vp]
    lib.fastmax_saved_state_bytes.restype = sz
    lib.fastmax_saved_state_bytes.argtypes = [dp]
    lib.fastmax_forward_saving.restype = C.c_int
    lib.fastmax_forward_saving.argtypes = [dp, vp, vp, vp, vp, i64, vp, i64, vp, vp, vp, sz, vp, sz, vp]
    lib.fastmax_backward_saved.restype = C.c_int
    lib.fastmax_backward_saved.argtypes = [dp, vp, vp, vp, vp, i64, vp, i64, vp, vp, vp, vp, vp, vp, vp, sz, vp,
                                           sz, vp]
    lp = C.POINTER(FastmaxLayout)
    lib.fastmax_workspace_bytes_strided.restype = sz
    lib.fastmax_workspace_bytes_strided.argtypes = [dp, lp, C.c_int]
    lib.fastmax_workspace_min_bytes_strided.restype = sz
    lib.fastmax_workspace_min_bytes_strided.argtypes = [dp, lp, C.c_int]
    lib.fastmax_saved_state_bytes_strided.restype = sz
    lib.fastmax_saved_state_bytes_strided.argtypes = [dp, lp]
    lib.fastmax_forward_strided.restype = C.c_int
    lib.fastmax_forward_strided.argtypes = [dp, lp, vp, vp, vp, vp, vp, i64, vp, vp, vp, sz, vp, sz, vp]
    lib.fastmax_backward_strided.restype = C.c_int
    lib.fastmax_backward_strided.argtypes = [dp, lp, vp, vp, vp, vp, vp, i64, vp, vp, vp, vp, vp, vp, vp, sz, vp,
                                             sz, vp]
    lib.fastmax_noalloc_scratch_bytes.restype = sz
    lib.fastmax_noalloc_scratch_bytes.argtypes = []
    lib.fastmax_forward_noalloc.restype = C.c_int
    lib.fastmax_forward_noalloc.argtypes = [dp, vp, vp, vp, vp, i64, vp, i64, vp, vp, vp]
    lib.fastmax_qkv_rope.restype = C.c_int
    lib.fastmax_qkv_rope.argtypes = [C.POINTER(RopeDesc), C.c_int, vp, vp, vp, vp, vp, vp, vp]
    lib.fastmax_normalize_inplace.restype = C.c_int
    lib.fastmax_normalize_inplace.argtypes = [dp, vp, vp, vp, sz, vp]
    lib.fastmax_state_bytes.restype = sz
    lib.fastmax_state_bytes.argtypes = [dp]
    lib.fastmax_decode_workspace_bytes.restype = sz
    lib.fastmax_decode_workspace_bytes.argtypes = [dp]
    lib.fastmax_state_update.restype = C.c_int
    lib.fastmax_state_update.argtypes = [dp, vp, vp, vp, vp, C.c_int, vp, sz, vp]
    lib.fastmax_decode_step.restype = C.c_int
    lib.fastmax_decode_step.argtypes = [dp, vp, vp, vp, vp, vp, vp, vp, i64, vp, i64, vp, sz, vp]
    lib.fastmax_profile_begin.restype = C.c_int
    lib.fastmax_profile_begin.argtypes = []
    lib.fastmax_profile_end.restype = C.c_int
    lib.fastmax_profile_end.argtypes = [C.POINTER(KernelTimes)]
    _lib = lib
    return lib


def last_error() -> str:
    return load().fastmax_last_error().decode()


def check(code: int) -> None:
    if code != 0:
        raise FastmaxError(code, last_error())


def make_desc(bh, n, d, dtype, mask, normalize, p, lim=1.0, temperature=1.0, a0=1.0, a1=1.0, a2=0.5,
              bhkv=None, nk=None) -> FastmaxDesc:
    return FastmaxDesc(int(bh), int(bh if bhkv is None else bhkv), int(n), int(n if nk is None else nk),
                       int(d), int(dtype), int(bool(mask)), int(bool(normalize)), int(p), float(lim),
                       float(temperature), float(a0), float(a1), float(a2))
