"""ctypes binding of libhtr_gfx950.so (declared in include/htr_gfx950.h).

Loading never compiles: the library is built ahead of time by `python -m htr_amd.build`
(or __graft_entry__.build()).  If it is missing, every operator raises; there is no CPU or
PyTorch fallback for the packed-linear path.
"""
import ctypes
import os

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
# HTR_GFX950_LIB names another build of the same library (e.g. a tuning build); it must exist, there is no fallback
LIB_PATH = os.environ.get("HTR_GFX950_LIB") or os.path.join(_CSRC, "libhtr_gfx950.so")

BF16, F16, F32 = 0, 1, 2
MAX_BATCH = 2048
MAX_ROWS_PER_TILE = 128
MAX_GROUP_ROWS = 32
MAX_GROUP = 4096
STATIC_SCRATCH_BYTES = 8 << 20

_lib = None

_vp, _i, _sz, _i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_int64

SIGNATURES = {
    "htr_strerror": (ctypes.c_char_p, [_i]),
    "htr_last_hip_error": (_i, []),
    "htr_abi_version": (_i, []),
    "htr_cbscale": (ctypes.c_float, []),
    "htr_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "htr_linear_plan": (_i, [_i, _i, _i, _i, _i, ctypes.POINTER(ctypes.c_int)]),
    "htr_plan_device_override": (_i, [_i, ctypes.c_long]),
    "htr_linear": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "htr_linear_static": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "htr_anchor_linear": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "htr_anchor_decode": (_i, [_i, _i, _i, _i, _vp, _vp]),
    "htr_grouped_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "htr_linear_grouped": (_i, [_vp, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "htr_set_spin_limit": (None, [_i]),
    "htr_workspace_init": (_i, [_vp, _sz, _vp, _vp]),
    "htr_stream_capture_id": (ctypes.c_ulonglong, [_vp]),
    "htr_viterbi_workspace_bytes": (_sz, [_i64, _i, _i]),
    "htr_viterbi": (_i, [_vp, _vp, _i64, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "htr_decode_raw": (_i, [_vp, _vp, _i64, _i, _vp]),
    "htr_dequant_q": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "htr_dequant_w": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
}


class NativeLibraryMissing(RuntimeError):
    pass


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NativeLibraryMissing(
                f"{LIB_PATH} is not built; run `python -m htr_amd.build` (hipcc, gfx950). "
                "The HTR packed-linear path has no fallback implementation.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def check(status):
    if status != 0:
        L = lib()
        msg = L.htr_strerror(status).decode()
        hip = L.htr_last_hip_error()
        raise RuntimeError(f"libhtr_gfx950: {msg} (status {status}" + (f", hipError {hip})" if status == 8 else ")"))
