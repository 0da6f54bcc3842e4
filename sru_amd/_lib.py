"""Loader of the HIP library behind the C ABI (include/sru_amd.h).

There is no fallback: if libsru_amd.so is missing or cannot be loaded, every
entry point of this package raises. The library is built in-tree by
`python -m sru_amd.build` (hipcc --offload-arch=gfx950).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsru_amd.so")
ABI_VERSION = 6
STATE_INTERVAL = 8   # SRU_AMD_STATE_INTERVAL
STATIC_MAX_COLUMNS = 262144   # SRU_AMD_STATIC_MAX_COLUMNS
NORM_MAX_FEATURES = 4096       # SRU_AMD_NORM_MAX_FEATURES

F32, F16, BF16, F64 = 0, 1, 2, 3
X_AS_STREAMS, X_F32 = 0, 1   # SRU_AMD_X_AS_STREAMS, SRU_AMD_X_F32


class Shape(ctypes.Structure):
    """struct sru_amd_shape."""
    _fields_ = [
        ("length", ctypes.c_int64),
        ("batch", ctypes.c_int64),
        ("hidden", ctypes.c_int64),
        ("dirs", ctypes.c_int32),
        ("k", ctypes.c_int32),
        ("activation_type", ctypes.c_int32),
        ("skip_type", ctypes.c_int32),
        ("is_custom", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("state_interval", ctypes.c_int32),
        ("x_dtype", ctypes.c_int32),
    ]


_P = ctypes.c_void_p
SIGNATURES = {
    # name: (restype, argtypes) exactly as declared in include/sru_amd.h
    "sru_amd_forward": (ctypes.c_int, [ctypes.POINTER(Shape)] + [_P] * 12),
    "sru_amd_state_bytes": (ctypes.c_size_t, [ctypes.POINTER(Shape)]),
    "sru_amd_backward_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(Shape)]),
    "sru_amd_backward": (ctypes.c_int, [ctypes.POINTER(Shape)] + [_P] * 17 + [ctypes.c_size_t, _P]),
    "sru_amd_backward_static": (ctypes.c_int, [ctypes.POINTER(Shape)] + [_P] * 17),
    "sru_amd_layer_norm_forward": (ctypes.c_int, [ctypes.c_int64, ctypes.c_int64, _P, ctypes.c_int, _P, _P,
                                                  ctypes.c_float, _P, ctypes.c_int, _P, _P, _P]),
    "sru_amd_layer_norm_backward_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64]),
    "sru_amd_layer_norm_backward": (ctypes.c_int, [ctypes.c_int64, ctypes.c_int64, _P, ctypes.c_int, _P, _P, _P, _P,
                                                   ctypes.c_int, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    "sru_amd_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "sru_amd_abi_version": (ctypes.c_int, []),
}

_lib = None


class LibraryError(RuntimeError):
    pass


def load():
    """Returns the loaded library with argument types set; raises LibraryError."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryError(
            f"{LIB_PATH} is missing: build it with `python -m sru_amd.build` "
            "(there is no fallback path for the SRU recurrence)")
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as exc:
        raise LibraryError(f"cannot load {LIB_PATH}: {exc}") from exc
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.sru_amd_abi_version() != ABI_VERSION:
        raise LibraryError(f"{LIB_PATH} has ABI version {lib.sru_amd_abi_version()}, "
                           f"this package needs {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def status_string(code):
    return load().sru_amd_status_string(code).decode()


def check(code, what):
    """Maps a non-zero status to the exception a caller of the reference would see:
    shape / flag problems are ValueError, everything else RuntimeError."""
    if code == 0:
        return
    msg = f"{what}: {status_string(code)} (sru_amd status {code})"
    if code in (2, 3, 4):
        raise ValueError(msg)
    raise RuntimeError(msg)
