"""ctypes binding of libwtconv_hip.so (C ABI declared in include/wtconv_hip.h)."""
import ctypes
import os
import threading

from . import _build

MAX_LEVELS = 5
F32, BF16, F16 = 0, 1, 2
PASS_FORWARD, PASS_BACKWARD_INPUT, PASS_BACKWARD_PARAMS, PASS_BACKWARD = 0, 1, 2, 3
ABI_VERSION = 5


class Params(ctypes.Structure):
    _fields_ = [("base_weight", ctypes.c_void_p), ("base_bias", ctypes.c_void_p),
                ("base_scale", ctypes.c_void_p),
                ("wt_weight", ctypes.c_void_p * MAX_LEVELS), ("wt_scale", ctypes.c_void_p * MAX_LEVELS)]


class ParamGrads(ctypes.Structure):
    _fields_ = Params._fields_


EXPORTS = {
    "wtconv_abi_version": (ctypes.c_int, []),
    "wtconv_last_error": (ctypes.c_char_p, []),
    "wtconv_max_kernel_size": (ctypes.c_int, []),
    "wtconv2d_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 7),
    "wtconv1d_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 6),
}
_p, _i, _z = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
for _name in ("wtconv2d_forward", "wtconv2d_backward_input"):
    EXPORTS[_name] = (_i, [_p, _p, ctypes.POINTER(Params)] + [_i] * 8 + [_p, _z, _p])
EXPORTS["wtconv_static_scratch_bytes"] = (_z, [])
EXPORTS["wtconv2d_forward_static"] = (_i, [_p, _p, ctypes.POINTER(Params)] + [_i] * 8 + [_p])
EXPORTS["wtconv2d_backward_params"] = (
    _i, [_p, _p, ctypes.POINTER(Params), ctypes.POINTER(ParamGrads)] + [_i] * 8 + [_p, _z, _p])
EXPORTS["wtconv2d_backward"] = (
    _i, [_p, _p, _p, ctypes.POINTER(Params), ctypes.POINTER(ParamGrads)] + [_i] * 8 + [_p, _z, _p])
EXPORTS["wtconv1d_backward"] = (
    _i, [_p, _p, _p, ctypes.POINTER(Params), ctypes.POINTER(ParamGrads)] + [_i] * 7 + [_p, _z, _p])
for _name in ("wtconv1d_forward", "wtconv1d_backward_input"):
    EXPORTS[_name] = (_i, [_p, _p, ctypes.POINTER(Params)] + [_i] * 7 + [_p, _z, _p])
EXPORTS["wtconv1d_backward_params"] = (
    _i, [_p, _p, ctypes.POINTER(Params), ctypes.POINTER(ParamGrads)] + [_i] * 7 + [_p, _z, _p])
_f = ctypes.c_float
EXPORTS["wtconv_channel_norm"] = (_i, [_p, _p, _p, _p, _i, _i, _i, _f, _i, _i, _i, _p])
EXPORTS["wtconv_block_residual"] = (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _p])
EXPORTS["wtconv_block_workspace_bytes"] = (_z, [_i, _i, _i, _i])
EXPORTS["wtconv_channel_norm_backward"] = (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _f, _i, _i, _i, _p, _z, _p])
EXPORTS["wtconv_block_residual_backward"] = (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _z, _p])

_ll = ctypes.c_longlong
EXPORTS["wtconv_haar2d"] = (_i, [_p, _p, _ll, _i, _i, _i, _i, _p])
EXPORTS["wtconv_haar1d"] = (_i, [_p, _p, _ll, _i, _i, _i, _p])

_lib = None
_lock = threading.Lock()


class WTConvLibraryError(RuntimeError):
    pass


def library_path():
    return os.environ.get("WTCONV_HIP_LIB", _build.LIB_PATH)


def load():
    """Load the built library (never builds, never falls back)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not os.path.exists(path):
            raise WTConvLibraryError(
                f"{path} is missing: build it with `python -m wtconv_amd._build` "
                "(hipcc --offload-arch=gfx950); there is no fallback implementation")
        lib = ctypes.CDLL(path)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(lib, name)          # AttributeError if a declared symbol is not exported
            fn.restype, fn.argtypes = res, args
        if lib.wtconv_abi_version() != ABI_VERSION:
            raise WTConvLibraryError(f"ABI version {lib.wtconv_abi_version()} != {ABI_VERSION}")
        _lib = lib
    return _lib


def check(rc, what):
    if rc != 0:
        msg = load().wtconv_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError(msg or f"{what}: invalid argument")
        raise RuntimeError(msg or f"{what} failed with code {rc}")
