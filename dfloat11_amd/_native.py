"""ctypes bindings of the C-ABI declared in include/df11.h."""
import ctypes
import os

from . import build as _build

_vp, _i32, _i64, _u32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_uint32

_hip = None
_codec = None


class DF11Error(RuntimeError):
    pass


ERR_UNSUPPORTED = -2    # DF11_ERR_UNSUPPORTED
ERR_HIP = -3            # DF11_ERR_HIP


def codec_lib():
    """Host codec library (no GPU needed)."""
    global _codec
    if _codec is None:
        if not os.path.exists(_build.CODEC_LIB):
            _build.build_codec()
        L = ctypes.CDLL(_build.CODEC_LIB)
        L.df11_histogram.argtypes = [_vp, _i64, _vp, _i32]
        L.df11_split.argtypes = [_vp, _i64, _vp, _vp, _i32]
        L.df11_build_code.argtypes = [_vp, _vp, _vp, ctypes.POINTER(_i32), ctypes.POINTER(_u32)]
        L.df11_build_luts.argtypes = [_vp, _vp, _vp, _i32, ctypes.POINTER(_i32)]
        L.df11_encode_size.argtypes = [_vp, _i64, _vp, ctypes.POINTER(_i64), ctypes.POINTER(_i64), _i32]
        L.df11_encode.argtypes = [_vp, _i64, _vp, _vp, _i32, _u32, _vp, _i64, _vp, _vp, _i64, _i32]
        for name in ("df11_histogram", "df11_split", "df11_build_code", "df11_build_luts",
                     "df11_encode_size", "df11_encode"):
            getattr(L, name).restype = _i32
        _codec = L
    return _codec


def hip_lib():
    """Device library.  There is no fallback: without it nothing decodes."""
    global _hip
    if _hip is None:
        import torch  # noqa: F401  (loads the HIP runtime this library binds to)
        if not os.path.exists(_build.HIP_LIB):
            _build.build_hip()
        L = ctypes.CDLL(_build.HIP_LIB)
        L.df11_version.restype = _i32
        L.df11_error_string.argtypes = [_i32]
        L.df11_error_string.restype = ctypes.c_char_p
        L.df11_last_hip_error.restype = ctypes.c_char_p
        L.df11_workspace_bytes.argtypes = [_i64]
        L.df11_workspace_bytes.restype = ctypes.c_size_t
        L.df11_prepare.argtypes = [_vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp, ctypes.POINTER(_i32), _vp]
        L.df11_prepare.restype = _i32
        L.df11_decode.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp, _i32, _vp]
        L.df11_decode.restype = _i32
        L.df11_decode_static_workspace.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _i32, _vp]
        L.df11_decode_static_workspace.restype = _i32
        L.df11_decode_with_plan.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp, _i32, _vp, _i32]
        L.df11_decode_with_plan.restype = _i32
        L.df11_decode_rows.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp, _i32, _vp, _vp, _i64, _i64]
        L.df11_decode_rows.restype = _i32
        L.df11_launch_plan_name.argtypes = [_i64, _i64, _i32]
        L.df11_launch_plan_name.restype = ctypes.c_char_p
        _hip = L
    return _hip


def check(rc, what):
    if rc != 0:
        L = hip_lib() if _hip is not None else None
        msg = f"{what} failed with code {rc}"
        if L is not None:
            msg += f" ({L.df11_error_string(rc).decode()})"
            if rc == ERR_HIP:
                msg += f": {L.df11_last_hip_error().decode()}"
        raise DF11Error(msg)
