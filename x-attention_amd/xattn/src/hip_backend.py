"""ctypes binding of libxattn_hip.so (the C ABI declared in include/xattn_hip.h).

The library is built ahead of time by ``x-attention_amd/csrc/build.py``; if it
is missing the import of this module's :func:`lib` fails loudly - there is no
fallback path.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.normpath(os.path.join(_HERE, "..", "..", "csrc", "libxattn_hip.so"))

c_i32, c_i64, c_f32, c_vp, c_sz = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t

_SIGNATURES = {
    "xattn_abi_version": (c_i32, []),
    "xattn_error_string": (ctypes.c_char_p, [c_i32]),
    "xattn_estimate_workspace_bytes": (c_sz, [c_i32] * 7),
    "xattn_estimate_block_sums": (
        c_i32,
        [c_vp, c_vp, c_vp, c_vp, c_sz, c_vp] + [c_i32] * 5 + [c_i64] * 4 + [c_i32] * 7
        + [c_f32, ctypes.POINTER(c_i32), c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    ),
    "xattn_estimate_select": (
        c_i32,
        [c_vp, c_vp, c_vp, c_vp, c_sz] + [c_i32] * 5 + [c_i64] * 4 + [c_i32] * 7
        + [c_f32, ctypes.POINTER(c_i32), c_i32, c_i32, c_i32, c_i32, c_i32]
        + [c_vp] * 4 + [c_i64, c_i32, c_i32, c_i32, c_vp],
    ),
    "xattn_select_blocks": (
        c_i32,
        [c_vp] * 5 + [c_i64] + [c_i32] * 15 + [c_vp],
    ),
    "xattn_calibration_copy": (c_i32, [c_vp, c_vp, c_sz, c_vp]),
    "xattn_mfma_rate_probe": (c_i32, [c_vp, c_i32, c_i32, c_vp, ctypes.POINTER(ctypes.c_double), c_vp]),
    "xattn_softmax_block_sums": (c_i32, [c_vp, c_vp] + [c_i32] * 3 + [c_i64] * 2 + [c_i32] * 3 + [c_f32, c_i32, c_vp]),
    "xattn_block_mass": (c_i32, [c_vp] * 3 + [c_i32] * 5 + [c_i64] * 4 + [c_i32, c_f32, c_vp]),
    "xattn_threshold_rows": (c_i32, [c_vp] * 3 + [c_i32] * 3 + [c_i64] * 2 + [c_f32, c_vp]),
    "xattn_decode_workspace_bytes": (c_sz, [c_i32] * 3),
    "xattn_decode_fwd": (
        c_i32,
        [c_vp] * 5 + [c_sz] + [c_i32] * 4 + [c_i64] * 6 + [c_f32, c_vp],
    ),
    "xattn_decode_fwd_static": (
        c_i32,
        [c_vp] * 4 + [c_i32] * 4 + [c_i64] * 6 + [c_f32, c_vp],
    ),
    "xattn_block_sparse_fwd": (
        c_i32,
        [c_vp] * 6 + [c_i64] + [c_i32] * 7 + [c_i64] * 8 + [c_i32, c_i32, c_i32, c_f32, c_vp],
    ),
}

_lib = None


class XattnHipError(RuntimeError):
    pass


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise XattnHipError(
                f"{LIB_PATH} is missing: build it with `python x-attention_amd/csrc/build.py` "
                "(there is no non-HIP fallback)"
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def exported_symbols():
    return list(_SIGNATURES)


def check(code, what):
    if code != 0:
        msg = lib().xattn_error_string(code).decode()
        raise XattnHipError(f"{what} failed: {msg} (code {code})")
