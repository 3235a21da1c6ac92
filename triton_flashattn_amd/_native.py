"""ctypes binding of libfa_mi355.so (the C ABI declared in include/fa_mi355.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfa_mi355.so")
ABI_VERSION = 3

FA_F16, FA_BF16 = 0, 1
FA_BIAS_NONE, FA_BIAS_BOOL, FA_BIAS_F16, FA_BIAS_BF16, FA_BIAS_F32, FA_BIAS_ALIBI = 0, 1, 2, 3, 4, 5

_i64x4 = ctypes.c_int64 * 4


class FaProblem(ctypes.Structure):
    _fields_ = [
        ("B", ctypes.c_int32), ("H", ctypes.c_int32), ("M", ctypes.c_int32), ("N", ctypes.c_int32),
        ("D", ctypes.c_int32), ("dtype", ctypes.c_int32), ("bias_dtype", ctypes.c_int32),
        ("causal", ctypes.c_int32), ("sm_scale", ctypes.c_float),
    ]


class FaFwdArgs(ctypes.Structure):
    _fields_ = [
        ("p", FaProblem),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("bias", ctypes.c_void_p),
        ("o", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("q_strides", _i64x4), ("k_strides", _i64x4), ("v_strides", _i64x4), ("o_strides", _i64x4),
        ("bias_strides", _i64x4),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
    ]


class FaBwdArgs(ctypes.Structure):
    _fields_ = [
        ("p", FaProblem),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("o", ctypes.c_void_p),
        ("dout", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("dq", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p), ("dbias", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("q_strides", _i64x4), ("k_strides", _i64x4), ("v_strides", _i64x4), ("o_strides", _i64x4),
        ("do_strides", _i64x4), ("dq_strides", _i64x4), ("dk_strides", _i64x4), ("dv_strides", _i64x4),
        ("bias_strides", _i64x4), ("dbias_strides", _i64x4),
    ]


EXPORTS = ("fa_abi_version", "fa_strerror", "fa_fwd", "fa_fwd_workspace_bytes", "fa_bwd_workspace_bytes", "fa_bwd", "fa_bwd_stages",
           "fa_bwd_noalloc")
FA_STAGE_PREP, FA_STAGE_MAIN, FA_STAGE_DQ, FA_STAGE_ALL, FA_STAGE_DQ_FROM_DBIAS = 1, 2, 4, 7, 8
FA_NOALLOC_MAX_ROWS = 1 << 20
FA_ERR_WORKSPACE = -6
FA_ERR_TOO_LARGE = -9
FA_ERR_HEAD_STRIDE = -10

_lib = None


class NativeLibraryError(RuntimeError):
    pass


def load():
    """Loads the shared library once and declares the signatures of its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryError(
            "%s is missing: build it with `python -m triton_flashattn_amd.build` "
            "(there is no non-HIP fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    lib.fa_abi_version.restype = ctypes.c_int
    lib.fa_abi_version.argtypes = []
    lib.fa_strerror.restype = ctypes.c_char_p
    lib.fa_strerror.argtypes = [ctypes.c_int]
    lib.fa_fwd.restype = ctypes.c_int
    lib.fa_fwd.argtypes = [ctypes.POINTER(FaFwdArgs), ctypes.c_void_p]
    lib.fa_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.fa_fwd_workspace_bytes.argtypes = [ctypes.POINTER(FaProblem)]
    lib.fa_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.fa_bwd_workspace_bytes.argtypes = [ctypes.POINTER(FaProblem)]
    lib.fa_bwd.restype = ctypes.c_int
    lib.fa_bwd.argtypes = [ctypes.POINTER(FaBwdArgs), ctypes.c_void_p]
    lib.fa_bwd_stages.restype = ctypes.c_int
    lib.fa_bwd_stages.argtypes = [ctypes.POINTER(FaBwdArgs), ctypes.c_void_p, ctypes.c_int]
    lib.fa_bwd_noalloc.restype = ctypes.c_int
    lib.fa_bwd_noalloc.argtypes = [ctypes.POINTER(FaBwdArgs), ctypes.c_void_p]
    if lib.fa_abi_version() != ABI_VERSION:
        raise NativeLibraryError("libfa_mi355.so has ABI %d, expected %d" % (lib.fa_abi_version(), ABI_VERSION))
    _lib = lib
    return lib


def check(status):
    if status != 0:
        raise NativeLibraryError("libfa_mi355: %s (status %d)" % (load().fa_strerror(status).decode(), status))
