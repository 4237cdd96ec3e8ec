"""ctypes binding of ``libflashbias_hip.so`` (C ABI declared in ``include/flashbias.h``).

The library is built in-tree by ``flashbias_amd/csrc/Makefile``.  There is no fallback: if it
is missing or a symbol is absent, importing the operator fails with an error that says so.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libflashbias_hip.so")

FB_F16, FB_BF16, FB_F32 = 0, 1, 2
FB_MASK_NONE, FB_MASK_VECTOR, FB_MASK_MATRIX = 0, 1, 2

#: every symbol that include/flashbias.h declares
EXPORTS = ("fb_version", "fb_init", "fb_last_error", "fb_bwd_workspace_bytes", "fb_suggest_bias_grad_group", "fb_check", "fb_fwd", "fb_bwd",
           "fb_sum_over_batch", "fb_resize_rank",
           "fb_bwd_preprocess", "fb_bwd_dkv", "fb_bwd_dq", "fb_bwd_static")


class FbTensor(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_b", ctypes.c_int64), ("stride_h", ctypes.c_int64),
                ("stride_s", ctypes.c_int64)]


class FbParams(ctypes.Structure):
    _fields_ = ([("size", ctypes.c_uint32), ("dtype", ctypes.c_int32)]
                + [(n, ctypes.c_int32) for n in ("B", "H", "Lq", "Lk", "d", "r", "causal", "mask_type",
                                                 "mask_dtype")]
                + [("scale", ctypes.c_float)]
                + [(n, FbTensor) for n in ("q", "k", "v", "q_bias", "k_bias", "mask", "o")]
                + [("lse", ctypes.c_void_p)]
                + [(n, FbTensor) for n in ("dout", "dq", "dk", "dv", "dq_bias", "dk_bias")]
                + [("delta", ctypes.c_void_p), ("bias_grad_group", ctypes.c_int32)])


class FlashBiasError(RuntimeError):
    """A non-zero status from the C library."""

    def __init__(self, code, text):
        super().__init__(f"flashbias status {code}: {text}")
        self.code = code


_lib = None


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C flashbias_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    for name in EXPORTS:
        if not hasattr(lib, name):
            raise ImportError(f"{LIB_PATH} does not export {name}")
    lib.fb_version.restype = ctypes.c_int
    lib.fb_init.restype = ctypes.c_int
    lib.fb_last_error.restype = ctypes.c_char_p
    lib.fb_bwd_workspace_bytes.argtypes = [ctypes.POINTER(FbParams)]
    lib.fb_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.fb_suggest_bias_grad_group.argtypes = [ctypes.POINTER(FbParams)]
    lib.fb_suggest_bias_grad_group.restype = ctypes.c_int
    lib.fb_check.argtypes = [ctypes.POINTER(FbParams), ctypes.c_int]
    lib.fb_check.restype = ctypes.c_int
    for name in ("fb_fwd", "fb_bwd", "fb_bwd_preprocess", "fb_bwd_dkv", "fb_bwd_dq", "fb_bwd_static"):
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(FbParams), ctypes.c_void_p]
        fn.restype = ctypes.c_int
    lib.fb_sum_over_batch.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                      ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]
    lib.fb_sum_over_batch.restype = ctypes.c_int
    lib.fb_resize_rank.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.fb_resize_rank.restype = ctypes.c_int
    _lib = lib
    return lib


def check_status(code):
    if code != 0:
        raise FlashBiasError(code, load().fb_last_error().decode())


def new_params():
    p = FbParams()
    p.size = ctypes.sizeof(FbParams)
    return p
