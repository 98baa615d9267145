"""ctypes binding of libcbk_hip.so (the C ABI declared in include/cbk.h).

The library is the only compute path of this package: if it is not built, every operator
raises instead of falling back to PyTorch."""
from __future__ import annotations

import ctypes
import os

from .format import CbkDesc  # noqa: F401 (re-exported for callers that build descriptor arrays)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcbk_hip.so")
_lib = None

_P = ctypes.c_void_p
_DP = ctypes.POINTER(CbkDesc)
_MM = [_DP, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int64, _P, ctypes.c_int, ctypes.c_int64, _P, _P,
       ctypes.c_size_t, _P]
SIGNATURES = {
    "cbk_abi_version": (ctypes.c_int, []),
    "cbk_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "cbk_desc_check": (ctypes.c_int, [_DP, _DP]),
    "cbk_row_stride": (ctypes.c_size_t, [_DP]),
    "cbk_stream_bytes": (ctypes.c_size_t, [_DP, ctypes.c_size_t]),
    "cbk_workspace_bytes": (ctypes.c_size_t, [_DP, ctypes.c_int]),
    "cbk_pack": (ctypes.c_int, [_DP, _P, _P, _P, _P, ctypes.c_int, ctypes.c_int, _P, _P]),
    "cbk_unpack": (ctypes.c_int, [_DP, _P, _P, _P]),
    "cbk_dequant": (ctypes.c_int, [_DP, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P, ctypes.c_int,
                                   ctypes.c_int64, _P]),
    "cbk_gemv": (ctypes.c_int, _MM),
    "cbk_gemm": (ctypes.c_int, _MM),
    "cbk_gemm_static": (ctypes.c_int, _MM[:9] + [_P]),
    "cbk_gemv_batch_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, _DP, ctypes.c_int]),
    "cbk_gemv_batch": (ctypes.c_int, [ctypes.c_int, _DP, ctypes.POINTER(_P), ctypes.POINTER(ctypes.c_int64),
                                      ctypes.c_int, ctypes.c_int, ctypes.POINTER(_P), ctypes.POINTER(ctypes.c_int64),
                                      ctypes.c_int, ctypes.POINTER(_P), _P, ctypes.c_size_t, _P]),
    "cbk_linear": (ctypes.c_int, _MM),
    "cbk_linear_act_workspace_bytes": (ctypes.c_size_t, [_DP, ctypes.c_int, ctypes.c_int]),
    "cbk_linear_act": (ctypes.c_int, _MM[:9] + [ctypes.c_int] + _MM[9:]),
}
ACT_CODE = {"gelu_tanh": 0, "silu": 1}


class CbkError(RuntimeError):
    pass


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise CbkError(f"{LIB_PATH} is missing: build it with `python -m cobalt_amd.build` "
                           "(hipcc, gfx950). There is no PyTorch fallback.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        if L.cbk_abi_version() != 1:
            raise CbkError(f"ABI version {L.cbk_abi_version()} != 1")
        _lib = L
    return _lib


def check(rc: int, what: str):
    if rc != 0:
        raise CbkError(f"{what} failed: {lib().cbk_strerror(rc).decode()} (status {rc})")
