"""ctypes front end of the C oracle (oracle/cbk_ref.c).  TEST INFRASTRUCTURE ONLY.

Takes the `packed` dictionaries of oracle/cbk_ref.py (data, scale, zero, optional row_off)
so the two oracles can be run on the same bytes.  Loaded by tests/, by
__graft_entry__.smoke() and by bench.py's cpu_baseline leg; never by the product package."""
import ctypes
import os

import numpy as np

from . import cbk_ref as R

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libcbk_ref.so")
        if not os.path.exists(path):
            from .build_c import build_oracle_c
            build_oracle_c()
        L = ctypes.CDLL(path)
        P, I = ctypes.c_void_p, ctypes.c_int
        L.cbk_ref_row_stride.restype = ctypes.c_size_t
        L.cbk_ref_row_stride.argtypes = [I] * 5
        L.cbk_ref_dequant.restype = I
        L.cbk_ref_dequant.argtypes = [P] * 5 + [I] * 11 + [P]
        L.cbk_ref_forward.restype = I
        L.cbk_ref_forward.argtypes = [P] * 5 + [I] * 9 + [P, I, P, P]
        L.cbk_ref_threads.restype = I
        L.cbk_ref_set_threads.argtypes = [I]
        _LIB = L
    return _LIB


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _args(packed, K, N, layout, col_scale, bits, group, keep_per_block, cs_splits):
    bits, group, kpb = R.canon(layout, bits, group, keep_per_block)
    data = np.ascontiguousarray(packed["data"], np.uint8)
    scale = np.ascontiguousarray(np.asarray(packed["scale"], np.float16)).view(np.uint16)
    zero = np.ascontiguousarray(packed["zero"], np.uint8)
    ro = packed.get("row_off")
    ro = None if ro is None else np.ascontiguousarray(ro, np.uint32)
    cs = None if col_scale is None else np.ascontiguousarray(np.asarray(col_scale, np.float16).reshape(-1, N)).view(np.uint16)
    cs_rows = 0 if cs is None else cs.shape[0]
    s0, s1 = (cs_splits[0], cs_splits[1]) if (cs_rows == 3 and cs_splits is not None) else (0, 0)
    keep = (data, scale, zero, ro, cs)
    return keep, [_ptr(data), _ptr(ro), _ptr(scale), _ptr(zero), _ptr(cs), K, N, layout, bits, group, kpb or 0,
                  cs_rows, s0, s1]


def dequant(packed, K, N, layout, col_scale=None, bits=None, group=None, keep_per_block=None, cs_splits=None,
            row0=0, nrows=None):
    nrows = K - row0 if nrows is None else nrows
    keep, a = _args(packed, K, N, layout, col_scale, bits, group, keep_per_block, cs_splits)
    out = np.empty((nrows, N), np.float32)
    rc = lib().cbk_ref_dequant(*a, row0, nrows, _ptr(out))
    if rc:
        raise ValueError(f"cbk_ref_dequant failed ({rc})")
    return out


def forward(packed, K, N, layout, x, col_scale=None, bias=None, bits=None, group=None, keep_per_block=None,
            cs_splits=None):
    """y[M, K] (float64) = x @ W_hat.T (+ bias), W_hat float32, double accumulate."""
    keep, a = _args(packed, K, N, layout, col_scale, bits, group, keep_per_block, cs_splits)
    x = np.ascontiguousarray(x, np.float32)
    M = x.shape[0]
    b = None if bias is None else np.ascontiguousarray(bias, np.float64)
    y = np.empty((M, K), np.float64)
    rc = lib().cbk_ref_forward(*a, _ptr(x), M, _ptr(b), _ptr(y))
    if rc:
        raise ValueError(f"cbk_ref_forward failed ({rc})")
    return y


def set_threads(n):
    lib().cbk_ref_set_threads(int(n))


def threads():
    return lib().cbk_ref_threads()
