"""Operator-level Python surface over the C ABI: dequant / gemv / gemm / linear on a
PackedMatrix.  torch is used for device memory and the current stream only."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib
from .format import PackedMatrix, dtype_code

_workspaces = {}


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_gpu(pm: PackedMatrix, *tensors):
    if pm.blob.device.type != "cuda":
        raise _lib.CbkError("the packed matrix must live on the GPU (PackedMatrix.to('cuda')); "
                            "this package has no CPU execution path")
    for t in tensors:
        if t is not None and t.device != pm.blob.device:
            raise _lib.CbkError(f"tensor on {t.device}, packed matrix on {pm.blob.device}")


def workspace_for(pm: PackedMatrix, M: int) -> Optional[torch.Tensor]:
    """A cached per-(device, stream) scratch tensor large enough for this call, or None."""
    need = _lib.lib().cbk_workspace_bytes(ctypes.byref(pm.desc()), int(M))
    if need == 0:
        return None
    key = (pm.blob.device, torch.cuda.current_stream(pm.blob.device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=pm.blob.device)
        _workspaces[key] = ws
    return ws


def dequant(pm: PackedMatrix, dtype=torch.float32, row0: int = 0, nrows: Optional[int] = None,
            with_col_scale: bool = True) -> torch.Tensor:
    """W_hat[row0:row0+nrows] as a dense tensor (bit-exact float32 formula, one cast)."""
    _require_gpu(pm)
    nrows = pm.K - row0 if nrows is None else nrows
    out = torch.empty(nrows, pm.N, dtype=dtype, device=pm.blob.device)
    d = pm.desc()
    rc = _lib.lib().cbk_dequant(ctypes.byref(d), row0, nrows, int(with_col_scale), out.data_ptr(),
                                dtype_code(dtype), pm.N, _stream_ptr(pm.blob.device))
    _lib.check(rc, "cbk_dequant")
    return out


def _matmul(entry: str, pm: PackedMatrix, x: torch.Tensor, bias, out_dtype, workspace):
    _require_gpu(pm, x, bias)
    if x.shape[-1] != pm.N:
        raise ValueError(f"x has {x.shape[-1]} input features, the matrix has N={pm.N}")
    lead = x.shape[:-1]
    x2 = x.reshape(-1, pm.N)
    if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) % 8) or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    M = x2.shape[0]
    out_dtype = out_dtype or x.dtype
    y = torch.empty(M, pm.K, dtype=out_dtype, device=x.device)
    if M == 0:
        return y.reshape(*lead, pm.K)
    if bias is not None and bias.dtype != out_dtype:
        bias = bias.to(out_dtype)
    ws = workspace if workspace is not None else workspace_for(pm, M)
    d = pm.desc()
    ldx = x2.stride(0) if M > 1 else pm.N
    rc = getattr(_lib.lib(), entry)(ctypes.byref(d), x2.data_ptr(), dtype_code(x2.dtype), M, ldx,
                                    y.data_ptr(), dtype_code(out_dtype), pm.K,
                                    bias.data_ptr() if bias is not None else None,
                                    ws.data_ptr() if ws is not None else None,
                                    ws.numel() if ws is not None else 0, _stream_ptr(x.device))
    _lib.check(rc, entry)
    return y.reshape(*lead, pm.K)


def gemv(pm, x, bias=None, out_dtype=None, workspace=None):
    """Decode path (at most 16 activation rows)."""
    return _matmul("cbk_gemv", pm, x, bias, out_dtype, workspace)


def gemm(pm, x, bias=None, out_dtype=None, workspace=None):
    """Prefill path."""
    return _matmul("cbk_gemm", pm, x, bias, out_dtype, workspace)


def linear(pm, x, bias=None, out_dtype=None, workspace=None):
    """y = x @ W_hat.T (+ bias): decode kernel up to 8 rows, prefill kernel above."""
    return _matmul("cbk_linear", pm, x, bias, out_dtype, workspace)


def linear_act(pm, x, act: str, bias=None, out_dtype=None):
    """First half of a gated MLP on a gate/up matrix (rows 2i gate, 2i+1 up):
    y[..., i] = act(t[..., 2i]) * t[..., 2i+1] with t = x @ W_hat.T (+ bias), act 'gelu_tanh' or
    'silu' (EPI_GEGLU_BF16 / EPI_SWIGLU_BF16, src/cobaltkernel/csrc/cobalt_gemm.cuh:30-33)."""
    if act not in _lib.ACT_CODE:
        raise ValueError(f"act must be one of {sorted(_lib.ACT_CODE)}, got {act!r}")
    _require_gpu(pm, x, bias)
    if x.shape[-1] != pm.N:
        raise ValueError(f"x has {x.shape[-1]} input features, the matrix has N={pm.N}")
    if pm.K % 2:
        raise ValueError("a gate/up matrix has an even number of rows")
    lead = x.shape[:-1]
    x2 = x.reshape(-1, pm.N)
    if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) % 8) or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    M = x2.shape[0]
    out_dtype = out_dtype or x.dtype
    y = torch.empty(M, pm.K // 2, dtype=out_dtype, device=x.device)
    if M == 0:
        return y.reshape(*lead, pm.K // 2)
    if bias is not None and bias.dtype != out_dtype:
        bias = bias.to(out_dtype)
    L = _lib.lib()
    d = pm.desc()
    need = L.cbk_linear_act_workspace_bytes(ctypes.byref(d), M, dtype_code(out_dtype))
    key = (pm.blob.device, torch.cuda.current_stream(pm.blob.device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=pm.blob.device)
        _workspaces[key] = ws
    ldx = x2.stride(0) if M > 1 else pm.N
    rc = L.cbk_linear_act(ctypes.byref(d), x2.data_ptr(), dtype_code(x2.dtype), M, ldx, y.data_ptr(),
                          dtype_code(out_dtype), pm.K // 2, bias.data_ptr() if bias is not None else None,
                          _lib.ACT_CODE[act], ws.data_ptr(), ws.numel(), _stream_ptr(x.device))
    _lib.check(rc, "cbk_linear_act")
    return y.reshape(*lead, pm.K // 2)


def gemv_batch(pms, xs, biases=None, out_dtype=None):
    """Independent decode GEMVs in one launch pair: ys[i] = xs[i] @ W_hat_i.T (+ biases[i]).
    All xs share the number of rows (<= 16) and the dtype; at most 8 matrices."""
    n = len(pms)
    if n == 0:
        return []
    L = _lib.lib()
    M = xs[0].reshape(-1, pms[0].N).shape[0]
    out_dtype = out_dtype or xs[0].dtype
    x2, ys, bs = [], [], []
    for i, (pm, x) in enumerate(zip(pms, xs)):
        bias = biases[i] if biases is not None else None
        _require_gpu(pm, x, bias)
        xi = x.reshape(-1, pm.N)
        if xi.shape[0] != M or xi.dtype != xs[0].dtype:
            raise ValueError("all activations of a batch share the row count and the dtype")
        if xi.stride(-1) != 1 or (M > 1 and xi.stride(0) % 8) or xi.data_ptr() % 16:
            xi = xi.contiguous()
        x2.append(xi)
        ys.append(torch.empty(M, pm.K, dtype=out_dtype, device=x.device))
        bs.append(None if bias is None else bias.to(out_dtype))
    descs = (_lib.CbkDesc * n)(*[pm.desc() for pm in pms])
    need = L.cbk_gemv_batch_workspace_bytes(n, descs, M)
    key = (pms[0].blob.device, torch.cuda.current_stream(pms[0].blob.device).cuda_stream)
    ws = _workspaces.get(key)
    if need and (ws is None or ws.numel() < need):
        ws = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=pms[0].blob.device)
        _workspaces[key] = ws
    P = ctypes.c_void_p
    xp = (P * n)(*[t.data_ptr() for t in x2])
    yp = (P * n)(*[t.data_ptr() for t in ys])
    bp = (P * n)(*[(t.data_ptr() if t is not None else None) for t in bs])
    ldx = (ctypes.c_int64 * n)(*[(t.stride(0) if M > 1 else pm.N) for t, pm in zip(x2, pms)])
    ldy = (ctypes.c_int64 * n)(*[pm.K for pm in pms])
    rc = L.cbk_gemv_batch(n, descs, xp, ldx, dtype_code(x2[0].dtype), M, yp, ldy, dtype_code(out_dtype), bp,
                          ws.data_ptr() if need else None, ws.numel() if need else 0,
                          _stream_ptr(pms[0].blob.device))
    _lib.check(rc, "cbk_gemv_batch")
    return [y.reshape(*x.shape[:-1], pm.K) for y, x, pm in zip(ys, xs, pms)]
