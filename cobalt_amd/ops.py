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


def pack_raw(mask_bits, q, scale, zero, col_scale, layout, bits=None, group=None, keep=None, fix_zero=True,
             cs_splits=(0, 0), tiled=True) -> PackedMatrix:
    """RAW arrays on the GPU -> PackedMatrix on the GPU, written by the library's packing kernel
    (rows, scale, zero point, and the re-derivation of zero points that are off the code grid,
    src/cobaltkernel/pack_cobalt.py:55-87), in the tiled order the decode kernel streams (`tiled`)
    or the reference's row-major order.  Same arguments and same bytes as `format.pack_raw`
    (which is torch and runs anywhere)."""
    from . import format as F
    bits, group, kpb = F.canon(layout, bits, group, keep)
    if layout in F._SPARSE:
        raise NotImplementedError("the variable-length SPARSE4* layouts are read, not produced, by this package")
    if q.device.type != "cuda":
        raise _lib.CbkError("ops.pack_raw packs on the GPU; use format.pack_raw for tensors on the CPU")
    dev = q.device
    K, N = q.shape
    if N % 128 or N % group:
        raise ValueError(f"N={N} must be a multiple of 128 and of the group size")
    G = N // group
    nl = (1 << bits) - 1
    mb = None if mask_bits is None else mask_bits.to(dev).reshape(K, N // 8).contiguous()
    q8 = (q if q.dtype == torch.uint8 else q.clamp(0, 255).to(torch.uint8)).contiguous()
    sc16 = scale.to(dev).to(torch.float16).reshape(K, G).contiguous()
    z = zero.to(dev).reshape(K, G)
    z = (z if z.dtype == torch.uint8 else z.to(torch.float16)).contiguous()
    stride = F.row_stride(layout, N, bits, group, kpb or None)
    kr = F._align(K, 16) if tiled else K
    sizes = {"data": kr * stride + (F.TILED_TAIL if tiled else F.BLOB_TAIL), "scale": kr * G * 2, "zero": kr * G}
    cs = None
    if col_scale is not None:
        cs = col_scale.to(dev).to(torch.float16).reshape(-1, N).contiguous()
        sizes["col_scale"] = cs.numel() * 2
    offs, pos = {}, 0
    for name, n in sizes.items():
        pos = F._align(pos, F.ARR_ALIGN)
        offs[name] = pos
        pos += n
    blob = torch.zeros(F._align(pos, F.ARR_ALIGN), dtype=torch.uint8, device=dev)
    if cs is not None:
        blob[offs["col_scale"]: offs["col_scale"] + sizes["col_scale"]] = cs.reshape(-1).view(torch.uint8)
    if layout in F._DENSE:
        n_surv = K * N if mb is None else int(F.unpack_mask(mb, N).sum())
    else:
        n_surv = K * (N // F.BLOCK) * kpb
    pm = PackedMatrix(blob, offs, K, N, layout, bits, group, kpb, 0 if cs is None else cs.shape[0], tuple(cs_splits),
                      kr * stride, n_surv, 0, (F.FLAG_TILED16 if tiled else 0))
    status = torch.zeros(2, dtype=torch.int32, device=dev)
    d = pm.desc()
    rc = _lib.lib().cbk_pack(ctypes.byref(d), mb.data_ptr() if mb is not None else None, q8.data_ptr(), sc16.data_ptr(),
                             z.data_ptr(), 3 if z.dtype == torch.uint8 else F.F16, int(bool(fix_zero)), status.data_ptr(),
                             _stream_ptr(dev))
    _lib.check(rc, "cbk_pack")
    wrong, pm.n_zero_fixed = (int(v) for v in status.tolist())
    if wrong & 2:
        raise ValueError(f"{F.LAYOUT_NAME[layout]} stores the zero point as the code of a pruned column, and a zero point "
                         f"of this matrix is above {nl}: such a column would not dequantise to 0 (pack with fix_zero=True, "
                         f"or keep a bitmap layout)")
    if wrong & 1:
        raise ValueError(f"{F.LAYOUT_NAME[layout]} needs exactly {kpb} survivors in every aligned block of "
                         f"{F.BLOCK} columns; the mask has a block with another count")
    pm.flags |= F.zero_flags(int(pm.array("zero").max()), bits)
    return pm.validate()


def unpack(pm: PackedMatrix):
    """(mask_bits uint8 [K, N/8], q uint8 [K, N]) of a packed matrix of any layout on the GPU: the
    inverse of `pack_raw` up to the zero-point repair (a dense layout returns its stored codes,
    the zero point at pruned columns, and an all-ones mask)."""
    _require_gpu(pm)
    q = torch.empty(pm.K, pm.N, dtype=torch.uint8, device=pm.blob.device)
    mask = torch.empty(pm.K, pm.N // 8, dtype=torch.uint8, device=pm.blob.device)
    d = pm.desc()
    _lib.check(_lib.lib().cbk_unpack(ctypes.byref(d), q.data_ptr(), mask.data_ptr(), _stream_ptr(pm.blob.device)), "cbk_unpack")
    return mask, q


def with_group_offsets(pm: PackedMatrix) -> PackedMatrix:
    """A SPARSE4 matrix as SPARSE4X: the same mask words and code bytes, plus, behind the mask
    plane of every row, the table of 16-bit byte offsets of its groups' codes that SPARSE4X / 4E
    rows carry (pack_cobalt.py:201-250: the running sum of ceil(survivors / 2) over the groups
    before), padded to 16 bytes.  Two bytes per group (0.125 bits per weight) more; with them the
    rows are served by the 16-row matrix-core stream kernel instead of the row kernel, which has
    to sum the offsets of every row itself.  Runs on the device the matrix is on."""
    from . import format as F
    if pm.layout != F.SPARSE4:
        raise ValueError("only SPARSE4 rows lack the offset table")
    K, N, G = pm.K, pm.N, pm.G
    dev = pm.device
    data = pm.array("data")
    ro = pm.array("row_off").to(torch.int64) & 0xFFFFFFFF                     # [K + 1]
    nm = N // 8
    gp = (2 * G + 15) // 16 * 16
    ar = lambda n: torch.arange(n, device=dev, dtype=torch.int64)
    mask = data[ro[:K, None] + ar(nm)[None, :]]                               # [K, N / 8]
    popc = torch.tensor([bin(i).count("1") for i in range(256)], dtype=torch.int64, device=dev)
    cnt = popc[mask.to(torch.int64)].view(K, G, pm.group // 8).sum(-1)
    gbytes = (cnt + 1) // 2
    goff = torch.cumsum(gbytes, 1) - gbytes
    if int(goff.max()) >= 1 << 16:
        raise ValueError("a row's codes exceed the 16-bit offsets of SPARSE4X")
    total = int(ro[K])
    new_ro = ro + ar(K + 1) * gp
    if int(new_ro[K]) >= 1 << 32:
        raise ValueError("the image would exceed 32-bit row offsets")
    out = torch.zeros(total + K * gp + F.BLOB_TAIL, dtype=torch.uint8, device=dev)
    out[new_ro[:K, None] + ar(nm)[None, :]] = mask
    gb = torch.stack([goff & 0xFF, goff >> 8], -1).to(torch.uint8).view(K, 2 * G)
    out[new_ro[:K, None] + nm + ar(2 * G)[None, :]] = gb
    clen = ro[1:] - ro[:K] - nm                                               # code bytes (with padding) of every row
    row = torch.repeat_interleave(ar(K), clen)
    within = ar(int(clen.sum())) - torch.repeat_interleave(torch.cumsum(clen, 0) - clen, clen)
    out[new_ro[row] + nm + gp + within] = data[ro[row] + nm + within]
    cs = pm.array("col_scale").view(pm.cs_rows, N) if pm.cs_rows else None
    res = F.from_arrays(out, pm.array("scale").view(K, G), pm.array("zero").view(K, G), cs, K, N, F.SPARSE4X,
                        pm.bits, pm.group, None, row_off=new_ro.to(torch.int32), cs_splits=pm.cs_splits, device=dev)
    res.n_survivors = pm.n_survivors
    return res


def transcode(pm: PackedMatrix, layout: int, bits=None, group=None, keep=None, tiled=True) -> PackedMatrix:
    """The same weights in another fixed-stride layout (same codes, scales, zero points and column
    scales; every weight dequantises to the same value).  The use: a survivor-stream matrix
    (SPARSE4*, which the row kernel serves at about a tenth of the matrix-core kernels' rate)
    as DENSE4, one bit per weight more for the fast kernels."""
    from . import format as F
    mask, q = unpack(pm)
    rm = pm.to_rowmajor() if pm.tiled else pm
    cs = rm.array("col_scale").view(rm.cs_rows, rm.N) if rm.cs_rows else None
    out = pack_raw(None if pm.layout in F._DENSE else mask, q, rm.array("scale").view(rm.K, rm.G), rm.array("zero").view(rm.K, rm.G),
                   cs, layout, bits, group, keep, fix_zero=False, cs_splits=rm.cs_splits, tiled=tiled)
    out.n_survivors = pm.n_survivors
    return out
