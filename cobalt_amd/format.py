"""CBK1 packed-weight container for the MI355X kernels: layout ids, the packer that turns a
RAW CoBALT matrix (mask, q, scale, zero, col_scale) into the byte image the kernels read,
and `PackedMatrix`, the object that owns that image and hands out C-ABI descriptors.

Byte layouts 0-7 are the reference's (docs/FORMAT.md:65-122, src/cobaltkernel/pack_cobalt.py:98-250);
8 (BLKC) and 9 (DENSEB) extend the two shipped families to 2/3/4-bit codes, a group of 64 or
128 and any per-32-column survivor count: one LSB-first bit stream per row, survivor i of
block t at bits [(t*keep+i)*bits, ...) after the N/8-byte bitmap (BLKC), or the code of
column j at bits [j*bits, ...) (DENSEB); code planes are zero-padded to 16 bytes.

Everything here is torch and runs on whatever device its inputs live on.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

import torch

GROUP = 128
ARR_ALIGN = 256
BLOB_TAIL = 64
BLOCK = 32

SPARSE4, DENSE4, DENSE8, SPARSE4X, BF16, SPARSE4E, BLK1632_4, BLK1632_6, BLKC, DENSEB = range(10)
LAYOUT_NAME = {0: "SPARSE4", 1: "DENSE4", 2: "DENSE8", 3: "SPARSE4X", 4: "BF16", 5: "SPARSE4E",
               6: "BLK1632_4", 7: "BLK1632_6", 8: "BLKC", 9: "DENSEB"}
_DENSE = (DENSE4, DENSE8, DENSEB)
_BLK = (BLK1632_4, BLK1632_6, BLKC)
_SPARSE = (SPARSE4, SPARSE4X, SPARSE4E)

F32, F16, BF16T = 0, 1, 2
FLAG_ZERO_LE_128 = 1
FLAG_TILED16 = 2
FLAG_ZERO_ON_GRID = 4          # every stored zero point is itself a code (<= 2^bits - 1)


def zero_flags(zero_max: int, bits: int) -> int:
    """The two promises about the zero points a descriptor can carry (include/cbk.h)."""
    return (FLAG_ZERO_LE_128 if zero_max <= 128 else 0) | (FLAG_ZERO_ON_GRID if zero_max <= (1 << bits) - 1 else 0)
TILED_TAIL = 512


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.float16:
        return F16
    if dt == torch.bfloat16:
        return BF16T
    raise TypeError(f"unsupported dtype {dt}; the layer takes float16 / bfloat16 activations")


class CbkDesc(ctypes.Structure):
    """Mirror of `cbk_desc` in include/cbk.h."""
    _fields_ = [("data", ctypes.c_void_p), ("row_off", ctypes.c_void_p), ("scale", ctypes.c_void_p),
                ("zero", ctypes.c_void_p), ("col_scale", ctypes.c_void_p),
                ("K", ctypes.c_int32), ("N", ctypes.c_int32), ("layout", ctypes.c_int32),
                ("bits", ctypes.c_int32), ("group", ctypes.c_int32), ("keep", ctypes.c_int32),
                ("cs_rows", ctypes.c_int32), ("cs_split0", ctypes.c_int32), ("cs_split1", ctypes.c_int32),
                ("flags", ctypes.c_int32)]


def _align(x: int, a: int) -> int:
    return (x + a - 1) // a * a


def canon(layout: int, bits=None, group=None, keep=None) -> Tuple[int, int, int]:
    if layout == DENSE4:
        return 4, GROUP, 0
    if layout == DENSE8:
        return 8, GROUP, 0
    if layout in _SPARSE:
        return 4, GROUP, 0
    if layout == BLK1632_4:
        return 4, GROUP, 16
    if layout == BLK1632_6:
        return 6, GROUP, 16
    if layout == BLKC:
        if bits not in (2, 3, 4) or group not in (64, 128) or not (1 <= int(keep) <= 32):
            raise ValueError(f"BLKC needs bits in (2,3,4), group in (64,128), 1<=keep<=32; got {bits},{group},{keep}")
        return int(bits), int(group), int(keep)
    if layout == DENSEB:
        if bits not in (2, 3, 4, 8) or group not in (64, 128):
            raise ValueError(f"DENSEB needs bits in (2,3,4,8), group in (64,128); got {bits},{group}")
        return int(bits), int(group), 0
    raise ValueError(f"unknown layout {layout}")


def row_stride(layout: int, N: int, bits=None, group=None, keep=None) -> int:
    bits, group, keep = canon(layout, bits, group, keep)
    if layout in _DENSE:
        return _align((N * bits + 7) // 8, 16)
    if layout == BLK1632_6:
        return N // 2
    if layout in _BLK:
        return N // 8 + _align(((N // BLOCK) * keep * bits + 7) // 8, 16)
    raise ValueError("variable-length layout has no fixed row stride")


def bits_per_weight(layout: int, bits=None, group=None, keep=None, density: float = 0.5) -> float:
    """codes + mask + (16 + 8)/group, docs/FORMAT.md:78-81."""
    bits, group, keep = canon(layout, bits, group, keep)
    if layout in _DENSE:
        return bits + 24.0 / group
    if layout in _BLK:
        return 1.0 + bits * keep / 32.0 + 24.0 / group
    return 1.0 + bits * density + 24.0 / group


# --------------------------------------------------------------------------- bit helpers
def unpack_mask(mask_bytes: torch.Tensor, N: int) -> torch.Tensor:
    """uint8 [K, N/8] LSB-first -> bool [K, N]."""
    K = mask_bytes.shape[0]
    sh = torch.arange(8, device=mask_bytes.device, dtype=torch.uint8)
    return ((mask_bytes.reshape(K, N // 8, 1) >> sh) & 1).reshape(K, N).bool()


def pack_mask(keep: torch.Tensor) -> torch.Tensor:
    K, N = keep.shape
    w = (1 << torch.arange(8, device=keep.device, dtype=torch.int32))
    return (keep.reshape(K, N // 8, 8).to(torch.int32) * w).sum(-1).to(torch.uint8)


def pack_stream(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """int [K, n] -> uint8 [K, ceil(n*bits/8)]: code i at bits [i*bits, (i+1)*bits), LSB first.
    Eight codes make `bits` whole bytes, so the stream is assembled from 8-code words."""
    K, n = codes.shape
    n8 = _align(n, 8)
    c = codes.to(torch.int64)
    if n8 != n:
        c = torch.cat([c, torch.zeros(K, n8 - n, dtype=torch.int64, device=c.device)], 1)
    sh = torch.arange(8, device=c.device, dtype=torch.int64) * bits
    v = (c.reshape(K, n8 // 8, 8) << sh).sum(-1)                      # 8*bits-bit words
    bsh = torch.arange(bits, device=c.device, dtype=torch.int64) * 8
    by = ((v.unsqueeze(-1) >> bsh) & 0xFF).to(torch.uint8).reshape(K, n8 // 8 * bits)
    return by[:, : (n * bits + 7) // 8]


def unpack_stream(by: torch.Tensor, n: int, bits: int) -> torch.Tensor:
    K = by.shape[0]
    n8 = _align(n, 8)
    need = n8 // 8 * bits
    b = by[:, :need].to(torch.int64)
    if b.shape[1] < need:
        b = torch.cat([b, torch.zeros(K, need - b.shape[1], dtype=torch.int64, device=b.device)], 1)
    bsh = torch.arange(bits, device=by.device, dtype=torch.int64) * 8
    v = (b.reshape(K, n8 // 8, bits) << bsh).sum(-1)
    sh = torch.arange(8, device=by.device, dtype=torch.int64) * bits
    return ((v.unsqueeze(-1) >> sh) & ((1 << bits) - 1)).reshape(K, n8)[:, :n].to(torch.int32)


# --------------------------------------------------------------------------- zero repair
def fix_zero_range(qf, scale, zero, keep, nlevels, group):
    """Re-derive (scale, zero, q) from a 0-inclusive hull for groups whose integer zero point
    is off the grid (src/cobaltkernel/pack_cobalt.py:55-87)."""
    K, N = qf.shape
    G = N // group
    z = zero.to(torch.int32) if zero.dtype == torch.uint8 else torch.round(zero.float()).to(torch.int32)
    bad = (z < 0) | (z > nlevels)
    n_bad = int(bad.sum())
    sc = scale.float()
    if n_bad == 0:
        return qf, sc, z, 0
    q3 = qf.reshape(K, G, group)
    v = (q3 - z.reshape(K, G, 1).float()) * sc.reshape(K, G, 1)
    kv = keep.reshape(K, G, group)
    big = torch.finfo(torch.float32).max
    vmin = torch.where(kv, v, torch.full_like(v, big)).amin(-1)
    vmax = torch.where(kv, v, torch.full_like(v, -big)).amax(-1)
    empty = ~kv.any(-1)
    vmin = torch.where(empty, torch.zeros_like(vmin), vmin).clamp(max=0.0)
    vmax = torch.where(empty, torch.zeros_like(vmax), vmax).clamp(min=0.0)
    s2 = ((vmax - vmin) / nlevels).clamp(min=1e-12)
    z2 = torch.round(-vmin / s2).clamp(0, nlevels)
    q2 = torch.clamp(torch.round(v / s2.unsqueeze(-1) + z2.unsqueeze(-1)), 0, nlevels)
    qf = torch.where(bad.unsqueeze(-1), q2, q3).reshape(K, N)
    sc = torch.where(bad, s2, sc)
    z = torch.where(bad, z2.to(torch.int32), z)
    return qf, sc, z, n_bad


# --------------------------------------------------------------------------- container
@dataclass
class PackedMatrix:
    """One packed matrix: a single uint8 image holding 256-byte aligned arrays
    (data [+ row_off], scale, zero, col_scale) plus the integers that describe it."""
    blob: torch.Tensor
    offs: Dict[str, int]
    K: int
    N: int
    layout: int
    bits: int
    group: int
    keep: int
    cs_rows: int = 0
    cs_splits: Tuple[int, int] = (0, 0)
    data_bytes: int = 0
    n_survivors: int = 0
    n_zero_fixed: int = 0
    flags: int = 0
    meta: dict = field(default_factory=dict)

    @property
    def G(self) -> int:
        return self.N // self.group

    @property
    def device(self):
        return self.blob.device

    def to(self, device) -> "PackedMatrix":
        return PackedMatrix(self.blob.to(device), dict(self.offs), self.K, self.N, self.layout, self.bits,
                            self.group, self.keep, self.cs_rows, self.cs_splits, self.data_bytes,
                            self.n_survivors, self.n_zero_fixed, self.flags, dict(self.meta))

    def clone(self) -> "PackedMatrix":
        p = self.to(self.device)
        p.blob = self.blob.clone()
        return p

    @property
    def tiled(self) -> bool:
        return bool(self.flags & FLAG_TILED16)

    def _krows(self) -> int:
        return _align(self.K, 16) if self.tiled else self.K

    def to_tiled(self) -> "PackedMatrix":
        """The same matrix in the 16-row tile-interleaved order the kernels stream fastest: byte o
        of row k moves to (k//16)*16*stride + ((o//16)*16 + k%16)*16 + o%16, scale/zero entry (k, g)
        to index ((k//16)*G + g)*16 + k%16; K is padded with zero rows to a multiple of 16.  A pure
        permutation of the packed bytes, done once when a layer is built or loaded."""
        if self.tiled:
            return self
        if self.layout in _SPARSE:
            raise ValueError("the variable-length SPARSE4* layouts have no tiled form")
        K, G, dev = self.K, self.G, self.blob.device
        stride = self.data_bytes // K
        K16 = _align(K, 16) // 16
        rows = torch.zeros(K16 * 16, stride, dtype=torch.uint8, device=dev)
        rows[:K] = self.array("data")[: K * stride].view(K, stride)
        data = torch.cat([rows.view(K16, 16, stride // 16, 16).permute(0, 2, 1, 3).reshape(-1),
                          torch.zeros(TILED_TAIL, dtype=torch.uint8, device=dev)])
        sc = torch.zeros(K16 * 16, G, dtype=torch.float16, device=dev)
        sc[:K] = self.array("scale").view(K, G)
        zr = torch.zeros(K16 * 16, G, dtype=torch.uint8, device=dev)
        zr[:K] = self.array("zero").view(K, G)
        arrays = {"data": data, "scale": sc.view(K16, 16, G).permute(0, 2, 1).contiguous(),
                  "zero": zr.view(K16, 16, G).permute(0, 2, 1).contiguous()}
        if self.cs_rows:
            arrays["col_scale"] = self.array("col_scale")
        blob, offs = _assemble(arrays, dev)
        return PackedMatrix(blob, offs, K, self.N, self.layout, self.bits, self.group, self.keep, self.cs_rows,
                            self.cs_splits, K16 * 16 * stride, self.n_survivors, self.n_zero_fixed,
                            self.flags | FLAG_TILED16, dict(self.meta))

    def to_rowmajor(self) -> "PackedMatrix":
        """Inverse of to_tiled(): the reference's row-major CBK1 byte order."""
        if not self.tiled:
            return self
        K, G, dev = self.K, self.G, self.blob.device
        K16 = _align(K, 16) // 16
        stride = self.data_bytes // (K16 * 16)
        rows = self.array("data")[: K16 * 16 * stride].view(K16, stride // 16, 16, 16).permute(0, 2, 1, 3)
        data = torch.cat([rows.reshape(K16 * 16, stride)[:K].reshape(-1),
                          torch.zeros(BLOB_TAIL, dtype=torch.uint8, device=dev)])
        arrays = {"data": data,
                  "scale": self.array("scale").view(K16, G, 16).permute(0, 2, 1).reshape(K16 * 16, G)[:K].contiguous(),
                  "zero": self.array("zero").view(K16, G, 16).permute(0, 2, 1).reshape(K16 * 16, G)[:K].contiguous()}
        if self.cs_rows:
            arrays["col_scale"] = self.array("col_scale")
        blob, offs = _assemble(arrays, dev)
        return PackedMatrix(blob, offs, K, self.N, self.layout, self.bits, self.group, self.keep, self.cs_rows,
                            self.cs_splits, K * stride, self.n_survivors, self.n_zero_fixed,
                            self.flags & ~FLAG_TILED16, dict(self.meta))

    def array(self, name: str) -> torch.Tensor:
        kr = self._krows()
        n = {"data": self.data_bytes + (TILED_TAIL if self.tiled else BLOB_TAIL), "scale": kr * self.G * 2,
             "zero": kr * self.G, "col_scale": self.cs_rows * self.N * 2, "row_off": (self.K + 1) * 4}[name]
        v = self.blob[self.offs[name]: self.offs[name] + n]
        if name in ("scale", "col_scale"):
            return v.view(torch.float16)
        if name == "row_off":
            return v.view(torch.int32)
        return v

    def validate(self, deep: bool = False) -> "PackedMatrix":
        """Raise ValueError unless the integers describe arrays that lie inside the image and agree
        with each other: the checks a kernel launch relies on, made where a description enters from
        outside (a manifest entry, a state dict).  `deep` also reads the row offsets of a
        variable-length matrix (a device-to-host copy when the image is on a GPU)."""
        def bad(msg):
            raise ValueError(f"packed matrix {self.K}x{self.N} {LAYOUT_NAME.get(self.layout, self.layout)}: {msg}")
        if self.blob.dtype != torch.uint8 or self.blob.dim() != 1:
            bad("the image is not a flat uint8 tensor")
        if self.layout not in LAYOUT_NAME or self.layout == BF16:
            bad("unknown layout")
        try:
            want = canon(self.layout, self.bits, self.group, self.keep)
        except (ValueError, TypeError) as e:
            bad(str(e))
        if (self.bits, self.group, self.keep) != want:
            bad(f"bits/group/keep {(self.bits, self.group, self.keep)} do not fit the layout (want {want})")
        if self.K < 1 or self.N < 1 or self.N % GROUP:
            bad(f"K >= 1 and N a positive multiple of {GROUP} are required")
        if not 0 <= self.cs_rows <= 3:
            bad(f"cs_rows {self.cs_rows} outside 0..3")
        if self.cs_rows == 3:
            s0, s1 = self.cs_splits
            if s0 < 0 or s1 < 0 or s0 + s1 > self.K:
                bad(f"row ranges {self.cs_splits} of the three column-scale rows do not fit K")
        sparse = self.layout in _SPARSE
        if sparse and self.tiled:
            bad("a variable-length layout cannot be in tiled order")
        if self.data_bytes < 0:
            bad("negative data_bytes")
        if not sparse:
            st = row_stride(self.layout, self.N, self.bits, self.group, self.keep or None)
            if self.data_bytes != self._krows() * st:
                bad(f"data_bytes {self.data_bytes} is not rows x stride = {self._krows()} x {st}")
        need = ["data", "scale", "zero"] + (["row_off"] if sparse else []) + (["col_scale"] if self.cs_rows else [])
        align = {"data": 16, "scale": 4, "zero": 4, "col_scale": 16, "row_off": 4}     # what the library asks of the pointers
        kr, n = self._krows(), self.blob.numel()
        size = {"data": self.data_bytes + (TILED_TAIL if self.tiled else BLOB_TAIL), "scale": kr * self.G * 2,
                "zero": kr * self.G, "col_scale": self.cs_rows * self.N * 2, "row_off": (self.K + 1) * 4}
        for name in need:
            if name not in self.offs:
                bad(f"no offset for the {name} array")
            off = self.offs[name]
            if off < 0 or off % align[name]:
                bad(f"{name} starts at {off}, not on a {align[name]}-byte boundary")
            if off + size[name] > n:
                bad(f"{name} runs past the image ({off} + {size[name]} > {n})")
        if sparse and deep:
            ro = self.array("row_off").cpu().to(torch.int64)
            if int(ro[0]) != 0 or bool((ro[1:] < ro[:-1]).any()) or bool((ro % 16 != 0).any()) or int(ro[-1]) > self.data_bytes:
                bad("row offsets are not an increasing sequence of multiples of 16 from 0 to at most data_bytes")
        return self

    def stream_bytes(self) -> int:
        """Weight bytes one pass streams: rows + scale + zero (pack_cobalt.py:431-433)."""
        return self.data_bytes + self._krows() * self.G * 3

    def bpw(self) -> float:
        ro = (self.K + 1) * 4 if "row_off" in self.offs else 0
        return 8.0 * (self.stream_bytes() + ro) / (self.K * self.N)

    def desc(self) -> CbkDesc:
        base = self.blob.data_ptr()
        d = CbkDesc()
        d.data = base + self.offs["data"]
        d.row_off = base + self.offs["row_off"] if "row_off" in self.offs else None
        d.scale = base + self.offs["scale"]
        d.zero = base + self.offs["zero"]
        d.col_scale = base + self.offs["col_scale"] if self.cs_rows else None
        d.K, d.N, d.layout = self.K, self.N, self.layout
        d.bits, d.group, d.keep = self.bits, self.group, self.keep
        d.cs_rows, d.cs_split0, d.cs_split1 = self.cs_rows, self.cs_splits[0], self.cs_splits[1]
        d.flags = self.flags
        return d


def _assemble(arrays: Dict[str, torch.Tensor], device) -> Tuple[torch.Tensor, Dict[str, int]]:
    offs, pos = {}, 0
    for name, a in arrays.items():
        pos = _align(pos, ARR_ALIGN)
        offs[name] = pos
        pos += a.numel() * a.element_size()
    blob = torch.zeros(_align(pos, ARR_ALIGN), dtype=torch.uint8, device=device)
    for name, a in arrays.items():
        # a copy with contiguous strides: a tensor whose only non-unit stride sits on a size-1
        # dimension counts as contiguous, and its flat view would keep that stride
        b = a.reshape(-1).clone(memory_format=torch.contiguous_format).view(torch.uint8)
        blob[offs[name]: offs[name] + b.numel()] = b.to(device)
    return blob, offs


def pack_raw(mask_bits: Optional[torch.Tensor], q: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor,
             col_scale: Optional[torch.Tensor], layout: int, bits=None, group=None, keep=None,
             fix_zero: bool = True, cs_splits: Tuple[int, int] = (0, 0), chunk_rows: int = 2048) -> PackedMatrix:
    """RAW matrix -> PackedMatrix (same device as q).

    mask_bits uint8 [K, N/8] LSB-first or None; q [K, N] integer codes; scale, zero [K, N/group]
    (zero fp16 integer-valued or uint8); col_scale fp16 [N] or [cs_rows, N] or None.
    Follows src/cobaltkernel/pack_cobalt.py:98-199 (fixed-stride layouts)."""
    bits, group, kpb = canon(layout, bits, group, keep)
    if layout in _SPARSE:
        raise NotImplementedError("the variable-length SPARSE4* layouts are read, not produced, by this package")
    dev = q.device
    K, N = q.shape
    if N % 128 or N % group:
        raise ValueError(f"N={N} must be a multiple of 128 and of the group size")
    G = N // group
    nl = (1 << bits) - 1
    stride = row_stride(layout, N, bits, group, kpb)
    data = torch.zeros(K * stride + BLOB_TAIL, dtype=torch.uint8, device=dev)
    rows = data[: K * stride].view(K, stride)
    out_scale = torch.empty(K, G, dtype=torch.float16, device=dev)
    out_zero = torch.empty(K, G, dtype=torch.uint8, device=dev)
    n_surv = n_fixed = 0
    for k0 in range(0, K, chunk_rows):
        sl = slice(k0, min(K, k0 + chunk_rows))
        kc = sl.stop - sl.start
        qf = q[sl].float()
        if mask_bits is None:
            keepm = torch.ones(kc, N, dtype=torch.bool, device=dev)
            mb = torch.full((kc, N // 8), 255, dtype=torch.uint8, device=dev)
        else:
            mb = mask_bits[sl].to(dev).reshape(kc, N // 8)
            keepm = unpack_mask(mb, N)
        if fix_zero:
            qf, sc, zi, nf = fix_zero_range(qf, scale[sl].to(dev), zero[sl].to(dev), keepm, nl, group)
        else:
            z0 = zero[sl].to(dev)
            sc, nf = scale[sl].to(dev).float(), 0
            zi = z0.to(torch.int32) if z0.dtype == torch.uint8 else torch.round(z0.float()).to(torch.int32)
        n_fixed += nf
        n_surv += int(keepm.sum())
        qc = torch.clamp(qf, 0, nl).to(torch.int32)
        out_scale[sl] = sc.half()
        out_zero[sl] = zi.to(torch.uint8)
        if layout in _DENSE:
            qc = torch.where(keepm, qc, zi.repeat_interleave(group, dim=1))
            s = pack_stream(qc, bits)
            rows[sl, : s.shape[1]] = s
            continue
        NB = N // BLOCK
        cnt = keepm.reshape(kc, NB, BLOCK).sum(-1)
        if not bool((cnt == kpb).all()):
            r, c = [int(v) for v in torch.nonzero(cnt != kpb)[0]]
            raise ValueError(f"{LAYOUT_NAME[layout]} needs exactly {kpb} survivors in every aligned block of "
                             f"{BLOCK} columns; row {k0 + r} block {c} has {int(cnt[r, c])}")
        cod = qc[keepm].reshape(kc, NB * kpb)                 # survivors in column order
        rows[sl, : N // 8] = mb
        if layout == BLK1632_6:
            c3 = cod.reshape(kc, NB, 16)
            nib = ((c3[:, :, 0::2] & 0xF) | ((c3[:, :, 1::2] & 0xF) << 4)).to(torch.uint8)
            rows[sl, N // 8: N // 8 + NB * 8] = nib.reshape(kc, NB * 8)
            sh = torch.arange(8, device=dev, dtype=torch.int64) * 2
            he = (((c3[:, :, 0::2] >> 4) & 3).to(torch.int64) << sh).sum(-1)
            ho = (((c3[:, :, 1::2] >> 4) & 3).to(torch.int64) << (sh + 16)).sum(-1)
            hw = he | ho
            bsh = torch.arange(4, device=dev, dtype=torch.int64) * 8
            rows[sl, N * 3 // 8:] = ((hw.unsqueeze(-1) >> bsh) & 0xFF).to(torch.uint8).reshape(kc, NB * 4)
        else:
            s = pack_stream(cod, bits)
            rows[sl, N // 8: N // 8 + s.shape[1]] = s
    arrays = {"data": data, "scale": out_scale, "zero": out_zero}
    cs_rows = 0
    if col_scale is not None:
        cs = col_scale.to(dev).to(torch.float16).reshape(-1, N)
        cs_rows = cs.shape[0]
        arrays["col_scale"] = cs
    blob, offs = _assemble(arrays, dev)
    flags = zero_flags(int(out_zero.max()), bits)
    return PackedMatrix(blob, offs, K, N, layout, bits, group, kpb, cs_rows, tuple(cs_splits),
                        K * stride, n_surv, n_fixed, flags)


def from_arrays(data, scale, zero, col_scale, K, N, layout, bits=None, group=None, keep=None, row_off=None,
                cs_splits=(0, 0), device=None) -> PackedMatrix:
    """Wrap already-packed arrays (e.g. read from a CBK1 `.bin`) without touching their bytes."""
    bits, group, kpb = canon(layout, bits, group, keep)
    data = torch.as_tensor(data).reshape(-1).view(torch.uint8)
    dev = device or data.device
    arrays = {"data": data}
    if row_off is not None:
        arrays["row_off"] = torch.as_tensor(row_off).reshape(-1).view(torch.uint8)
    arrays["scale"] = torch.as_tensor(scale).reshape(-1).view(torch.uint8)
    arrays["zero"] = torch.as_tensor(zero).reshape(-1).view(torch.uint8)
    cs_rows = 0
    if col_scale is not None:
        cs = torch.as_tensor(col_scale).reshape(-1, N)
        cs_rows = cs.shape[0]
        arrays["col_scale"] = cs.reshape(-1).clone(memory_format=torch.contiguous_format).view(torch.uint8)
    blob, offs = _assemble(arrays, dev)
    flags = zero_flags(int(torch.as_tensor(zero).reshape(-1).view(torch.uint8).max()), bits)
    return PackedMatrix(blob, offs, K, N, layout, bits, group, kpb, cs_rows, tuple(cs_splits),
                        data.numel() - BLOB_TAIL, flags=flags)


def fuse_rows(parts, interleave: bool = False) -> PackedMatrix:
    """Row-fused matrix of several packed matrices that multiply the same activation
    (docs/FORMAT.md:126-151): `interleave=False` concatenates two or three of them (q | k | v;
    col_scale [3, N], cs_splits = the first two row counts; two parts get an empty third range),
    `interleave=True` alternates the rows of two equally sized ones (gate, up: row 2i = gate i,
    row 2i+1 = up i; col_scale [2, N] by row parity).  The parts are row-major, fixed-stride and
    share layout, code width, group and survivors per block."""
    parts = list(parts)
    p0 = parts[0]
    if interleave and len(parts) != 2:
        raise ValueError("interleaving takes exactly two matrices")
    if not interleave and not 2 <= len(parts) <= 3:
        raise ValueError("concatenation takes two or three matrices")
    for p in parts:
        if p.tiled or "row_off" in p.offs:
            raise ValueError("fuse the row-major, fixed-stride form")
        if (p.N, p.layout, p.bits, p.group, p.keep) != (p0.N, p0.layout, p0.bits, p0.group, p0.keep):
            raise ValueError("the parts must share N, layout, bits, group and keep")
        if p.cs_rows != 1:
            raise ValueError("every part carries one col_scale vector")
    stride = row_stride(p0.layout, p0.N, p0.bits, p0.group, p0.keep or None)
    rows = [p.array("data")[: p.K * stride].view(p.K, stride) for p in parts]
    sc = [p.array("scale").view(p.K, p.G) for p in parts]
    zp = [p.array("zero").view(p.K, p.G) for p in parts]
    cs = torch.stack([p.array("col_scale").view(p.N) for p in parts])
    if interleave:
        if parts[0].K != parts[1].K:
            raise ValueError("interleaving needs equally many rows")
        il = lambda a, b: torch.stack([a, b], 1).reshape(2 * a.shape[0], a.shape[1])
        data, scale, zero = il(*rows), il(*sc), il(*zp)
        splits = (0, 0)
    else:
        data, scale, zero = torch.cat(rows), torch.cat(sc), torch.cat(zp)
        if len(parts) == 2:
            cs = torch.cat([cs, cs[1:]])
        splits = (parts[0].K, parts[1].K)
    K = data.shape[0]
    tail = torch.zeros(BLOB_TAIL, dtype=torch.uint8, device=data.device)
    out = from_arrays(torch.cat([data.reshape(-1), tail]), scale.contiguous(), zero.contiguous(), cs, K, p0.N,
                      p0.layout, p0.bits, p0.group, p0.keep or None, cs_splits=splits, device=data.device)
    out.n_survivors = sum(p.n_survivors for p in parts)
    return out


def _synth_sparse(K, N, layout, bits, group, g, dev, cs_rows) -> PackedMatrix:
    """synth_packed for the survivor-stream layouts: every column kept with probability 1/2, rows
    laid out as src/cobaltkernel/pack_cobalt.py:201-250 does ([bitmap N/8][group byte offsets u16,
    SPARSE4X / SPARSE4E][pad to 16][codes, every group padded to whole bytes], rows padded to 16)."""
    G = N // group
    has_goff = layout != SPARSE4
    hdr = _align(N // 8 + (_align(G * 2, 16) if has_goff else 0), 16)
    mask = torch.randint(0, 256, (K, N // 8), generator=g, device=dev, dtype=torch.int32).to(torch.uint8)
    cnt = unpack_mask(mask, N).reshape(K, G, group).sum(-1).to(torch.int64)
    gbytes = (cnt + 1) // 2
    gcum = torch.cumsum(gbytes, 1) - gbytes
    row_bytes = (hdr + gbytes.sum(1) + 15) // 16 * 16
    row_off = torch.zeros(K + 1, dtype=torch.int64, device=dev)
    row_off[1:] = torch.cumsum(row_bytes, 0)
    total = int(row_off[K])
    if total >= 1 << 32:
        raise ValueError("the rows do not fit 32-bit offsets")
    data = torch.randint(0, 256, (total + BLOB_TAIL,), generator=g, device=dev, dtype=torch.int32).to(torch.uint8)
    head = torch.zeros(K, hdr, dtype=torch.uint8, device=dev)
    head[:, : N // 8] = mask
    if has_goff:
        head[:, N // 8: N // 8 + 2 * G] = gcum.to(torch.int16).view(torch.uint8).reshape(K, 2 * G)
    pos = row_off[:K, None] + torch.arange(hdr, device=dev)[None, :]
    data[pos.reshape(-1)] = head.reshape(-1)
    scale = (torch.rand(K, G, generator=g, device=dev) * 0.01 + 1e-3).half()
    zero = torch.randint(0, 1 << bits, (K, G), generator=g, device=dev, dtype=torch.int32).to(torch.uint8)
    arrays = {"data": data, "scale": scale, "zero": zero, "row_off": row_off.to(torch.int32).view(torch.uint8)}
    if cs_rows:
        arrays["col_scale"] = (torch.rand(cs_rows, N, generator=g, device=dev) * 1.5 + 0.5).half()
    blob, offs = _assemble(arrays, dev)
    return PackedMatrix(blob, offs, K, N, layout, bits, group, 0, cs_rows, (0, 0), total, int(cnt.sum()), 0,
                        FLAG_ZERO_LE_128 | FLAG_ZERO_ON_GRID)


def synth_packed(K: int, N: int, layout: int, bits=None, group=None, keep=None, seed: int = 0,
                 device="cpu", cs_rows: int = 1) -> PackedMatrix:
    """A VALID packed matrix with random content, made directly in packed form (the idea of
    src/cobaltkernel/test_gemv.py:84-138): random per-block masks with the exact cardinality,
    random code bytes, scales in [1e-3, 1.1e-2), zeros on the grid, col_scale in [0.5, 2).
    For the dense family every column counts as a survivor.  Used for bandwidth runs, where the
    kernel's time depends on the mask statistics and not on the values."""
    bits, group, kpb = canon(layout, bits, group, keep)
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed)
    G = N // group
    if layout in _SPARSE:
        return _synth_sparse(K, N, layout, bits, group, g, dev, cs_rows)
    stride = row_stride(layout, N, bits, group, kpb)
    data = torch.zeros(K * stride + BLOB_TAIL, dtype=torch.uint8, device=dev)
    rows = data[: K * stride].view(K, stride)
    code_lo = 0 if layout in _DENSE else N // 8
    nbytes = ((N * bits + 7) // 8) if layout in _DENSE else \
        ((N // 2 - N // 8) if layout == BLK1632_6 else ((N // BLOCK) * kpb * bits + 7) // 8)
    rows[:, code_lo: code_lo + nbytes] = torch.randint(0, 256, (K, nbytes), generator=g, device=dev,
                                                       dtype=torch.int32).to(torch.uint8)
    n_surv = K * N
    if layout in _BLK:
        r = torch.rand(K, N // BLOCK, BLOCK, generator=g, device=dev)
        idx = torch.topk(r, kpb, dim=-1).indices
        kb = torch.zeros_like(r, dtype=torch.bool).scatter_(-1, idx, True)
        rows[:, : N // 8] = pack_mask(kb.reshape(K, N))
        n_surv = K * (N // BLOCK) * kpb
        tailbits = (N // BLOCK) * kpb * bits
        if layout == BLKC and tailbits % 8:                     # keep the stream padding zero
            rows[:, code_lo + nbytes - 1] &= (1 << (tailbits % 8)) - 1
    scale = (torch.rand(K, G, generator=g, device=dev) * 0.01 + 1e-3).half()
    zero = torch.randint(0, 1 << bits, (K, G), generator=g, device=dev, dtype=torch.int32).to(torch.uint8)
    arrays = {"data": data, "scale": scale, "zero": zero}
    if cs_rows:
        arrays["col_scale"] = (torch.rand(cs_rows, N, generator=g, device=dev) * 1.5 + 0.5).half()
    blob, offs = _assemble(arrays, dev)
    return PackedMatrix(blob, offs, K, N, layout, bits, group, kpb, cs_rows, (0, 0), K * stride, n_surv, 0,
                        FLAG_ZERO_LE_128 | FLAG_ZERO_ON_GRID)
