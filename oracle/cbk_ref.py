"""CPU oracle for the CBK1 sparse low-bit linear layer.  TEST INFRASTRUCTURE ONLY.

This module is a numpy restatement of the reference's packed-weight format, its
packer, its dequantiser and its dequantise-then-matmul forward.  It exists so that the
HIP kernels can be checked against it; it is never imported by the product package
(`cobalt_amd/`), only by `tests/`, by `__graft_entry__.smoke()` and by the `cpu_baseline`
leg of `bench.py`.

Reference files each function follows (paths relative to the reference checkout):

  unpack_bits / pack_bits      src/cobaltkernel/pack_cobalt.py:90-94, quantize_cobalt.py:326
  fix_zero_range               src/cobaltkernel/pack_cobalt.py:55-87
  pack_matrix                  src/cobaltkernel/pack_cobalt.py:98-250, docs/FORMAT.md:83-122
  unpack_codes / dequant       src/cobaltkernel/dequant_ref.py:36-103,
                               src/cobaltkernel/pack_cobalt.py:277-334,
                               src/cobaltkernel/cobalt_math.py:328-332,
                               sinq/sparse_quant.py:1635-1681
  col_scale_rows               src/cobaltkernel/csrc/cobalt_format.h:77-99,
                               src/cobaltkernel/dequant_ref.py:73-82
  forward_ref                  benchmarks/benchmark_suite.py:1200-1217
  synth_raw_matrix             src/cobaltkernel/pack_cobalt.py:338-371 (same recipe, numpy RNG)
  rtn_dense                    src/cobaltkernel/pack_cobalt.py:375-386
  stream_bytes / bpw           src/cobaltkernel/pack_cobalt.py:414-434, docs/FORMAT.md:65-81
  make_blob                    src/cobaltkernel/test_gemv.py:57-80, pack_cobalt.py:390-411

Layouts 0-7 are the reference's CBK1 layouts, byte for byte.  Layouts 8 and 9 are this
build's extension (the reference has no packed layout for 2/3-bit codes, for a group of
64 or for a block cardinality other than 16 of 32); their *dequantisation semantics* are
the reference's formula, their byte layout is defined here:

  BLKC  (8): per row  [mask plane N/8 B][code plane], exactly `keep` survivors in every
             aligned block of 32 columns.  The code plane is one LSB-first bit stream:
             survivor i (column order) of block t occupies bits [(t*keep+i)*bits,
             (t*keep+i+1)*bits).  The plane is zero-padded to a multiple of 16 bytes.
             (bits=4, keep=16, group=128) is byte-identical to BLK1632_4.
  DENSEB(9): per row one LSB-first bit stream with the code of column j at bits
             [j*bits, (j+1)*bits); pruned columns hold the group's zero point; padded to
             a multiple of 16 bytes.  bits=4 is byte-identical to DENSE4, bits=8 to DENSE8.

Parity status: every function here is pinned by tests/test_oracle_*.py through hand
vectors, the reference documentation's known answers, an independent per-position
decoder and round trips, except where a docstring says "parity unpinned"; the zero-point
repair, the variable-length layouts (SPARSE4, SPARSE4X, SPARSE4E), the fixed-stride layouts
(DENSE4, DENSE8, BLK1632_4, BLK1632_6), the interleaved gate/up fusion with two column-scale
rows and the row-concatenated q|k|v with three in addition by bytes and values the reference's
own packer and decoder wrote (tests/golden/fix_zero_range.npz, sparse_stream.npz,
fixed_stride.npz, cbk1_dir/ with cbk1_dir_expect.npz).
"""
from __future__ import annotations

import numpy as np

# ----------------------------------------------------------------------------- constants
GROUP = 128            # the reference's only group size (pack_cobalt.py:23)
ROW_ALIGN = 16
ARR_ALIGN = 256
BLOB_TAIL = 64
BLOCK = 32

SPARSE4, DENSE4, DENSE8, SPARSE4X, BF16, SPARSE4E, BLK1632_4, BLK1632_6 = range(8)
BLKC, DENSEB = 8, 9
LAYOUT_NAME = {0: "SPARSE4", 1: "DENSE4", 2: "DENSE8", 3: "SPARSE4X", 4: "BF16",
               5: "SPARSE4E", 6: "BLK1632_4", 7: "BLK1632_6", 8: "BLKC", 9: "DENSEB"}
SPARSE_FAMILY = (SPARSE4, SPARSE4X, SPARSE4E)
DENSE_FAMILY = (DENSE4, DENSE8, DENSEB)
BLK_FAMILY = (BLK1632_4, BLK1632_6, BLKC)


def _align(x, a):
    return (x + a - 1) // a * a


def canon(layout, bits=None, group=None, keep=None):
    """Fill in the parameters the reference layouts imply. Returns (bits, group, keep)."""
    if layout == DENSE4:
        return 4, GROUP, 0
    if layout == DENSE8:
        return 8, GROUP, 0
    if layout in SPARSE_FAMILY:
        return 4, GROUP, 0
    if layout == BLK1632_4:
        return 4, GROUP, 16
    if layout == BLK1632_6:
        return 6, GROUP, 16
    if layout == BLKC:
        assert bits in (2, 3, 4) and group in (64, 128) and 1 <= keep <= 32
        return bits, group, keep
    if layout == DENSEB:
        assert bits in (2, 3, 4, 8) and group in (64, 128)
        return bits, group, 0
    raise ValueError(f"layout {layout}")


def row_stride(layout, N, bits=None, group=None, keep=None):
    """Bytes per row of a fixed-stride layout (cobalt_format.h:59-68 for ids 1,2,6,7)."""
    bits, group, keep = canon(layout, bits, group, keep)
    if layout in DENSE_FAMILY:
        return _align((N * bits + 7) // 8, 16)
    if layout == BLK1632_6:
        return N // 2
    if layout in (BLK1632_4, BLKC):
        return N // 8 + _align(((N // BLOCK) * keep * bits + 7) // 8, 16)
    raise ValueError("variable-length layout has no fixed stride")


# ----------------------------------------------------------------------------- bit helpers
def unpack_bits(mask_bytes, N):
    """uint8 [K, N/8], LSB-first -> bool [K, N]."""
    mask_bytes = np.asarray(mask_bytes, np.uint8)
    return np.unpackbits(mask_bytes, axis=-1, bitorder="little")[..., :N].astype(bool)


def pack_bits(keep):
    """bool [K, N] -> uint8 [K, N/8], LSB-first (bit j%8 of byte j//8 is column j)."""
    return np.packbits(np.asarray(keep, bool), axis=-1, bitorder="little")


def _pack_stream(codes, bits):
    """int [K, n] -> uint8 [K, ceil(n*bits/8)], code i at bits [i*bits, (i+1)*bits), LSB first."""
    codes = np.asarray(codes, np.uint8)
    K, n = codes.shape
    b = ((codes[:, :, None] >> np.arange(bits, dtype=np.uint8)) & 1).reshape(K, n * bits)
    return np.packbits(b, axis=1, bitorder="little")


def _unpack_stream(bytes_, n, bits):
    """Inverse of _pack_stream: uint8 [K, >=ceil(n*bits/8)] -> int32 [K, n]."""
    K = bytes_.shape[0]
    b = np.unpackbits(bytes_, axis=1, bitorder="little")[:, : n * bits].reshape(K, n, bits)
    return (b.astype(np.int32) << np.arange(bits, dtype=np.int32)).sum(-1)


# ----------------------------------------------------------------------------- zero repair
def _to_int_zero(zero):
    """RAW `zero` may be fp16 (a rounded integer) or uint8 (pack_cobalt.py:46-52)."""
    zero = np.asarray(zero)
    if zero.dtype == np.uint8:
        return zero.astype(np.int32)
    return np.rint(zero.astype(np.float32)).astype(np.int32)


def fix_zero_range(qf, scale, zero, keep, nlevels, group=GROUP):
    """Guarantee zero in [0, nlevels]; restates pack_cobalt._fix_zero_range (:55-87).

    Groups whose integer zero point falls outside the grid get (scale, zero, q)
    re-derived from a 0-inclusive hull of their dequantised survivors.  All arithmetic is
    float32, in the reference's operation order.  Returns (qf, scale_f32, zero_i32, n_fixed).
    """
    qf = np.asarray(qf, np.float32)
    K, N = qf.shape
    G = N // group
    z = _to_int_zero(zero)
    bad = (z < 0) | (z > nlevels)
    n_bad = int(bad.sum())
    sc = np.asarray(scale).astype(np.float32)
    if n_bad == 0:
        return qf, sc, z, 0
    q3 = qf.reshape(K, G, group)
    v = (q3 - z.reshape(K, G, 1).astype(np.float32)) * sc.reshape(K, G, 1)
    kv = keep.reshape(K, G, group)
    big = np.finfo(np.float32).max
    vmin = np.where(kv, v, np.float32(big)).min(-1)
    vmax = np.where(kv, v, np.float32(-big)).max(-1)
    empty = ~kv.any(-1)
    vmin = np.minimum(np.where(empty, np.float32(0), vmin), np.float32(0))
    vmax = np.maximum(np.where(empty, np.float32(0), vmax), np.float32(0))
    s2 = np.maximum((vmax - vmin) / np.float32(nlevels), np.float32(1e-12)).astype(np.float32)
    z2 = np.clip(np.rint(-vmin / s2), 0, nlevels).astype(np.float32)
    q2 = np.clip(np.rint(v / s2[..., None] + z2[..., None]), 0, nlevels).astype(np.float32)
    b3 = np.broadcast_to(bad[..., None], q3.shape)
    qf = np.where(b3, q2, q3).reshape(K, N)
    sc = np.where(bad, s2, sc)
    z = np.where(bad, z2.astype(np.int32), z)
    return qf, sc, z, n_bad


# ----------------------------------------------------------------------------- packer
def pack_matrix(mask_bits, q, scale, zero, layout, bits=None, group=None, keep_per_block=None,
                fix_zero=True, return_ref=False):
    """RAW (mask, q, scale, zero) -> packed arrays; restates pack_cobalt.pack_matrix (:98-250).

    mask_bits uint8 [K, N/8] or None (unmasked); q [K, N] codes; scale/zero [K, N/group].
    Returns dict(data u8 (+64 B tail), row_off u32 [K+1] or None, scale fp16 [K,G],
    zero u8 [K,G], n_survivors, n_zero_fixed, W_ref (fp32, before col_scale) if asked).
    """
    bits, group, kpb = canon(layout, bits, group, keep_per_block)
    q = np.asarray(q)
    K, N = q.shape
    assert N % group == 0 and N % 128 == 0
    G = N // group
    nlevels = (1 << bits) - 1
    qf = q.astype(np.float32)
    if mask_bits is None:
        keep = np.ones((K, N), bool)
        mask_bits = np.full((K, N // 8), 255, np.uint8)
    else:
        mask_bits = np.ascontiguousarray(mask_bits, np.uint8).reshape(K, N // 8)
        keep = unpack_bits(mask_bits, N)
    if fix_zero:
        qf, sc, zi, n_fixed = fix_zero_range(qf, scale, zero, keep, nlevels, group)
    else:
        sc, zi, n_fixed = np.asarray(scale).astype(np.float32), _to_int_zero(zero), 0
    qc = np.clip(qf, 0, nlevels).astype(np.int32)
    zrep = np.repeat(zi, group, axis=1)
    if layout in DENSE_FAMILY:
        qc = np.where(keep, qc, zrep)          # pruned positions must dequantise to 0
    out_scale = sc.astype(np.float16)
    out_zero = zi.astype(np.uint8)
    res = dict(row_off=None, scale=out_scale, zero=out_zero, n_survivors=int(keep.sum()),
               n_zero_fixed=n_fixed, W_ref=None)
    if return_ref:
        ref = (qc.astype(np.float32) - zrep.astype(np.float32)) * \
            np.repeat(out_scale.astype(np.float32), group, axis=1)
        if layout not in DENSE_FAMILY:
            ref = ref * keep.astype(np.float32)
        res["W_ref"] = ref
    tail = np.zeros(BLOB_TAIL, np.uint8)

    if layout in DENSE_FAMILY:
        stride = row_stride(layout, N, bits, group)
        rows = np.zeros((K, stride), np.uint8)
        s = _pack_stream(qc & 0xFF, bits)
        rows[:, : s.shape[1]] = s
        res["data"] = np.concatenate([rows.reshape(-1), tail])
        return res

    if layout in BLK_FAMILY:
        NB = N // BLOCK
        cnt = keep.reshape(K, NB, BLOCK).sum(-1)
        if not (cnt == kpb).all():
            r, c = np.argwhere(cnt != kpb)[0]
            raise ValueError(f"{LAYOUT_NAME[layout]} needs exactly {kpb} survivors in every aligned "
                             f"block of {BLOCK} columns; row {r} block {c} has {cnt[r, c]}")
        cod = qc[keep].reshape(K, NB * kpb)            # survivors in column order
        stride = row_stride(layout, N, bits, group, kpb)
        rows = np.zeros((K, stride), np.uint8)
        rows[:, : N // 8] = mask_bits
        if layout == BLK1632_6:
            c3 = cod.reshape(K, NB, 16)
            nib = ((c3[:, :, 0::2] & 0xF) | ((c3[:, :, 1::2] & 0xF) << 4)).astype(np.uint8)
            rows[:, N // 8: N // 8 + NB * 8] = nib.reshape(K, NB * 8)
            sh = (np.arange(8, dtype=np.int64) * 2)
            he = ((((c3[:, :, 0::2] >> 4) & 3).astype(np.int64)) << sh).sum(-1)
            ho = ((((c3[:, :, 1::2] >> 4) & 3).astype(np.int64)) << (sh + 16)).sum(-1)
            hw = (he | ho).astype(np.uint32)
            rows[:, N * 3 // 8:] = hw.reshape(K, NB).astype("<u4").view(np.uint8).reshape(K, NB * 4)
        else:
            s = _pack_stream(cod, bits)
            rows[:, N // 8: N // 8 + s.shape[1]] = s
        res["data"] = np.concatenate([rows.reshape(-1), tail])
        return res

    # ---------------- SPARSE4 / SPARSE4X / SPARSE4E (pack_cobalt.py:201-250)
    has_goff = layout in (SPARSE4X, SPARSE4E)
    hdr = N // 8 + (_align(G * 2, 16) if has_goff else 0)
    hdr_a = _align(hdr, ROW_ALIGN)
    cnt = keep.reshape(K, G, group).sum(-1).astype(np.int64)
    gbytes = (cnt + 1) // 2                                  # each group padded to an even nibble count
    gcum = np.cumsum(gbytes, axis=1) - gbytes
    row_bytes = _align_arr(hdr_a + gbytes.sum(1), ROW_ALIGN)
    row_off = np.zeros(K + 1, np.int64)
    row_off[1:] = np.cumsum(row_bytes)
    total = int(row_off[K])
    assert total < 2 ** 32
    data = np.zeros(total + BLOB_TAIL, np.uint8)
    for k in range(K):
        rb = int(row_off[k])
        data[rb: rb + N // 8] = mask_bits[k]
        if has_goff:
            data[rb + N // 8: rb + N // 8 + 2 * G] = gcum[k].astype("<u2").view(np.uint8)
        for g in range(G):
            cg = qc[k, g * group:(g + 1) * group][keep[k, g * group:(g + 1) * group]]
            if cg.size % 2:
                cg = np.concatenate([cg, [0]])
            by = (cg[0::2] | (cg[1::2] << 4)).astype(np.uint8)
            o = rb + hdr_a + int(gcum[k, g])
            data[o: o + by.size] = by
    res["data"] = data
    res["row_off"] = row_off.astype(np.uint32)
    return res


def _align_arr(x, a):
    return (x + a - 1) // a * a


# ----------------------------------------------------------------------------- unpack / dequant
def unpack_codes(packed, K, N, layout, bits=None, group=None, keep_per_block=None):
    """Packed bytes -> (q int32 [K,N] with 0 at pruned positions, keep bool [K,N]).

    Vectorised reader; restates dequant_ref.dequant_matrix (:43-68) and
    pack_cobalt.dequant_reference (:277-331)."""
    bits, group, kpb = canon(layout, bits, group, keep_per_block)
    data = np.asarray(packed["data"], np.uint8)
    if layout in DENSE_FAMILY:
        stride = row_stride(layout, N, bits, group)
        rows = data[: K * stride].reshape(K, stride)
        return _unpack_stream(rows, N, bits), np.ones((K, N), bool)
    if layout in BLK_FAMILY:
        stride = row_stride(layout, N, bits, group, kpb)
        rows = data[: K * stride].reshape(K, stride)
        keep = unpack_bits(rows[:, : N // 8], N)
        NB = N // BLOCK
        if layout == BLK1632_6:
            nib = rows[:, N // 8: N // 8 + NB * 8].reshape(K, NB, 8).astype(np.int32)
            q16 = np.stack([nib & 0xF, nib >> 4], -1).reshape(K, NB, 16)
            hw = rows[:, N * 3 // 8: N // 2].copy().view("<u4").reshape(K, NB).astype(np.int64)
            sh = np.arange(8, dtype=np.int64) * 2
            he = (hw[..., None] >> sh) & 3
            ho = (hw[..., None] >> (sh + 16)) & 3
            q16 = q16 | (np.stack([he, ho], -1).reshape(K, NB, 16).astype(np.int32) << 4)
            cod = q16.reshape(K, NB * 16)
        else:
            cod = _unpack_stream(rows[:, N // 8:], NB * kpb, bits)
        q = np.zeros((K, N), np.int32)
        q[keep] = cod.reshape(-1)
        return q, keep
    # sparse family
    G = N // group
    has_goff = layout in (SPARSE4X, SPARSE4E)
    hdr_a = _align(N // 8 + (_align(G * 2, 16) if has_goff else 0), ROW_ALIGN)
    ro = np.asarray(packed["row_off"]).astype(np.int64)
    q = np.zeros((K, N), np.int32)
    keep = np.zeros((K, N), bool)
    for k in range(K):
        rb = int(ro[k])
        kp = unpack_bits(data[rb: rb + N // 8][None], N)[0]
        keep[k] = kp
        cnt = kp.reshape(G, group).sum(1)
        gb = (cnt + 1) // 2
        gcum = np.cumsum(gb) - gb
        if has_goff:
            stored = data[rb + N // 8: rb + N // 8 + 2 * G].copy().view("<u2").astype(np.int64)
            assert (stored == gcum).all(), "goff table disagrees with the bitmap"
        for g in range(G):
            c = int(cnt[g])
            by = data[rb + hdr_a + int(gcum[g]): rb + hdr_a + int(gcum[g]) + (c + 1) // 2].astype(np.int32)
            nib = np.stack([by & 0xF, by >> 4], -1).reshape(-1)[:c]
            cols = np.nonzero(kp[g * group:(g + 1) * group])[0] + g * group
            q[k, cols] = nib
    return q, keep


def col_scale_rows(K, cs_rows, cs_splits=None):
    """Which col_scale row each weight row uses (cobalt_format.h:77-99).

    cs_rows 1: one vector; 2: fused gate/up, row parity; 3: fused q|k|v, row ranges
    [0,Kq), [Kq,Kq+Kk), rest, with cs_splits = (Kq, Kk)."""
    r = np.arange(K)
    if cs_rows <= 1:
        return np.zeros(K, np.int64)
    if cs_rows == 2:
        return r & 1
    if cs_rows == 3:
        kq, kk = cs_splits
        return np.where(r < kq, 0, np.where(r < kq + kk, 1, 2))
    raise ValueError(cs_rows)


def dequant(packed, K, N, layout, col_scale=None, bits=None, group=None, keep_per_block=None,
            cs_splits=None):
    """Packed bytes -> W_hat fp32 [K, N].

    W_hat = ((q - zero) * scale) * keep * col_scale, every step in float32, in the order of
    dequant_ref.dequant_matrix (:69-82).  (q - zero) * scale is exact in float32 (at most
    8 + 11 significant bits), so the result carries exactly one rounding (the col_scale
    product) and is independent of association order."""
    bits, group, kpb = canon(layout, bits, group, keep_per_block)
    G = N // group
    q, keep = unpack_codes(packed, K, N, layout, bits, group, kpb)
    s = np.asarray(packed["scale"]).reshape(K, G).astype(np.float32)
    z = np.asarray(packed["zero"]).reshape(K, G).astype(np.float32)
    w = (q.reshape(K, G, group).astype(np.float32) - z[:, :, None]) * s[:, :, None]
    w = w.reshape(K, N)
    if layout not in DENSE_FAMILY:
        w = w * keep.astype(np.float32)
    if col_scale is not None:
        cs = np.asarray(col_scale).astype(np.float32).reshape(-1, N)
        w = w * cs[col_scale_rows(K, cs.shape[0], cs_splits)]
    return w


def dequant_scalar(packed, K, N, layout, col_scale=None, bits=None, group=None,
                   keep_per_block=None, cs_splits=None):
    """Independent per-position decoder written from the format text alone
    (docs/FORMAT.md:83-107 and the layout notes at the top of this file).  Slow; used only
    to cross-check `dequant` on small matrices."""
    bits, group, kpb = canon(layout, bits, group, keep_per_block)
    data = np.asarray(packed["data"], np.uint8)
    G = N // group
    sc = np.asarray(packed["scale"]).reshape(K, G)
    zr = np.asarray(packed["zero"]).reshape(K, G)
    cs = None if col_scale is None else np.asarray(col_scale).reshape(-1, N)
    csr = col_scale_rows(K, 1 if cs is None else cs.shape[0], cs_splits)
    W = np.zeros((K, N), np.float32)

    def getbits(base, bitpos, nb):
        v = 0
        for i in range(nb):
            p = bitpos + i
            v |= ((int(data[base + (p >> 3)]) >> (p & 7)) & 1) << i
        return v

    for k in range(K):
        if layout in SPARSE_FAMILY:
            rb = int(packed["row_off"][k])
            has_goff = layout != SPARSE4
            hdr_a = _align(N // 8 + (_align(G * 2, 16) if has_goff else 0), 16)
            nibpos = 0
        else:
            rb = k * row_stride(layout, N, bits, group, kpb)
        rank = 0
        for j in range(N):
            g = j // group
            if layout in DENSE_FAMILY:
                kept, code = True, getbits(rb, j * bits, bits)
            else:
                kept = (int(data[rb + (j >> 3)]) >> (j & 7)) & 1
                code = 0
                if layout in SPARSE_FAMILY:
                    if j % group == 0 and nibpos % 2:
                        nibpos += 1                # every group starts on a byte boundary
                    if kept:
                        b = int(data[rb + hdr_a + (nibpos >> 1)])
                        code = (b >> 4) if (nibpos & 1) else (b & 0xF)
                        nibpos += 1
                elif kept:
                    if layout == BLK1632_6:
                        t, i = rank // 16, rank % 16
                        b = int(data[rb + N // 8 + 8 * t + (i >> 1)])
                        lo = (b >> 4) if (i & 1) else (b & 0xF)
                        hw = int.from_bytes(bytes(data[rb + 3 * N // 8 + 4 * t: rb + 3 * N // 8 + 4 * t + 4]), "little")
                        hi = (hw >> (2 * (i >> 1) + (16 if (i & 1) else 0))) & 3
                        code = lo | (hi << 4)
                    else:
                        code = getbits(rb + N // 8, rank * bits, bits)
                    rank += 1
            if kept:
                v = np.float32(np.float32(code) - np.float32(zr[k, g])) * np.float32(sc[k, g])
                if cs is not None:
                    v = np.float32(v) * np.float32(cs[csr[k], j])
                W[k, j] = v
    return W


def forward_ref(W_hat, x, bias=None, accumulate=np.float64):
    """y = x @ W_hat.T (+ bias): the dequantise-then-matmul forward of
    benchmark_suite.SparseQuantLinear.forward (:1200-1217) with W_hat kept in float32
    (not rounded to the activation dtype) and a wide accumulator.  x is [M, N] float."""
    y = np.asarray(x, accumulate) @ np.asarray(W_hat, accumulate).T
    if bias is not None:
        y = y + np.asarray(bias, accumulate)
    return y


# ----------------------------------------------------------------------------- synthetic RAW
def synth_raw_matrix(K, N, sparsity=0.5, bits=4, seed=0, block=0, group=GROUP, balanced=True):
    """Random RAW-schema matrix, the recipe of pack_cobalt.synth_raw_matrix (:338-371):
    uniform importances, row- then column-quantile normalised, then a global top-k
    (block=0) or a per-aligned-block top-(block - int(block*sparsity)) selection; random
    codes, scales in [1e-3, 1.1e-2), integer zeros on the grid, col_scale in [0.5, 2).
    The random stream is numpy's, not torch's, so values differ from the reference's
    generator; only the recipe is the same."""
    rng = np.random.default_rng(seed)
    imp = rng.random((K, N), dtype=np.float32)
    if balanced:
        kr = max(1, int(N * sparsity)); kc = max(1, int(K * sparsity))
        imp = imp / np.maximum(np.partition(imp, kr - 1, axis=1)[:, kr - 1: kr], 1e-30)
        imp = imp / np.maximum(np.partition(imp, kc - 1, axis=0)[kc - 1: kc, :], 1e-30) ** 0.5
    if block:
        nk = block - int(block * sparsity)
        ib = imp.reshape(K, N // block, block)
        idx = np.argsort(-ib, axis=-1, kind="stable")[..., :nk]
        keep = np.zeros(ib.shape, bool)
        np.put_along_axis(keep, idx, True, axis=-1)
        keep = keep.reshape(K, N)
    else:
        npr = max(1, int(K * N * sparsity))
        thr = np.partition(imp.reshape(-1), npr - 1)[npr - 1]
        keep = imp > thr
    G = N // group
    nl = (1 << bits) - 1
    q = rng.integers(0, nl + 1, (K, N), dtype=np.uint8) * keep.astype(np.uint8)
    scale = (rng.random((K, G), dtype=np.float32) * 0.01 + 0.001).astype(np.float16)
    zero = rng.integers(0, nl + 1, (K, G)).astype(np.float16)
    col_scale = (rng.random(N, dtype=np.float32) * 1.5 + 0.5).astype(np.float16)
    return dict(mask=pack_bits(keep), q=q, scale=scale, zero=zero, col_scale=col_scale)


def rtn_dense(W, bits, group=GROUP):
    """Plain asymmetric group min-max RTN with a 0-inclusive hull (pack_cobalt.py:375-386)."""
    W = np.asarray(W, np.float32)
    K, N = W.shape
    G = N // group
    nl = np.float32((1 << bits) - 1)
    Wg = W.reshape(K, G, group)
    wmin = np.minimum(Wg.min(-1), np.float32(0))
    wmax = np.maximum(Wg.max(-1), np.float32(0))
    scale = np.maximum((wmax - wmin) / nl, np.float32(1e-12))
    zero = np.clip(np.rint(-wmin / scale), 0, nl)
    q = np.clip(np.rint(Wg / scale[..., None] + zero[..., None]), 0, nl).reshape(K, N)
    return q, scale.astype(np.float16), zero.astype(np.uint8)


# ----------------------------------------------------------------------------- sizes
def stream_bytes(packed):
    """Weight bytes a GEMV over this matrix streams (pack_cobalt.py:431-433)."""
    return int(packed["data"].size - BLOB_TAIL + packed["scale"].size * 2 + packed["zero"].size)


def bpw(packed, K, N):
    ro = 0 if packed.get("row_off") is None else packed["row_off"].size * 4
    return 8.0 * (stream_bytes(packed) + ro) / (K * N)


def bpw_formula(layout, bits=None, group=None, keep_per_block=None, density=None):
    """Closed-form bits per weight (docs/FORMAT.md:78-81): codes + mask + (16+8)/group."""
    bits, group, kpb = canon(layout, bits, group, keep_per_block)
    meta = 24.0 / group
    if layout in DENSE_FAMILY:
        return bits + meta
    if layout in BLK_FAMILY:
        return 1.0 + bits * kpb / 32.0 + meta
    return 1.0 + bits * density + meta


def make_blob(packed, col_scale=None):
    """Concatenate {data,row_off,scale,zero,col_scale} into one 256-B aligned image
    (test_gemv.make_blob :57-80; array alignment of pack_cobalt.BlobWriter :390-411).
    Returns (uint8 array, {name: byte offset})."""
    parts, offs, pos = [], {}, 0

    def add(name, arr):
        nonlocal pos
        pad = _align(pos, ARR_ALIGN) - pos
        if pad:
            parts.append(np.zeros(pad, np.uint8)); pos += pad
        offs[name] = pos
        b = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        parts.append(b); pos += b.size

    add("data", packed["data"])
    if packed.get("row_off") is not None:
        add("row_off", packed["row_off"])
    add("scale", packed["scale"])
    add("zero", packed["zero"])
    if col_scale is not None:
        add("col_scale", np.asarray(col_scale, np.float16))
    pad = _align(pos, ARR_ALIGN) - pos
    if pad:
        parts.append(np.zeros(pad, np.uint8))
    return np.concatenate(parts), offs


# ----------------------------------------------------------------------------- tile-interleaved device order
TILE_ROWS = 16
TILE_UNIT = 16
TILED_TAIL = 512


def tile16(packed, K, N, layout, bits=None, group=None, keep_per_block=None):
    """Row-major fixed-stride arrays -> the 16-row tile-interleaved order the MI355X kernels
    stream.  This is a permutation of the same bytes (plus zero rows up to a multiple of 16)
    and has no counterpart in the reference, whose kernels read row-major rows: byte o of row
    k moves to  (k//16)*16*stride + ((o//16)*16 + k%16)*16 + o%16 ; scale/zero entry (k, g)
    moves to index ((k//16)*G + g)*16 + k%16.  The data array ends with 512 zero bytes."""
    bits, group, kpb = canon(layout, bits, group, keep_per_block)
    stride = row_stride(layout, N, bits, group, kpb)
    G = N // group
    K16 = (K + 15) // 16
    rows = np.zeros((K16 * 16, stride), np.uint8)
    rows[:K] = np.asarray(packed["data"], np.uint8)[: K * stride].reshape(K, stride)
    data = rows.reshape(K16, 16, stride // 16, 16).transpose(0, 2, 1, 3).reshape(-1)
    sc = np.zeros((K16 * 16, G), np.float16); sc[:K] = np.asarray(packed["scale"]).reshape(K, G)
    zr = np.zeros((K16 * 16, G), np.uint8); zr[:K] = np.asarray(packed["zero"]).reshape(K, G)
    out = dict(packed)
    out["data"] = np.concatenate([data, np.zeros(TILED_TAIL, np.uint8)])
    out["scale"] = sc.reshape(K16, 16, G).transpose(0, 2, 1).reshape(-1).copy()
    out["zero"] = zr.reshape(K16, 16, G).transpose(0, 2, 1).reshape(-1).copy()
    return out


def untile16(tiled, K, N, layout, bits=None, group=None, keep_per_block=None):
    """Inverse of tile16 (drops the padding rows; restores the 64-byte tail)."""
    bits, group, kpb = canon(layout, bits, group, keep_per_block)
    stride = row_stride(layout, N, bits, group, kpb)
    G = N // group
    K16 = (K + 15) // 16
    d = np.asarray(tiled["data"], np.uint8)[: K16 * 16 * stride]
    rows = d.reshape(K16, stride // 16, 16, 16).transpose(0, 2, 1, 3).reshape(K16 * 16, stride)[:K]
    out = dict(tiled)
    out["data"] = np.concatenate([rows.reshape(-1), np.zeros(BLOB_TAIL, np.uint8)])
    out["scale"] = np.asarray(tiled["scale"]).reshape(K16, G, 16).transpose(0, 2, 1).reshape(K16 * 16, G)[:K].copy()
    out["zero"] = np.asarray(tiled["zero"]).reshape(K16, G, 16).transpose(0, 2, 1).reshape(K16 * 16, G)[:K].copy()
    return out
