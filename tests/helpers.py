"""Shared helpers for the parity tests: oracle-side RAW matrices handed to the product packer."""
import numpy as np
import torch

from oracle import cbk_ref as R
from cobalt_amd import format as F

# (layout, bits, group, keep) of every fixed-stride case the kernels take
FIXED_CASES = [
    (F.DENSE4, 4, 128, 0), (F.DENSE8, 8, 128, 0), (F.BLK1632_4, 4, 128, 16), (F.BLK1632_6, 6, 128, 16),
    (F.BLKC, 4, 128, 16), (F.BLKC, 3, 128, 10), (F.BLKC, 2, 128, 16), (F.BLKC, 4, 64, 23),
    (F.BLKC, 3, 64, 23), (F.BLKC, 2, 64, 10), (F.BLKC, 4, 64, 10), (F.BLKC, 3, 64, 16), (F.BLKC, 2, 64, 23),
    (F.DENSEB, 3, 128, 0), (F.DENSEB, 2, 64, 0), (F.DENSEB, 4, 64, 0),
]
SPARSE_CASES = [(F.SPARSE4, 4, 128, 0), (F.SPARSE4X, 4, 128, 0), (F.SPARSE4E, 4, 128, 0)]


def case_id(c):
    return f"{F.LAYOUT_NAME[c[0]]}-b{c[1]}-g{c[2]}-k{c[3]}"


def kw_of(case):
    layout, bits, group, keep = case
    if layout in (F.BLKC,):
        return dict(bits=bits, group=group, keep_per_block=keep)
    if layout == F.DENSEB:
        return dict(bits=bits, group=group)
    return {}


def make_raw(case, K, N, seed):
    layout, bits, group, keep = case
    if keep:
        return R.synth_raw_matrix(K, N, sparsity=1.0 - keep / 32.0, bits=bits, seed=seed, block=32, group=group)
    return R.synth_raw_matrix(K, N, sparsity=0.5, bits=bits, seed=seed, group=group)


def oracle_pack(case, raw, **extra):
    return R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], case[0], **kw_of(case), **extra)


def product_pack(case, raw, device="cpu", col_scale="raw", **extra):
    layout, bits, group, keep = case
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    cs = raw["col_scale"] if isinstance(col_scale, str) else col_scale
    return F.pack_raw(t(raw["mask"]), t(raw["q"]), t(raw["scale"]), t(raw["zero"]),
                      None if cs is None else t(cs), layout, bits, group, keep or None, **extra)


def packed_from_oracle(case, pk, col_scale, K, N, device, cs_splits=(0, 0), tiled=False):
    """Oracle-packed arrays (including the variable-length layouts) -> product PackedMatrix,
    optionally re-ordered into the 16-row tile-interleaved device order."""
    layout, bits, group, keep = case
    pm = _from_oracle(case, pk, col_scale, K, N, device, cs_splits)
    return pm.to_tiled() if tiled else pm


def _from_oracle(case, pk, col_scale, K, N, device, cs_splits):
    layout, bits, group, keep = case
    return F.from_arrays(torch.from_numpy(pk["data"]), torch.from_numpy(pk["scale"].view(np.uint8)),
                         torch.from_numpy(pk["zero"]),
                         None if col_scale is None else torch.from_numpy(np.asarray(col_scale, np.float16)),
                         K, N, layout, bits, group, keep or None,
                         row_off=None if pk.get("row_off") is None else torch.from_numpy(pk["row_off"].view(np.uint8)),
                         cs_splits=cs_splits, device=device)


def rel_fro(y, ref):
    y = np.asarray(y, np.float64); ref = np.asarray(ref, np.float64)
    return float(np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30))


def acts(M, N, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(M, N, generator=g) * scale).to(dtype)
