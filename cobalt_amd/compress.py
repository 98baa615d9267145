"""CoBALT compression of one weight matrix into the RAW schema the packer reads, in torch
(runs on whatever device the weight is on; on the GPU it is a handful of dense torch kernels).

Pipeline (reference: src/cobaltkernel/cobalt_math.py:336-371 `cobalt_quantize`, quant mode
'rtn', no clipping; driver loop src/cobaltkernel/quantize_cobalt.py:424-443):

  Wanda importance |W| * sqrt(diag H)                       cobalt_math.py:341-342
  -> row- and column-quantile balancing, exponent beta      cobalt_math.py:15-32, 66-76
  -> keep-mask: exactly `keep` survivors per 32-column block (the layouts the kernels read),
     or one global top-k                                      cobalt_math.py:35-63
  -> OBS compensation of the survivors against H            cobalt_math.py:105-124
  -> per-column scale = clipped masked std / geometric mean cobalt_math.py:128-140
  -> asymmetric min-max group RTN on the survivor hull      cobalt_math.py:144-168

H = X^T X of the calibration activations ([N, N], float32).  All arithmetic is float32.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from . import format as F


def _rescale(imp: torch.Tensor) -> torch.Tensor:
    m = imp.max()
    if torch.isfinite(m) and m > 0:
        return imp / m
    return torch.nan_to_num(imp, nan=0.0, posinf=0.0, neginf=0.0)


def balance_importance(imp: torch.Tensor, sparsity: float, beta: float) -> torch.Tensor:
    """Divide every row by its `sparsity` quantile, then every column by its quantile to the
    power beta, rescaling to a maximum of 1 after each step (positive scalars: they change no
    ranking, they keep float32 from overflowing)."""
    K, N = imp.shape
    kr, kc = int(N * sparsity), int(K * sparsity)
    if kr > 0:
        imp = _rescale(imp / torch.kthvalue(imp, kr, dim=1, keepdim=True).values.clamp_min(1e-30))
    if beta > 0 and kc > 0:
        imp = _rescale(imp / torch.kthvalue(imp, kc, dim=0, keepdim=True).values.clamp_min(1e-30) ** beta)
    return imp


def keep_mask(imp: torch.Tensor, sparsity: float, beta: float = 0.5, block: int = 32) -> torch.Tensor:
    """Float 0/1 keep-mask.  block > 0: exactly block - int(block * sparsity) survivors in every
    aligned block of `block` columns; block = 0: the int(K * N * sparsity) least important
    entries of the whole matrix are pruned."""
    K, N = imp.shape
    if sparsity <= 0.0:
        return torch.ones_like(imp)
    imp = balance_importance(imp.float(), sparsity, beta)
    if block > 0:
        if N % block:
            raise ValueError(f"N={N} is not a multiple of the mask block {block}")
        keep = block - int(block * sparsity)
        v = imp.reshape(K, N // block, block)
        idx = torch.topk(v, keep, dim=-1, sorted=False).indices
        return torch.zeros_like(v).scatter_(-1, idx, 1.0).reshape(K, N)
    n_prune = int(K * N * sparsity)
    thr = torch.kthvalue(imp.reshape(-1), n_prune).values
    return (imp > thr).float()


def obs_compensate(W: torch.Tensor, mask: torch.Tensor, H: torch.Tensor, damping_frac: float = 0.01,
                   damping_min: float = 1e-2) -> torch.Tensor:
    """Survivors absorb the error of the pruned entries of their row:
    W_comp = (W - ((W * (1 - mask)) / diag(Hinv)) @ Hinv) * mask, Hinv = (H + damping I)^-1."""
    damping = max(damping_frac * float(torch.diagonal(H).mean()), damping_min)
    Hd = H.float().clone()
    Hd.diagonal().add_(damping)
    Hinv = torch.cholesky_inverse(torch.linalg.cholesky(Hd))
    d = torch.diagonal(Hinv).clamp_min(1e-12)
    P = W * (1.0 - mask)
    return (W - (P / d.unsqueeze(0)) @ Hinv) * mask


def column_scale(W: torch.Tensor, mask: torch.Tensor, ratio: float = 10.0) -> torch.Tensor:
    """Per-column standard deviation of the survivors, divided by its geometric mean over the
    columns and clipped to [1/ratio, ratio]."""
    cnt = mask.sum(0).clamp_min(1.0)
    mean = (W * mask).sum(0) / cnt
    var = (((W - mean.unsqueeze(0)) * mask) ** 2).sum(0) / cnt
    s = torch.nan_to_num(var.sqrt().clamp_min(1e-8), nan=1.0, posinf=1.0, neginf=1.0).clamp_min(1e-8)
    gm = torch.exp(torch.log(s).mean())
    return (s / gm).clamp(1.0 / ratio, ratio)


def group_rtn(Wn: torch.Tensor, mask: torch.Tensor, bits: int, group: int,
              survivor_hull: bool = True) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """scale = max(w_max - w_min, 1e-4) / (2^bits - 1), zero = -round(w_min / scale),
    q = clamp(round(w / scale + zero)), min / max over the survivors of the group (or over all
    its entries).  Returns float32 (q [K, N], scale [K, G], zero [K, G])."""
    K, N = Wn.shape
    G = N // group
    Wg = Wn.reshape(K, G, group)
    nl = float(2 ** bits - 1)
    if survivor_hull:
        Mg = mask.reshape(K, G, group) != 0
        big = torch.finfo(torch.float32).max
        w_min = torch.where(Mg, Wg, torch.full_like(Wg, big)).amin(-1, keepdim=True)
        w_max = torch.where(Mg, Wg, torch.full_like(Wg, -big)).amax(-1, keepdim=True)
        empty = ~Mg.any(-1, keepdim=True)
        w_min = torch.where(empty, torch.zeros_like(w_min), w_min)
        w_max = torch.where(empty, torch.zeros_like(w_max), w_max)
    else:
        w_min, w_max = Wg.amin(-1, keepdim=True), Wg.amax(-1, keepdim=True)
    scale = (w_max - w_min).clamp_min(1e-4) / nl
    zero = -torch.round(w_min / scale)
    q = torch.clamp(torch.round(Wg / scale + zero), 0, nl)
    return q.reshape(K, N), scale.reshape(K, G), zero.reshape(K, G)


def cobalt_compress(W: torch.Tensor, H: torch.Tensor, sparsity: float = 0.5, bits: int = 4, group: int = 128,
                    beta: float = 0.5, mask_block: int = 32, survivor_hull: bool = True,
                    damping_frac: float = 0.01, damping_min: float = 1e-2) -> Dict[str, torch.Tensor]:
    """One matrix W [K, N] and its calibration Hessian H [N, N] -> RAW schema
    `{mask u8 [K, N/8], q u8 [K, N], scale f16 [K, G], zero f16 [K, G], col_scale f16 [N]}`
    (src/cobaltkernel/pack_cobalt.py:3-11) plus the float32 `W_hat` it dequantises to."""
    W = W.float()
    H = H.float()
    act = torch.diagonal(H).clamp_min(0).sqrt()
    mask = keep_mask(W.abs() * act.unsqueeze(0), sparsity, beta, mask_block)
    if float(mask.sum()) == 0.0 and sparsity < 1.0:
        raise RuntimeError("degenerate all-zero keep-mask")
    Wc = obs_compensate(W, mask, H, damping_frac, damping_min)
    c = column_scale(Wc, mask)
    q, scale, zero = group_rtn(Wc / c.unsqueeze(0), mask, bits, group, survivor_hull)
    K, N = W.shape
    G = N // group
    W_hat = ((q.reshape(K, G, group) - zero.unsqueeze(-1)) * scale.unsqueeze(-1)).reshape(K, N) * mask * c.unsqueeze(0)
    keep = mask != 0
    return dict(mask=F.pack_mask(keep), q=(q * mask).to(torch.uint8), scale=scale.half(), zero=zero.half(),
                col_scale=c.half(), W_hat=W_hat)


def hessian(X: torch.Tensor) -> torch.Tensor:
    """H = X^T X of calibration activations X [tokens, N], accumulated in float32."""
    X = X.reshape(-1, X.shape[-1]).float()
    return X.T @ X


def layout_for(sparsity: float, bits: int, group: int, mask_block: int) -> Tuple[int, Optional[int]]:
    """The packed layout a compression setting maps to, and its survivors per 32 columns."""
    if sparsity <= 0.0:
        return (F.DENSE4 if (bits, group) == (4, 128) else F.DENSEB), None
    if mask_block != 32:
        if (bits, group) != (4, 128):
            raise ValueError("a global top-k mask has a packed layout only for 4-bit codes and group 128 (SPARSE4E)")
        return F.SPARSE4E, None
    keep = 32 - int(32 * sparsity)
    if (bits, group, keep) == (4, 128, 16):
        return F.BLK1632_4, 16
    if (bits, group, keep) == (6, 128, 16):
        return F.BLK1632_6, 16
    return F.BLKC, keep
