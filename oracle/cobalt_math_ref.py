"""CPU oracle for the CoBALT compressor that PRODUCES the bytes the hot path reads.
TEST INFRASTRUCTURE ONLY (same rule as cbk_ref.py: never imported by the product).

numpy/float32 restatement of src/cobaltkernel/cobalt_math.py in the reference:

  balanced_keepmask   cobalt_math.py:15-32    (row quantile, column^beta quantile, global top-k)
  blocked_keepmask    cobalt_math.py:35-63    (same normalisation, per-32-block top-keep)
  _rescale            cobalt_math.py:66-76
  obs_compensate      cobalt_math.py:105-124
  masked_std          cobalt_math.py:128-134
  robust_scale        cobalt_math.py:137-140
  group_rtn           cobalt_math.py:144-168  (== sinq/dual_shift.py:133-139 for hull='all')
  dequant             cobalt_math.py:328-332
  cobalt_quantize     cobalt_math.py:336-371  (quant_mode='rtn', clip='none': the shipped path)

Parity status.  Mask cardinalities, the RTN error bound, the OBS closed form (against a
float64 per-row solve) and dequant are pinned by tests/test_oracle_math.py; the whole recipe is
pinned against four seeded runs of the reference's own cobalt_quantize
(tests/golden/cobalt_quantize.npz, tests/test_golden_cobalt_quantize.py): keep-masks, codes and
zero points identical, scales and column scales equal to 2e-4 (float32 chains of LAPACK here
and torch there; at most 3 % of them one fp16 step apart once stored).  What stays "parity
unpinned": the order in which torch.topk / torch.kthvalue break EXACT ties, which those
continuous inputs do not contain.  It only chooses which valid RAW matrix gets produced.
"""
from __future__ import annotations

import numpy as np
import scipy.linalg

f32 = np.float32


def _kth(a, k, axis):
    """k-th smallest (1-indexed) along axis, keepdims (torch.kthvalue semantics)."""
    p = np.partition(a, k - 1, axis=axis)
    return np.take(p, [k - 1], axis=axis)


def _rescale(imp):
    m = imp.max()
    if np.isfinite(m) and m > 0:
        return imp / m
    return np.nan_to_num(imp, nan=0.0, posinf=0.0, neginf=0.0)


def _normalise(imp, sparsity, col_exp):
    K, N = imp.shape
    kr, kc = int(N * sparsity), int(K * sparsity)
    if kr > 0:
        imp = _rescale(imp / np.maximum(_kth(imp, kr, 1), f32(1e-30)))
    if col_exp > 0 and kc > 0:
        imp = _rescale(imp / np.maximum(_kth(imp, kc, 0), f32(1e-30)) ** f32(col_exp))
    return imp.astype(f32)


def balanced_keepmask(imp, sparsity, col_exp):
    imp = np.asarray(imp, f32)
    K, N = imp.shape
    if sparsity <= 0.0:
        return np.ones_like(imp)
    imp = _normalise(imp, sparsity, col_exp)
    n_prune = int(K * N * sparsity)
    flat = imp.reshape(-1)
    thr = np.partition(flat, n_prune - 1)[n_prune - 1]
    return (flat > thr).reshape(K, N).astype(f32)


def blocked_keepmask(imp, sparsity, col_exp, block=32):
    imp = np.asarray(imp, f32)
    K, N = imp.shape
    if sparsity <= 0.0:
        return np.ones_like(imp)
    assert N % block == 0
    imp = _normalise(imp, sparsity, col_exp)
    keep = block - int(block * sparsity)
    v = imp.reshape(K, N // block, block)
    idx = np.argsort(-v, axis=-1, kind="stable")[..., :keep]
    mask = np.zeros(v.shape, f32)
    np.put_along_axis(mask, idx, f32(1), axis=-1)
    return mask.reshape(K, N)


def obs_compensate(W, mask, H, damping_frac=0.01, damping_min=1e-2):
    """W_comp = (W - ((W*(1-mask)) / diag(Hinv)) @ Hinv) * mask."""
    W = np.asarray(W, f32); mask = np.asarray(mask, f32); H = np.asarray(H, f32)
    damping = max(damping_frac * float(np.diagonal(H).mean()), damping_min)
    Hd = H.copy()
    Hd[np.diag_indices_from(Hd)] += f32(damping)
    c, low = scipy.linalg.cho_factor(Hd, lower=True)
    Hinv = scipy.linalg.cho_solve((c, low), np.eye(H.shape[0], dtype=f32)).astype(f32)
    d = np.maximum(np.diagonal(Hinv), f32(1e-12))
    P = W * (f32(1) - mask)
    return ((W - (P / d[None, :]) @ Hinv) * mask).astype(f32), damping


def masked_std(W, mask, axis, eps=1e-8):
    cnt = np.maximum(mask.sum(axis=axis), f32(1))
    mean = (W * mask).sum(axis=axis) / cnt
    centered = (W - (mean[None, :] if axis == 0 else mean[:, None])) * mask
    var = (centered ** 2).sum(axis=axis) / cnt
    return np.maximum(np.sqrt(var), f32(eps)).astype(f32)


def robust_scale(s, ratio=10.0):
    s = np.maximum(np.nan_to_num(s, nan=1.0, posinf=1.0, neginf=1.0), f32(1e-8)).astype(f32)
    gm = np.exp(np.log(s).mean())
    return np.clip(s / gm, f32(1.0 / ratio), f32(ratio)).astype(f32)


def group_rtn(W_norm, mask, nbits, gsize, hull="survivor"):
    """Asymmetric unsigned min-max group RTN along axis 1 -> (q, scale, zero), float32."""
    W_norm = np.asarray(W_norm, f32)
    K, N = W_norm.shape
    assert N % gsize == 0
    ng = N // gsize
    Wg = W_norm.reshape(K, ng, gsize)
    nl = f32(2 ** nbits - 1)
    if hull == "survivor":
        Mg = np.asarray(mask).reshape(K, ng, gsize) != 0
        big = np.finfo(f32).max
        w_min = np.where(Mg, Wg, f32(big)).min(-1, keepdims=True)
        w_max = np.where(Mg, Wg, f32(-big)).max(-1, keepdims=True)
        empty = ~Mg.any(-1, keepdims=True)
        w_min = np.where(empty, f32(0), w_min)
        w_max = np.where(empty, f32(0), w_max)
    else:
        w_min = Wg.min(-1, keepdims=True)
        w_max = Wg.max(-1, keepdims=True)
    scale = (np.maximum(w_max - w_min, f32(1e-4)) / nl).astype(f32)
    zero = -np.rint(w_min / scale)
    q = np.clip(np.rint(Wg / scale + zero), 0, nl)
    return q.reshape(K, N).astype(f32), scale.reshape(K, ng), zero.reshape(K, ng).astype(f32)


def dequant(q, scale, zero, col_scale, mask, gsize):
    K, N = q.shape
    ng = N // gsize
    W = (q.reshape(K, ng, gsize).astype(f32) - zero.reshape(K, ng, 1).astype(f32)) * \
        scale.reshape(K, ng, 1).astype(f32)
    return W.reshape(K, N) * np.asarray(col_scale, f32).reshape(1, -1) * np.asarray(mask, f32)


def cobalt_quantize(W, H, sparsity, beta, nbits, gsize, hull="survivor", mask_block=0,
                    damping_frac=0.01, damping_min=1e-2):
    """Wanda importance -> keep-mask -> OBS -> per-column scale -> group RTN.
    Returns (q, scale, zero, col_scale, mask, W_hat), all float32."""
    W = np.asarray(W, f32); H = np.asarray(H, f32)
    act_norms = np.sqrt(np.maximum(np.diagonal(H), 0))
    imp = np.abs(W) * act_norms[None, :]
    if mask_block and mask_block > 0:
        mask = blocked_keepmask(imp, sparsity, beta, mask_block)
    else:
        mask = balanced_keepmask(imp, sparsity, beta)
    W_comp, _ = obs_compensate(W, mask, H, damping_frac, damping_min)
    c = robust_scale(masked_std(W_comp, mask, 0))
    W_norm = W_comp / c[None, :]
    if float(mask.sum()) == 0.0 and sparsity < 1.0:
        raise RuntimeError("degenerate all-zero keep-mask")
    q, scale, zero = group_rtn(W_norm, mask, nbits, gsize, hull)
    W_hat = dequant(q, scale, zero, c, mask, gsize)
    return q, scale, zero, c, mask, W_hat


def to_raw(q, scale, zero, col_scale, mask):
    """The RAW per-matrix schema of quantize_cobalt.py:325-329 / pack_cobalt.py:3-11:
    mask u8 [K,N/8] LSB-first, q u8 [K,N] (0 at pruned), scale fp16, zero fp16, col_scale fp16."""
    keep = np.asarray(mask) != 0
    return dict(mask=np.packbits(keep, axis=-1, bitorder="little"),
                q=(np.asarray(q) * keep).astype(np.uint8),
                scale=np.asarray(scale).astype(np.float16),
                zero=np.asarray(zero).astype(np.float16),
                col_scale=np.asarray(col_scale).astype(np.float16))
