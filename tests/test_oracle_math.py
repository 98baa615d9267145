"""Pins oracle/cobalt_math_ref.py (the compressor that produces the RAW matrices) through
the invariants the reference's own CPU tests state (src/cobaltkernel/test_maskblock.py:25-65,
test_deadcols.py:70-87) and through float64 brute force on small inputs."""
import numpy as np

from oracle import cbk_ref as R
from oracle import cobalt_math_ref as M


def _problem(K=48, N=256, seed=0, outliers=True):
    rng = np.random.default_rng(seed)
    W = rng.normal(0, 0.02, (K, N)).astype(np.float32)
    if outliers:
        W[:, rng.choice(N, max(1, N // 100), replace=False)] *= 10
    X = rng.normal(0, 1, (128, N)).astype(np.float32)
    return W, (X.T @ X).astype(np.float32)


def test_blocked_mask_exact_cardinality():
    W, H = _problem()
    imp = np.abs(W) * np.sqrt(np.diagonal(H))[None]
    for s, want in ((0.3, 23), (0.5, 16), (0.7, 10)):
        m = M.blocked_keepmask(imp, s, 0.5, 32)
        assert (m.reshape(48, 8, 32).sum(-1) == want).all()
        assert abs((1 - m.mean()) - int(32 * s) / 32) < 1e-12


def test_balanced_mask_exact_sparsity_and_bruteforce():
    W, H = _problem(K=12, N=128)
    imp = (np.abs(W) * np.sqrt(np.diagonal(H))[None]).astype(np.float32)
    m = M.balanced_keepmask(imp, 0.5, 0.5)
    assert int((m == 0).sum()) == int(12 * 128 * 0.5)
    # brute force with sorted() as kthvalue
    a = imp.copy()
    kr, kc = 64, 6
    a = a / np.maximum(np.array([sorted(r)[kr - 1] for r in a], np.float32)[:, None], 1e-30)
    a = a / a.max()
    a = a / np.maximum(np.array([sorted(c)[kc - 1] for c in a.T], np.float32)[None, :], 1e-30) ** np.float32(0.5)
    a = (a / a.max()).astype(np.float32)
    thr = sorted(a.reshape(-1))[768 - 1]
    assert np.array_equal(m, (a > thr).astype(np.float32))
    # a positive global rescale never changes the support
    assert np.array_equal(m, M.balanced_keepmask(imp * 37.0, 0.5, 0.5))


def test_obs_matches_float64_per_row_solve():
    W, H = _problem(K=6, N=64)
    rng = np.random.default_rng(3)
    mask = (rng.random(W.shape) > 0.5).astype(np.float32)
    Wc, damp = M.obs_compensate(W, mask, H)
    assert damp == max(0.01 * float(np.diagonal(H).mean()), 1e-2)
    Hd = H.astype(np.float64) + damp * np.eye(64)
    Hinv = np.linalg.inv(Hd)
    want = np.zeros_like(W, dtype=np.float64)
    for r in range(6):                       # the per-row loop form (src/nosink.py:123-126)
        w = W[r].astype(np.float64)
        p = w * (1 - mask[r])
        want[r] = (w - (p / np.diagonal(Hinv)) @ Hinv) * mask[r]
    assert np.abs(Wc - want).max() < 2e-5 * np.abs(want).max() + 1e-7
    assert (Wc[mask == 0] == 0).all()


def test_group_rtn_formula_and_bound():
    rng = np.random.default_rng(2)
    W = rng.normal(0, 1, (8, 256)).astype(np.float32)
    mask = (rng.random(W.shape) > 0.5).astype(np.float32)
    mask[3, :128] = 0                                   # an empty group
    for bits in (2, 3, 4):
        for g in (64, 128):
            q, s, z = M.group_rtn(W * mask, mask, bits, g, "survivor")
            nl = 2 ** bits - 1
            assert q.min() >= 0 and q.max() <= nl
            Wd = M.dequant(q, s, z, np.ones(256, np.float32), mask, g)
            err = np.abs(Wd - W * mask)
            assert (err <= 0.5001 * np.repeat(s, g, 1) + 1e-6)[mask != 0].all()
            # hull endpoints are on the grid
            Wg = np.where(mask.reshape(8, -1, g) != 0, W.reshape(8, -1, g), np.nan)
            lo = np.nan_to_num(np.nanmin(Wg, -1), nan=0.0); hi = np.nan_to_num(np.nanmax(Wg, -1), nan=0.0)
            assert np.allclose(s, np.maximum(hi - lo, 1e-4) / nl, rtol=1e-6)
            assert np.array_equal(z, -np.rint(lo.astype(np.float32) / s))
    q, s, z = M.group_rtn(W, mask, 4, 128, "all")
    assert np.allclose(s, (W.reshape(8, 2, 128).max(-1) - W.reshape(8, 2, 128).min(-1)) / 15, rtol=1e-6)


def test_robust_scale_and_masked_std():
    rng = np.random.default_rng(5)
    W = rng.normal(0, 1, (64, 32)).astype(np.float32) * np.linspace(0.01, 30, 32, dtype=np.float32)
    mask = (rng.random(W.shape) > 0.3).astype(np.float32)
    sd = M.masked_std(W, mask, 0)
    for j in (0, 7, 31):
        v = W[mask[:, j] != 0, j]
        assert abs(sd[j] - v.std()) < 1e-4 * v.std() + 1e-8
    c = M.robust_scale(sd)
    assert c.min() >= 0.1 - 1e-7 and c.max() <= 10 + 1e-6


def test_cobalt_quantize_end_to_end_packs():
    W, H = _problem(K=64, N=256)
    for (s, bits, g, kpb) in ((0.5, 4, 128, 16), (0.7, 3, 128, 10), (0.3, 2, 64, 23)):
        q, sc, z, c, mask, W_hat = M.cobalt_quantize(W, H, s, 0.5, bits, g, mask_block=32)
        assert (W_hat[mask == 0] == 0).all()
        rel = np.linalg.norm(W_hat - W) / np.linalg.norm(W)
        assert rel < {4: 0.85, 3: 0.95, 2: 1.0}[bits]
        raw = M.to_raw(q, sc, z, c, mask)
        pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.BLKC,
                           bits=bits, group=g, keep_per_block=kpb)
        Wp = R.dequant(pk, 64, 256, R.BLKC, col_scale=raw["col_scale"], bits=bits, group=g, keep_per_block=kpb)
        assert (Wp[mask == 0] == 0).all()
        # the packed matrix reproduces the quantiser's W_hat up to the fp16 rounding of
        # scale / col_scale (and the zero repair, which only touches off-grid groups)
        ok = np.repeat((z >= 0) & (z <= 2 ** bits - 1), g, 1)
        assert np.abs(Wp - W_hat)[ok].max() <= 2.5e-3 * np.abs(W_hat).max()
    # unconstrained balanced mask goes into the dense layout
    q, sc, z, c, mask, W_hat = M.cobalt_quantize(W, H, 0.5, 0.5, 4, 128)
    raw = M.to_raw(q, sc, z, c, mask)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.DENSE4)
    Wp = R.dequant(pk, 64, 256, R.DENSE4, col_scale=raw["col_scale"])
    assert (Wp[mask == 0] == 0).all()


def test_dead_columns_dequantise_to_zero():
    # restates test_deadcols.py:70-87: a column no row keeps is exactly 0 after the round trip
    W, H = _problem(K=32, N=256, outliers=False)
    W[:, 5] = 0.0; H[5, :] = 0; H[:, 5] = 0
    q, sc, z, c, mask, W_hat = M.cobalt_quantize(W, H, 0.5, 0.5, 4, 128)
    assert (W_hat[:, 5] == 0).all()
