"""The compressor (Wanda importance -> balanced / blocked keep-mask -> OBS compensation ->
column scale -> group RTN) against vectors written by the reference's own
`cobalt_math.cobalt_quantize` (src/cobaltkernel/cobalt_math.py:336-394;
tests/golden/make_cobalt_quantize_vectors.py made the fixture): four seeded matrices covering
the balanced and the 32-column blocked mask, 2/3/4-bit codes, groups of 64 and 128, sparsity
0.3 / 0.5 / 0.6875, more and fewer calibration rows than columns."""
import os

import numpy as np
import torch

from cobalt_amd import compress as C
from oracle import cobalt_math_ref as M

FIX = np.load(os.path.join(os.path.dirname(__file__), "golden", "cobalt_quantize.npz"))
N_CASES = 4


def _case(i):
    p = f"c{i}_"
    c = {k[len(p):]: FIX[k] for k in FIX.files if k.startswith(p)}
    X = c["X"].astype(np.float64)
    c["H"] = (X.T @ X).astype(np.float32)                     # float64 accumulate, one rounding: as the generator
    sp, beta, bits, group, mb = c["cfg"]
    c["args"] = (float(sp), float(beta), int(bits), int(group), int(mb))
    c["keep"] = np.unpackbits(c["mask"], axis=-1, bitorder="little")[:, : c["W"].shape[1]].astype(bool)
    return c


def test_oracle_compressor_matches_reference_vectors():
    for i in range(N_CASES):
        c = _case(i)
        sp, beta, bits, group, mb = c["args"]
        q, s, z, cs, mask, W_hat = M.cobalt_quantize(c["W"], c["H"], sp, beta, bits, group, mask_block=mb)
        keep = c["keep"]
        assert np.array_equal(mask != 0, keep), f"case {i}: keep-mask differs in {(keep != (mask != 0)).sum()} places"
        assert np.array_equal(q[keep], c["q"][keep].astype(q.dtype)), f"case {i}: codes"
        assert np.array_equal(z, c["zero"]), f"case {i}: zero points"
        # float32 chains of different libraries (numpy here, torch there): equal to a few ulp;
        # stored as fp16, as the RAW schema stores them, at most a few values fall on the other
        # side of a rounding boundary, by one fp16 step
        assert np.allclose(s, c["scale"], rtol=2e-4, atol=0) and np.allclose(cs, c["col_scale"], rtol=2e-4, atol=0)
        for mine, ref in ((s, c["scale"]), (cs, c["col_scale"])):
            a, b = mine.astype(np.float16), ref.astype(np.float16)
            assert (a != b).mean() <= 0.03
            assert np.all(np.abs(a.astype(np.float32) - b.astype(np.float32)) <= np.abs(b.astype(np.float32)) * 2.0 ** -10)
        rel = np.linalg.norm(W_hat - c["W"]) / np.linalg.norm(c["W"])
        assert abs(rel - float(c["relerr"])) < 1e-4 * float(c["relerr"])


def test_product_compressor_matches_reference_vectors_bit_for_bit():
    """`cobalt_amd.compress.cobalt_compress` (torch; the same code runs on the GPU) gives the
    reference's RAW arrays: mask bytes, codes on the kept positions, fp16 scale, zero, col_scale."""
    for i in range(N_CASES):
        c = _case(i)
        sp, beta, bits, group, mb = c["args"]
        r = C.cobalt_compress(torch.from_numpy(c["W"]), torch.from_numpy(c["H"]), sp, bits, group, beta, mb)
        keep = c["keep"]
        assert np.array_equal(r["mask"].numpy(), c["mask"]), f"case {i}: mask bytes"
        assert np.array_equal(r["q"].numpy()[keep], c["q"][keep]), f"case {i}: codes"
        assert (r["q"].numpy()[~keep] == 0).all()
        assert np.array_equal(r["scale"].numpy(), c["scale"].astype(np.float16)), f"case {i}: scale"
        assert np.array_equal(r["zero"].float().numpy(), c["zero"]), f"case {i}: zero"
        assert np.array_equal(r["col_scale"].numpy(), c["col_scale"].astype(np.float16)), f"case {i}: col_scale"


def test_fixture_is_not_degenerate():
    """The vectors exercise what they are meant to: exact sparsity, off-centre zero points, every
    code value, a damping above its floor."""
    for i in range(N_CASES):
        c = _case(i)
        sp, beta, bits, group, mb = c["args"]
        keep = c["keep"]
        assert abs(keep.mean() - (1 - sp)) < 0.01
        if mb:
            assert (keep.reshape(keep.shape[0], -1, mb).sum(-1) == round((1 - sp) * mb)).all()
        assert set(np.unique(c["q"][keep]).tolist()) == set(range(2 ** bits))
        assert float(c["damping"]) > 1e-2 and len(np.unique(c["zero"])) > 1
