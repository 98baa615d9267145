"""Zero-point repair against vectors written by the reference's own
`pack_cobalt._fix_zero_range` (tests/golden/make_fix_zero_vectors.py made the fixture)."""
import os

import numpy as np
import torch

from cobalt_amd import format as F
from oracle import cbk_ref as R

FIX = np.load(os.path.join(os.path.dirname(__file__), "golden", "fix_zero_range.npz"))


def _case(i):
    p = f"c{i}_"
    return {k[len(p):]: FIX[k] for k in FIX.files if k.startswith(p)}


def test_oracle_fix_zero_range_matches_reference_vectors():
    for i in range(3):
        c = _case(i)
        q, s, z, n = R.fix_zero_range(c["q"], c["scale"], c["zero"], c["keep"], int(c["nlevels"]))
        assert n == int(c["n_fixed"]) and n >= 3
        assert np.array_equal(q, c["q_out"]) and np.array_equal(z, c["zero_out"])
        assert np.array_equal(s.astype(np.float32), c["scale_out"])


def test_product_fix_zero_range_matches_reference_vectors():
    for i in range(3):
        c = _case(i)
        q, s, z, n = F.fix_zero_range(torch.from_numpy(c["q"]), torch.from_numpy(c["scale"]), torch.from_numpy(c["zero"]),
                                      torch.from_numpy(c["keep"]), int(c["nlevels"]), 128)
        assert n == int(c["n_fixed"])
        assert np.array_equal(q.numpy(), c["q_out"]) and np.array_equal(z.numpy(), c["zero_out"])
        assert np.array_equal(s.numpy(), c["scale_out"])
