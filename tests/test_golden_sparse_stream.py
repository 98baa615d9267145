"""The variable-length survivor-stream layouts (SPARSE4, SPARSE4X, SPARSE4E) against bytes
written by the reference's own packer and decoded by its own `dequant_reference`
(tests/golden/make_sparse_stream_vectors.py made the fixture): rows with an empty group, a full
group and no survivors at all, densities 0.3 / 0.5 / 0.8."""
import os

import numpy as np
import pytest
import torch

from oracle import cbk_ref as R

FIX = np.load(os.path.join(os.path.dirname(__file__), "golden", "sparse_stream.npz"))
CASES = [(0, 5, 256), (1, 4, 384), (2, 6, 256)]
LAYOUTS = ["SPARSE4", "SPARSE4X", "SPARSE4E"]


def _ref_packed(i, name):
    p = f"c{i}_{name}_"
    return dict(data=FIX[p + "data"], row_off=FIX[p + "row_off"], scale=FIX[p + "scale"], zero=FIX[p + "zero"])


@pytest.mark.parametrize("name", LAYOUTS)
def test_oracle_packer_writes_the_reference_bytes(name):
    for i, K, N in CASES:
        p = f"c{i}_"
        pk = R.pack_matrix(FIX[p + "mask"], FIX[p + "q"], FIX[p + "scale"], FIX[p + "zero"], getattr(R, name))
        ref = _ref_packed(i, name)
        assert np.array_equal(pk["data"], ref["data"]), f"case {i}: row bytes"
        assert np.array_equal(pk["row_off"], ref["row_off"]), f"case {i}: row offsets"
        assert np.array_equal(pk["scale"], ref["scale"]) and np.array_equal(pk["zero"], ref["zero"])
        assert pk["n_survivors"] == int(FIX[p + name + "_nsurv"])


@pytest.mark.parametrize("name", LAYOUTS)
def test_oracle_decoder_reads_the_reference_bytes(name):
    for i, K, N in CASES:
        W = R.dequant(_ref_packed(i, name), K, N, getattr(R, name))
        assert np.array_equal(W, FIX[f"c{i}_{name}_W"]), f"case {i}"


@pytest.mark.gpu
@pytest.mark.parametrize("name", LAYOUTS)
def test_gpu_reads_the_reference_bytes(name):
    """The HIP dequantiser and the row GEMV on the reference's own bytes, through the C ABI."""
    from cobalt_amd import format as F, ops
    from helpers import packed_from_oracle
    for i, K, N in CASES:
        layout = getattr(F, name)
        pm = packed_from_oracle((layout, 4, 128, 0), _ref_packed(i, name), None, K, N, "cuda")
        Wref = FIX[f"c{i}_{name}_W"]
        assert np.array_equal(ops.dequant(pm, torch.float32).cpu().numpy(), Wref), f"case {i}"
        x = torch.randn(3, N, generator=torch.Generator().manual_seed(i)).half()
        y = ops.gemv(pm, x.cuda(), out_dtype=torch.float32).cpu().numpy()
        ref = x.double().numpy() @ Wref.astype(np.float64).T
        assert np.linalg.norm(y - ref) <= 1e-3 * np.linalg.norm(ref)
