"""The fixed-stride layouts (DENSE4, DENSE8, BLK1632_4, BLK1632_6) and the row-interleaved gate/up
fusion against bytes written by the reference's own packer and decoded by its own
`dequant_reference` (tests/golden/make_fixed_stride_vectors.py made the fixture): a 16-of-32 mask,
two zero points off the grid per matrix (repaired from the 0-inclusive hull), a column scale."""
import os

import numpy as np
import pytest
import torch

from oracle import cbk_ref as R

FIX = np.load(os.path.join(os.path.dirname(__file__), "golden", "fixed_stride.npz"))
CASES = [("DENSE4", 4, 6, 256), ("DENSE8", 8, 6, 384), ("BLK1632_4", 4, 6, 256), ("BLK1632_6", 6, 6, 384)]


def _ref_packed(p):
    return dict(data=FIX[p + "data"], row_off=None, scale=FIX[p + "scale"], zero=FIX[p + "zero"])


def _same(a, b):
    return np.array_equal(np.asarray(a, np.float32) + np.float32(0), np.asarray(b, np.float32) + np.float32(0))


@pytest.mark.parametrize("name,bits,K,N", CASES)
def test_oracle_packer_writes_the_reference_bytes(name, bits, K, N):
    p = name + "_"
    pk = R.pack_matrix(FIX[p + "mask"], FIX[p + "q"], FIX[p + "scale_in"], FIX[p + "zero_in"], getattr(R, name))
    assert np.array_equal(pk["data"], FIX[p + "data"])
    assert np.array_equal(pk["scale"], FIX[p + "scale"]) and np.array_equal(pk["zero"], FIX[p + "zero"])
    assert pk["n_survivors"] == int(FIX[p + "nsurv"]) and pk["n_zero_fixed"] == int(FIX[p + "nfixed"]) == 2


@pytest.mark.parametrize("name,bits,K,N", CASES)
def test_oracle_decoder_reads_the_reference_bytes(name, bits, K, N):
    p = name + "_"
    W = R.dequant(_ref_packed(p), K, N, getattr(R, name), col_scale=FIX[p + "col_scale"].reshape(1, N))
    assert _same(W, FIX[p + "W"])
    assert _same(R.dequant_scalar(_ref_packed(p), K, N, getattr(R, name), col_scale=FIX[p + "col_scale"].reshape(1, N)), FIX[p + "W"])


@pytest.mark.parametrize("name,bits,K,N", CASES)
def test_product_packer_writes_the_reference_bytes(name, bits, K, N):
    from cobalt_amd import format as F
    p = name + "_"
    t = lambda k: torch.from_numpy(FIX[p + k])
    pm = F.pack_raw(t("mask"), t("q"), t("scale_in"), t("zero_in"), t("col_scale"), getattr(F, name))
    assert np.array_equal(pm.array("data").numpy(), FIX[p + "data"])
    assert np.array_equal(pm.array("scale").numpy().reshape(K, -1), FIX[p + "scale"])
    assert np.array_equal(pm.array("zero").numpy().reshape(K, -1), FIX[p + "zero"])
    assert (pm.n_survivors, pm.n_zero_fixed) == (int(FIX[p + "nsurv"]), 2)


def _gateup_raw():
    il = lambda k: np.stack([FIX[f"gateup_gate_{k}"], FIX[f"gateup_up_{k}"]], 1).reshape(10, -1)
    return il("mask"), il("q"), il("scale_in"), il("zero_in")


def test_interleaved_gate_up_with_two_column_scale_rows():
    """Row 2i is gate row i under column-scale row 0, row 2i+1 is up row i under row 1
    (pack_cobalt.py:654-667, docs/FORMAT.md:126-133)."""
    pk = R.pack_matrix(*_gateup_raw(), R.BLK1632_4)
    assert np.array_equal(pk["data"], FIX["gateup_data"]) and np.array_equal(pk["zero"], FIX["gateup_zero"])
    assert np.array_equal(pk["scale"], FIX["gateup_scale"])
    W = R.dequant(_ref_packed("gateup_"), 10, 256, R.BLK1632_4, col_scale=FIX["gateup_col_scale"])
    assert _same(W, FIX["gateup_W"])
    assert _same(R.dequant_scalar(_ref_packed("gateup_"), 10, 256, R.BLK1632_4, col_scale=FIX["gateup_col_scale"]), FIX["gateup_W"])
    # the product's fusion of the two separately packed halves lands on the same bytes
    from cobalt_amd import format as F
    t = lambda h, k: torch.from_numpy(FIX[f"gateup_{h}_{k}"])
    halves = [F.pack_raw(t(h, "mask"), t(h, "q"), t(h, "scale_in"), t(h, "zero_in"),
                         torch.from_numpy(FIX["gateup_col_scale"][i]), F.BLK1632_4) for i, h in enumerate(("gate", "up"))]
    fused = F.fuse_rows(halves, interleave=True)
    assert fused.cs_rows == 2 and np.array_equal(fused.array("data").numpy(), FIX["gateup_data"])
    assert np.array_equal(fused.array("col_scale").numpy().reshape(2, 256), FIX["gateup_col_scale"])


@pytest.mark.gpu
def test_gpu_reads_the_reference_bytes():
    """The HIP dequantiser (row-major and tiled order) and the decode GEMV on the reference's own
    bytes, through the C ABI."""
    from cobalt_amd import format as F, ops
    from helpers import packed_from_oracle
    todo = [(n + "_", getattr(F, n), b, K, N, FIX[n + "_col_scale"].reshape(1, N)) for n, b, K, N in CASES]
    todo.append(("gateup_", F.BLK1632_4, 4, 10, 256, FIX["gateup_col_scale"]))
    for p, layout, bits, K, N, cs in todo:
        case = (layout, bits, 128, 16 if layout in (F.BLK1632_4, F.BLK1632_6) else 0)
        for tiled in (False, True):
            pm = packed_from_oracle(case, _ref_packed(p), cs, K, N, "cuda", tiled=tiled)
            assert _same(ops.dequant(pm, torch.float32).cpu().numpy(), FIX[p + "W"]), (p, tiled)
            x = torch.randn(2, N, generator=torch.Generator().manual_seed(K)).half()
            y = ops.gemv(pm, x.cuda(), out_dtype=torch.float32).cpu().numpy()
            ref = x.double().numpy() @ FIX[p + "W"].astype(np.float64).T
            assert np.abs(y - ref).max() <= 2e-5 * np.abs(ref).max(), (p, tiled)
