"""The torch restatement of the reference's CPU forward (oracle/torch_ref.py, the timed CPU
baseline of bench.py) against the numpy oracle, bit for bit."""
import numpy as np
import pytest
import torch

from oracle import cbk_ref as R
from oracle import torch_ref as T
from tests.helpers import case_id, kw_of, make_raw, oracle_pack
from cobalt_amd import format as F

CASES = [(F.BLK1632_4, 4, 128, 16), (F.BLKC, 3, 128, 10), (F.BLKC, 2, 64, 23), (F.BLKC, 4, 64, 16),
         (F.DENSE4, 4, 128, 0), (F.DENSE8, 8, 128, 0), (F.DENSEB, 3, 64, 0), (F.DENSEB, 2, 128, 0)]


@pytest.mark.parametrize("case", CASES, ids=case_id)
@pytest.mark.parametrize("cs_rows", [0, 1, 2])
def test_torch_dequant_equals_numpy_oracle(case, cs_rows):
    layout, bits, group, keep = case
    K, N = 24, 512
    raw = make_raw(case, K, N, seed=5 + bits)
    pk = oracle_pack(case, raw)
    cs = None
    if cs_rows:
        cs = (np.random.default_rng(1).random((cs_rows, N)) * 1.5 + 0.5).astype(np.float16)
    W = R.dequant(pk, K, N, layout, col_scale=cs, **kw_of(case))
    kw = kw_of(case)
    stride = R.row_stride(layout, N, kw.get("bits"), kw.get("group"), kw.get("keep_per_block"))
    rows = torch.from_numpy(np.asarray(pk["data"], np.uint8))[: K * stride].reshape(K, stride)
    Wt = T.dequant(rows, torch.from_numpy(pk["scale"].reshape(K, -1)), torch.from_numpy(pk["zero"].reshape(K, -1)),
                   None if cs is None else torch.from_numpy(cs), K, N, layout, bits, group, keep or 16)
    assert np.array_equal(Wt.numpy(), W)
    x = torch.randn(3, N, generator=torch.Generator().manual_seed(2)).half()
    y = T.forward(Wt, x).numpy()
    ref = R.forward_ref(W, x.float().numpy())
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-6
