"""The C oracle against the numpy oracle and against the mathematics (CPU only).

The numpy oracle is pinned by hand-computed byte vectors in test_oracle_format.py; the C
decoder is written separately from the format text, so agreement of the two on random
matrices of every layout checks both."""
import numpy as np
import pytest

from oracle import cbk_ref as R
from oracle import cbk_ref_c as C
from helpers import FIXED_CASES, SPARSE_CASES, case_id, kw_of, make_raw, oracle_pack


@pytest.mark.parametrize("case", FIXED_CASES + SPARSE_CASES, ids=case_id)
def test_c_dequant_is_bit_identical_to_numpy_oracle(case):
    K, N = 24, 512
    raw = make_raw(case, K, N, seed=3 + case[0])
    pk = oracle_pack(case, raw)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
    Wc = C.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
    assert np.array_equal(W.view(np.uint32) & 0x7FFFFFFF, Wc.view(np.uint32) & 0x7FFFFFFF) and np.array_equal(W, Wc)
    # a row range
    assert np.array_equal(C.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], row0=5, nrows=7, **kw_of(case)), W[5:12])
    assert C.lib().cbk_ref_row_stride(case[0], N, case[1], case[2], case[3]) == (
        0 if case[0] in R.SPARSE_FAMILY else R.row_stride(case[0], N, *[kw_of(case).get(k) for k in ("bits", "group", "keep_per_block")]))


def test_c_dequant_hand_vector_blk1632_4():
    """One row, N=128, the block bytes worked out by hand: mask 0x0000FFFF in every block keeps
    columns 0..15; code bytes 0x10, 0x32, ... give survivor i the code i; zero 3, scale 0.5."""
    N = 128
    row = bytearray()
    row += bytes([0xFF, 0xFF, 0x00, 0x00] * 4)
    row += bytes([0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE] * 4)
    pk = dict(data=np.frombuffer(bytes(row) + bytes(64), np.uint8), scale=np.array([[0.5]], np.float16),
              zero=np.array([[3]], np.uint8))
    W = C.dequant(pk, 1, N, R.BLK1632_4)
    want = np.zeros(N, np.float32)
    for t in range(4):
        want[32 * t: 32 * t + 16] = (np.arange(16) - 3) * 0.5
    assert np.array_equal(W[0], want)


def test_c_dequant_fused_col_scale_rows_and_float64_witness():
    case = (R.BLKC, 3, 64, 10)
    K, N = 18, 256
    raw = make_raw(case, K, N, seed=11)
    pk = oracle_pack(case, raw)
    rng = np.random.default_rng(0)
    for cs_rows, splits in ((2, None), (3, (6, 4))):
        cs = (0.5 + rng.random((cs_rows, N))).astype(np.float16)
        W = R.dequant(pk, K, N, case[0], col_scale=cs, cs_splits=splits, **kw_of(case))
        Wc = C.dequant(pk, K, N, case[0], col_scale=cs, cs_splits=splits, **kw_of(case))
        assert np.array_equal(W, Wc)
        # float64 evaluation of the closed form, rounded once
        q, keep = R.unpack_codes(pk, K, N, case[0], **kw_of(case))
        G = N // 64
        s = np.asarray(pk["scale"], np.float64).reshape(K, G).repeat(64, 1)
        z = np.asarray(pk["zero"], np.float64).reshape(K, G).repeat(64, 1)
        w64 = (q - z) * s * keep * cs.astype(np.float64)[R.col_scale_rows(K, cs_rows, splits)]
        assert np.array_equal(w64.astype(np.float32), Wc)


@pytest.mark.parametrize("case", [(R.BLK1632_4, 4, 128, 16), (R.DENSE4, 4, 128, 0), (R.SPARSE4E, 4, 128, 0),
                                  (R.BLKC, 2, 64, 23)], ids=case_id)
def test_c_forward_matches_numpy_forward(case):
    K, N, M = 40, 384, 3
    raw = make_raw(case, K, N, seed=21)
    pk = oracle_pack(case, raw)
    x = np.random.default_rng(2).standard_normal((M, N)).astype(np.float16).astype(np.float32)
    bias = np.random.default_rng(3).standard_normal(K)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
    ref = R.forward_ref(W, x, bias=bias)
    C.set_threads(2)
    y = C.forward(pk, K, N, case[0], x, col_scale=raw["col_scale"], bias=bias, **kw_of(case))
    assert np.allclose(y, ref, rtol=1e-12, atol=1e-12)
    # linearity in x and exact zero for an all-pruned input direction
    y2 = C.forward(pk, K, N, case[0], 2 * x, col_scale=raw["col_scale"], **kw_of(case))
    y1 = C.forward(pk, K, N, case[0], x, col_scale=raw["col_scale"], **kw_of(case))
    assert np.array_equal(y2, 2 * y1)


def test_c_rejects_bad_arguments():
    pk = dict(data=np.zeros(4096, np.uint8), scale=np.ones((1, 1), np.float16), zero=np.zeros((1, 1), np.uint8))
    with pytest.raises(ValueError):
        C.dequant(pk, 1, 100, R.DENSE4)          # N not a multiple of 128
    with pytest.raises(ValueError):
        C.dequant(pk, 1, 128, 4)                 # BF16 layout id has no packed form here
