"""GPU parity: the HIP library, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Bars: dequantised weights bit-exact (value equality; -0.0 == 0.0, as the
reference's own check does, src/prod/verify.py:139); layer outputs within relative Frobenius
error 1e-3 of x @ W_hat.T with W_hat in float32 and a float64 accumulator."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import cbk_ref as R
from cobalt_amd import format as F
from cobalt_amd import _lib, ops
from cobalt_amd.linear import CobaltLinear
from helpers import (FIXED_CASES, SPARSE_CASES, acts, case_id, kw_of, make_raw, oracle_pack, packed_from_oracle,
                     product_pack, rel_fro)

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 1e-3          # relative Frobenius error of a layer output (the bar this layer is held to)


def _np(t):
    return t.detach().float().cpu().numpy()


def _bf16_round(a):
    return _np(torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16))


def _f16_round(a):
    return _np(torch.from_numpy(np.asarray(a, np.float32)).to(torch.float16))


# ------------------------------------------------------------------ dequant, bit-exact
@pytest.mark.parametrize("tiled", [False, True], ids=["rowmajor", "tiled"])
@pytest.mark.parametrize("case", FIXED_CASES + SPARSE_CASES, ids=case_id)
def test_dequant_bit_exact(case, tiled):
    if tiled and case in SPARSE_CASES:
        pytest.skip("the variable-length layouts have no tiled form")
    for (K, N) in ((64, 1024), (40, 5376)):
        raw = make_raw(case, K, N, seed=K + N + case[0])
        pk = oracle_pack(case, raw)
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
        W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
        got = _np(ops.dequant(pm, torch.float32))
        assert np.array_equal(got, W), f"{case_id(case)} {K}x{N}: {np.abs(got - W).max()}"
        W0 = R.dequant(pk, K, N, case[0], **kw_of(case))
        assert np.array_equal(_np(ops.dequant(pm, torch.float32, with_col_scale=False)), W0)
        assert np.array_equal(_np(ops.dequant(pm, torch.bfloat16)), _bf16_round(W))
        assert np.array_equal(_np(ops.dequant(pm, torch.float16)), _f16_round(W))
        # a row window
        assert np.array_equal(_np(ops.dequant(pm, torch.float32, row0=8, nrows=16)), W[8:24])


def test_dequant_fused_col_scale_rows_and_subnormal_scales():
    K, N = 48, 512
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=3, block=32)
    raw["scale"][::5] = np.float16(6.7e-6)                # fp16 subnormal scale
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.BLK1632_4)
    rng = np.random.default_rng(0)
    for cs_rows, splits in ((2, (0, 0)), (3, (32, 8))):
        cs = (rng.random((cs_rows, N)) * 1.5 + 0.5).astype(np.float16)
        pm = packed_from_oracle((F.BLK1632_4, 4, 128, 16), pk, cs, K, N, DEV, cs_splits=splits)
        W = R.dequant(pk, K, N, R.BLK1632_4, col_scale=cs, cs_splits=splits)
        assert np.array_equal(_np(ops.dequant(pm, torch.float32)), W)
        assert (W[::5] != 0).any()


def test_pruned_positions_exactly_zero_off_grid_zero_point():
    K, N = 32, 1024
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=9, block=32)
    keep = R.unpack_bits(raw["mask"], N)
    off = np.full((K, N // 128), 15 + 37, np.float16)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], off, R.BLK1632_4, fix_zero=False)
    pm = packed_from_oracle((F.BLK1632_4, 4, 128, 16), pk, raw["col_scale"], K, N, DEV)
    W = _np(ops.dequant(pm, torch.float32))
    assert (W[~keep] == 0).all() and np.array_equal(W, R.dequant(pk, K, N, R.BLK1632_4, col_scale=raw["col_scale"]))


# ------------------------------------------------------------------ decode GEMV
@pytest.mark.parametrize("tiled", [False, True], ids=["rowmajor", "tiled"])
@pytest.mark.parametrize("case", FIXED_CASES + SPARSE_CASES, ids=case_id)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_gemv_matches_oracle(case, dtype, tiled):
    if tiled and case in SPARSE_CASES:
        pytest.skip("the variable-length layouts have no tiled form")
    for (K, N) in ((192, 4096), (72, 5376)):
        raw = make_raw(case, K, N, seed=K + N + 31 * case[0])
        pk = oracle_pack(case, raw)
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
        W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
        for M in (1, 2, 3, 4, 8, 16):
            x = acts(M, N, dtype, seed=M)
            ref = R.forward_ref(W, _np(x))
            y = ops.gemv(pm, x.to(DEV), out_dtype=torch.float32)
            err = rel_fro(_np(y), ref)
            assert err < TOL, f"{case_id(case)} {K}x{N} M={M}: {err}"
            # the reference's own GEMV gate: max|err| / max|ref| < 2e-5 (test_gemv.py:162-167)
            assert np.abs(_np(y) - ref).max() / np.abs(ref).max() < 2e-5


@pytest.mark.parametrize("case", SPARSE_CASES, ids=case_id)
def test_gemv_sparse_streams_on_long_rows(case):
    """Variable-length layouts with more than 64 groups per row (N = 14336: 112 groups), where the
    row kernel sums the SPARSE4 group offsets over the wavefront in more than one round."""
    K, N = 24, 14336
    raw = make_raw(case, K, N, seed=3 + case[0])
    pk = oracle_pack(case, raw)
    pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
    for M in (1, 3, 6):
        x = acts(M, N, torch.float16, seed=M)
        y = ops.gemv(pm, x.to(DEV), out_dtype=torch.float32)
        assert rel_fro(_np(y), R.forward_ref(W, _np(x))) < 1e-5, (case_id(case), M)


@pytest.mark.parametrize("case", SPARSE_CASES + [(F.DENSE8, 8, 128, 0)], ids=case_id)
def test_gemv_integer_dot_row_kernels(case):
    """The decode kernels of the survivor streams and of DENSE8 (activation digits in LDS, integer
    dot products; the streams with the byte-permute expansion, the 8-bit codes as q - 128 and the
    zero point, any uint8 value, through the groups' digit sums): rows shorter than the 64 blocks of a wavefront, more rows than one pass of
    the resident wavefronts, the longest row whose digits fit (one activation row per pass) and one
    beyond it (float row kernel); one to nine activation rows, both activation types, a bias;
    a row's result does not depend on how many rows the call has."""
    for (K, N) in ((5, 128), (37, 384), (300, 4096), (4200, 256), (16, 21504), (9, 32768), (6, 32896)):
        raw = make_raw(case, K, N, seed=K + N + case[0])
        pk = oracle_pack(case, raw)
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV)
        W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
        bias = acts(1, K, torch.float32, seed=K)[0]
        for M, dtype in ((1, torch.float16), (2, torch.bfloat16), (3, torch.float16), (4, torch.bfloat16), (5, torch.float16),
                         (9, torch.float16)):
            x = acts(M, N, dtype, seed=M + N)
            ref = R.forward_ref(W, _np(x))
            y = ops.gemv(pm, x.to(DEV), out_dtype=torch.float32)
            assert rel_fro(_np(y), ref) < 1e-5, (case_id(case), K, N, M)
            yb = ops.gemv(pm, x.to(DEV), bias=bias.to(DEV), out_dtype=torch.float32)
            assert rel_fro(_np(yb), ref + _np(bias)[None, :]) < 1e-5, (case_id(case), K, N, M)
            if N <= 32768:
                y1 = ops.gemv(pm, x[M - 1:M].to(DEV), out_dtype=torch.float32)
                assert torch.equal(y1[0], y[M - 1]), (case_id(case), K, N, M)


@pytest.mark.parametrize("shape", [(49200, 128), (24600, 640), (1768, 14336), (6160, 4096)], ids=lambda s: f"{s[0]}x{s[1]}")
def test_gemv_survivor_streams_on_matrix_cores(shape):
    """SPARSE4X / SPARSE4E from 1536 tile-steps (16 rows x 512 columns) on: the 16-row matrix-core
    kernel for rows of different lengths.  One step per row and thirteen rounds of sixteen tiles
    (49200 x 128), a last step with one group of four (640 columns), one tile per workgroup cut
    into fourteen parts with two wavefronts idle (14336 columns, two activation rows per pass), two
    tiles per round (6160 x 4096); a last tile of fewer than sixteen rows in each.  One to nine
    activation rows, both activation types, a bias, run-to-run identical, and a row's result does
    not depend on how many rows the call has."""
    K, N = shape
    small = torch.empty(256, dtype=torch.uint8, device=DEV)
    for case in ([(F.SPARSE4X, 4, 128, 0), (F.SPARSE4E, 4, 128, 0)] if N == 640 else [(F.SPARSE4X, 4, 128, 0)]):
        raw = make_raw(case, K, N, seed=K + N + case[0])
        pk = oracle_pack(case, raw)
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV)
        W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
        bias = acts(1, K, torch.float32, seed=K)[0]
        for M, dtype in ((1, torch.float16), (2, torch.bfloat16), (4, torch.float16), (5, torch.bfloat16), (8, torch.float16),
                         (9, torch.float16)):
            x = acts(M, N, dtype, seed=M + N)
            ref = R.forward_ref(W, _np(x))
            y = ops.gemv(pm, x.to(DEV), out_dtype=torch.float32)
            assert rel_fro(_np(y), ref) < 1e-5, (case_id(case), K, N, M)
            assert np.abs(_np(y) - ref).max() / np.abs(ref).max() < 2e-5
            assert torch.equal(ops.gemv(pm, x.to(DEV), out_dtype=torch.float32), y)
            y1 = ops.gemv(pm, x[M - 1:M].to(DEV), out_dtype=torch.float32)
            assert torch.equal(y1[0], y[M - 1]), (case_id(case), K, N, M)
            # More rows than fit in LDS as whole rows (14336 columns: from four on): split over the
            # workgroups by columns where the caller has left room for the part sums, in passes
            # of fewer rows where not; the same bits either way.
            need = _lib.lib().cbk_workspace_bytes(ctypes.byref(pm.desc()), M)
            assert (need >= (K + 15) // 16 * 2 * min(M, 8) * 16 * 4) == (N == 14336 and M >= 4), (K, N, M, need)
            assert torch.equal(ops.gemv(pm, x.to(DEV), out_dtype=torch.float32, workspace=small), y), (case_id(case), K, N, M)
            if M in (1, 8):
                yb = ops.gemv(pm, x.to(DEV), bias=bias.to(DEV), out_dtype=dtype)
                want = (y + bias.to(DEV).to(dtype).float()[None, :]).to(dtype)      # (the bias has the output's type)
                assert torch.equal(yb, want), (case_id(case), K, N, M)


@pytest.mark.parametrize("shape", [(6160, 4096), (1768, 14336)], ids=lambda s: f"{s[0]}x{s[1]}")
def test_gemv_survivor_streams_fused_gate_up(shape):
    """A fused gate/up matrix (two col_scale vectors by row parity, docs/FORMAT.md:126-151) as
    SPARSE4X on the matrix-core stream kernel: every activation row is staged twice, once per
    vector, and a weight row keeps the sums of its own parity.  Whole rows in LDS (4096 columns)
    and split by columns or in passes of one row (14336 columns); bias; row by row against M = 1."""
    K, N = shape
    case = (F.SPARSE4X, 4, 128, 0)
    raw = make_raw(case, K, N, seed=K + N)
    pk = oracle_pack(case, raw)
    rng = np.random.default_rng(K)
    cs = (rng.random((2, N)) * 1.5 + 0.5).astype(np.float16)
    pm = packed_from_oracle(case, pk, cs, K, N, DEV)
    W = R.dequant(pk, K, N, case[0], col_scale=cs, cs_splits=(0, 0))
    small = torch.empty(256, dtype=torch.uint8, device=DEV)
    bias = acts(1, K, torch.float32, seed=K)[0].to(DEV)
    for M, dtype in ((1, torch.float16), (2, torch.bfloat16), (3, torch.float16), (5, torch.bfloat16), (8, torch.float16)):
        x = acts(M, N, dtype, seed=M + N)
        ref = R.forward_ref(W, _np(x))
        y = ops.gemv(pm, x.to(DEV), out_dtype=torch.float32)
        assert rel_fro(_np(y), ref) < 1e-5, (K, N, M)
        assert torch.equal(ops.gemv(pm, x.to(DEV), out_dtype=torch.float32, workspace=small), y), (K, N, M)
        y1 = ops.gemv(pm, x[M - 1:M].to(DEV), out_dtype=torch.float32)
        assert torch.equal(y1[0], y[M - 1]), (K, N, M)
        yb = ops.gemv(pm, x.to(DEV), bias=bias, out_dtype=torch.float32)
        assert torch.equal(yb, y + bias[None, :]), (K, N, M)


@pytest.mark.parametrize("case", SPARSE_CASES, ids=case_id)
def test_gemv_survivor_streams_fused_qkv(case):
    """A fused q | k | v matrix (three col_scale vectors by row range, docs/FORMAT.md:126-151) of
    survivor streams: run range by range, each with its vector (here the q range is large enough
    for the matrix-core kernel where the layout has group offsets, k and v go to the row kernel);
    range boundaries off the 16-row grid."""
    kq, kk, kv, N = 4100, 1020, 1024, 4096
    K = kq + kk + kv
    raw = make_raw(case, K, N, seed=K + case[0])
    pk = oracle_pack(case, raw)
    rng = np.random.default_rng(K)
    cs = (rng.random((3, N)) * 1.5 + 0.5).astype(np.float16)
    pm = packed_from_oracle(case, pk, cs, K, N, DEV, cs_splits=(kq, kk))
    W = R.dequant(pk, K, N, case[0], col_scale=cs, cs_splits=(kq, kk))
    bias = acts(1, K, torch.float32, seed=K)[0].to(DEV)
    for M, dtype in ((1, torch.float16), (3, torch.bfloat16), (8, torch.float16)):
        x = acts(M, N, dtype, seed=M + N)
        ref = R.forward_ref(W, _np(x))
        y = ops.gemv(pm, x.to(DEV), out_dtype=torch.float32)
        assert rel_fro(_np(y), ref) < 1e-5, (case_id(case), M)
        y1 = ops.gemv(pm, x[M - 1:M].to(DEV), out_dtype=torch.float32)
        assert torch.equal(y1[0], y[M - 1]), (case_id(case), M)
        assert torch.equal(ops.gemv(pm, x.to(DEV), bias=bias, out_dtype=torch.float32), y + bias[None, :]), (case_id(case), M)


def test_gemv_survivor_streams_over_many_rounds():
    """The matrix-core stream kernel where a workgroup goes through several rounds of two tiles
    with eight parts each (20496 x 4096: five or six tiles per workgroup): the part sums of a
    round meet in one of two LDS buffers, behind a barrier at one activation row, through arrival
    counters from two rows on (a wavefront that is rounds ahead waits for the buffer).  Checked
    against float64 products with the library's own dequantised matrix (itself bit-exact against
    the oracle in the tests above): every M, run to run, and row by row against M = 1."""
    K, N = 20496, 4096
    pm = F.synth_packed(K, N, F.SPARSE4X, 4, 128, None, seed=17, device=DEV)
    W = ops.dequant(pm, torch.float32).double()
    x8 = acts(8, N, torch.float16, seed=3).to(DEV)
    rows = [ops.gemv(pm, x8[i:i + 1], out_dtype=torch.float32)[0] for i in range(8)]
    for M in (1, 2, 3, 4, 5, 8):
        x = x8[:M]
        y = ops.gemv(pm, x, out_dtype=torch.float32)
        ref = x.double() @ W.T
        assert float((y.double() - ref).norm() / ref.norm()) < 1e-5, M
        for _ in range(3):
            assert torch.equal(ops.gemv(pm, x, out_dtype=torch.float32), y), M
        for i in range(M):
            assert torch.equal(y[i], rows[i]), (M, i)


def test_gemv_survivor_streams_of_uneven_density():
    """The matrix-core stream kernel on rows whose groups keep nothing, a tenth, half, nine tenths
    or all of their columns, group by group at random, with whole rows kept and whole rows pruned:
    blocks of 0 to 32 survivors at every skew of the code stream (the fifth code dword of a block
    is loaded only where its survivors reach it)."""
    K, N = 4112, 3072
    case = (F.SPARSE4X, 4, 128, 0)
    raw = make_raw(case, K, N, seed=5)
    rng = np.random.default_rng(11)
    dens = rng.choice(np.array([0.0, 0.1, 0.5, 0.9, 1.0]), size=(K, N // 128))
    keep = rng.random((K, N)) < np.repeat(dens, 128, axis=1)
    keep[::97] = True
    keep[5::101] = False
    raw["q"] = (rng.integers(0, 16, (K, N), dtype=np.uint8) * keep).astype(np.uint8)
    raw["mask"] = R.pack_bits(keep)
    pk = oracle_pack(case, raw)
    pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
    assert (W[5::101] == 0).all()
    for M, dtype in ((1, torch.float16), (3, torch.bfloat16), (8, torch.float16)):
        x = acts(M, N, dtype, seed=M + N)
        ref = R.forward_ref(W, _np(x))
        y = ops.gemv(pm, x.to(DEV), out_dtype=torch.float32)
        assert rel_fro(_np(y), ref) < 1e-5, M
        assert np.abs(_np(y) - ref).max() / np.abs(ref).max() < 2e-5
        assert (_np(y)[:, 5::101] == 0).all()
        y1 = ops.gemv(pm, x[M - 1:M].to(DEV), out_dtype=torch.float32)
        assert torch.equal(y1[0], y[M - 1]), M


ALL_MFMA_CASES = [(F.BLKC, b, g, k) for b in (2, 3, 4) for g in (64, 128) for k in (10, 16, 23)] + \
                 [(F.DENSEB, b, g, 0) for b in (2, 3, 4) for g in (64, 128)]


@pytest.mark.parametrize("tiled", [False, True], ids=["rowmajor", "tiled"])
@pytest.mark.parametrize("case", ALL_MFMA_CASES, ids=case_id)
def test_gemv_every_kernel_configuration(case, tiled):
    """Every instantiation of the matrix-core decode kernel (code width x survivors per block x
    group size x activation rows 1..8), on shapes that give one, two and several macro-steps per
    wavefront and a partial last step, run twice: results must match the oracle and each other."""
    for (K, N) in ((32, 4096), (48, 5376), (16, 14336)):
        raw = make_raw(case, K, N, seed=K + N + 7 * case[1])
        pk = oracle_pack(case, raw)
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
        W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
        for M in range(1, 9):
            x = acts(M, N, torch.bfloat16, seed=M) * (1.0 + 99.0 * (M == 5))
            ref = R.forward_ref(W, _np(x))
            y = ops.gemv(pm, x.to(DEV), out_dtype=torch.float32)
            assert rel_fro(_np(y), ref) < TOL, f"{case_id(case)} {K}x{N} M={M}"
            assert torch.equal(ops.gemv(pm, x.to(DEV), out_dtype=torch.float32), y)


def test_gemv_batch_matches_single_calls():
    """A batched launch against one call per matrix.  How a row is cut into parts depends on the
    launch as a whole (its tiles against the 256 workgroups), so the two agree to float32 rounding
    of the partial sums, not to the bit; each of them is run-to-run identical, and inside one
    grouping a row's result does not depend on M (the tests further down)."""
    case = (F.BLK1632_4, 4, 128, 16)
    shapes = [(4096, 4096), (1024, 4096), (1024, 4096), (512, 14336)]
    pms = [F.synth_packed(K, N, *case[:3], case[3], seed=i, device=DEV).to_tiled() for i, (K, N) in enumerate(shapes)]
    for M in (1, 3, 8, 12):
        xs = [acts(M, N, torch.float16, seed=N + i).to(DEV) for i, (K, N) in enumerate(shapes)]
        bs = [torch.randn(K, device=DEV).half() for K, N in shapes]
        ys = ops.gemv_batch(pms, xs, biases=bs, out_dtype=torch.float32)
        again = ops.gemv_batch(pms, xs, biases=bs, out_dtype=torch.float32)
        for pm, x, b, y, y2 in zip(pms, xs, bs, ys, again):
            single = ops.gemv(pm, x, bias=b, out_dtype=torch.float32)
            assert float((y - single).abs().max() / single.abs().max()) < 1e-6
            assert torch.equal(y, y2)
    # a mixed batch (different code widths) degrades to single calls and still agrees
    pm3 = F.synth_packed(256, 4096, F.BLKC, 3, 128, 10, seed=5, device=DEV)
    xs = [acts(2, 4096, torch.bfloat16, seed=1).to(DEV)] * 2
    ys = ops.gemv_batch([pms[0], pm3], xs, out_dtype=torch.float32)
    assert torch.equal(ys[0], ops.gemv(pms[0], xs[0], out_dtype=torch.float32))     # (the same launches either way)
    assert torch.equal(ys[1], ops.gemv(pm3, xs[1], out_dtype=torch.float32))


def test_gemv_batch_of_staged_and_column_split_matrices():
    """One call over matrices of different row lengths at two to eight activation rows: the long
    rows go to the column-split kernel (one launch for all of them), the others to the main kernel.
    Every output against float64 on the dequantised weights, against one call per matrix (to
    float32 rounding: a row's parts follow the launch), and row m of the batch at M rows against
    the same batch at one row, bit for bit.  Eight long matrices fill the argument block."""
    case = (F.BLK1632_4, 4, 128, 16)
    for shapes in ([(40, 14336), (100, 4096), (16, 21504), (2000, 5376)], [(16 + 16 * i, 8192 + 1024 * i) for i in range(8)]):
        pms = [F.synth_packed(K, N, *case[:3], case[3], seed=i, device=DEV).to_tiled() for i, (K, N) in enumerate(shapes)]
        Ws = [ops.dequant(pm, torch.float32).double() for pm in pms]
        for M in (8, 3):
            xs = [acts(M, N, torch.bfloat16, seed=N + i).to(DEV) for i, (K, N) in enumerate(shapes)]
            bs = [torch.randn(K, device=DEV) for K, N in shapes]
            ys = ops.gemv_batch(pms, xs, biases=bs, out_dtype=torch.float32)
            again = ops.gemv_batch(pms, xs, biases=bs, out_dtype=torch.float32)
            rows = [ops.gemv_batch(pms, [x[i:i + 1] for x in xs], biases=bs, out_dtype=torch.float32) for i in range(M)]
            for j, (pm, W, x, b, y, y2) in enumerate(zip(pms, Ws, xs, bs, ys, again)):
                ref = x.double() @ W.t() + b.double()
                assert float((y.double() - ref).abs().max() / ref.abs().max()) < 2e-5, (shapes[j], M)
                single = ops.gemv(pm, x, bias=b, out_dtype=torch.float32)
                assert float((y - single).abs().max() / single.abs().max()) < 1e-6, (shapes[j], M)
                assert torch.equal(y, y2)
                for i in range(M):
                    assert torch.equal(rows[i][j][0], y[i]), (shapes[j], M, i)


def test_gemv_batch_of_mixed_layouts_with_and_without_workspace():
    """A batch that the one-launch path does not take (a survivor-stream matrix with long rows
    beside fixed-stride ones) runs matrix by matrix, each with its slice of the workspace; with
    no workspace at all the call still succeeds (cbk_gemv does without) and gives the same bits."""
    pms = [F.synth_packed(2048, 14336, F.SPARSE4X, 4, 128, None, seed=1, device=DEV),
           F.synth_packed(64, 14336, F.BLK1632_4, 4, 128, 16, seed=2, device=DEV).to_tiled(),
           F.synth_packed(4112, 3072, F.SPARSE4, 4, 128, None, seed=3, device=DEV)]
    M = 8
    xs = [acts(M, pm.N, torch.float16, seed=i).to(DEV) for i, pm in enumerate(pms)]
    ys = ops.gemv_batch(pms, xs, out_dtype=torch.float32)
    L = _lib.lib()
    n = len(pms)
    P = ctypes.c_void_p
    descs = (_lib.CbkDesc * n)(*[pm.desc() for pm in pms])
    assert L.cbk_gemv_batch_workspace_bytes(n, descs, M) > 0
    outs = [torch.empty(M, pm.K, dtype=torch.float32, device=DEV) for pm in pms]
    rc = L.cbk_gemv_batch(n, descs, (P * n)(*[x.data_ptr() for x in xs]), (ctypes.c_int64 * n)(*[pm.N for pm in pms]),
                          F.dtype_code(torch.float16), M, (P * n)(*[o.data_ptr() for o in outs]),
                          (ctypes.c_int64 * n)(*[pm.K for pm in pms]), F.dtype_code(torch.float32), None, None, 0,
                          torch.cuda.current_stream().cuda_stream)
    assert rc == 0, L.cbk_strerror(rc)
    torch.cuda.synchronize()
    for pm, x, y, o in zip(pms, xs, ys, outs):
        ref = x.double() @ ops.dequant(pm, torch.float32).double().t()
        assert float((y.double() - ref).norm() / ref.norm()) < 1e-5
        assert torch.equal(y, o)
        assert torch.equal(y, ops.gemv(pm, x, out_dtype=torch.float32))


def test_gemv_output_dtypes_bias_and_strided_x():
    case = (F.BLK1632_4, 4, 128, 16)
    K, N = 128, 2048
    raw = make_raw(case, K, N, seed=5)
    pk = oracle_pack(case, raw)
    pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"])
    for dtype in (torch.float16, torch.bfloat16):
        bias = (torch.randn(K) * 0.5).to(dtype)
        xb = acts(4, N + 64, dtype, seed=2)
        x = xb[:, :N]                                       # leading dimension N + 64
        ref = R.forward_ref(W, _np(x), bias=_np(bias))
        y = ops.gemv(pm, x.to(DEV), bias=bias.to(DEV))
        assert y.dtype == dtype and y.shape == (4, K)
        tol = 3e-3 if dtype == torch.bfloat16 else 6e-4     # + one rounding of y to its dtype
        assert rel_fro(_np(y), ref) < tol
        y3 = ops.linear(pm, x.to(DEV).reshape(2, 2, N), bias=bias.to(DEV))
        assert y3.shape == (2, 2, K) and torch.equal(y3.reshape(4, K), y)
    # no col_scale at all
    pm0 = packed_from_oracle(case, pk, None, K, N, DEV)
    x = acts(2, N, torch.float16, seed=8)
    assert rel_fro(_np(ops.gemv(pm0, x.to(DEV), out_dtype=torch.float32)),
                   R.forward_ref(R.dequant(pk, K, N, case[0]), _np(x))) < TOL


@pytest.mark.parametrize("case", [(F.BLK1632_4, 4, 128, 16), (F.BLKC, 3, 128, 10), (F.BLKC, 2, 64, 23),
                                  (F.BLK1632_6, 6, 128, 16)], ids=case_id)
@pytest.mark.parametrize("tiled", [False, True], ids=["rowmajor", "tiled"])
def test_gemv_pruned_columns_contribute_exactly_zero(case, tiled):
    """Restates test_gemv.py:403-455: a column-uniform mask and huge activations at the pruned
    columns, with the zero point on and off the grid.  A pruned column multiplies a literal 0 in
    every kernel.  The matrix-core kernel quantises activations per 128-column chunk relative to
    the chunk's largest magnitude, so (a) activations that keep every chunk maximum unchanged must
    leave the output bit-identical, and (b) 1e4 at every pruned column (which rescales the chunks)
    must still agree with the oracle, which it could not if a pruned weight leaked at all."""
    layout, bits, group, keep = case
    K, N = 256, 5376
    rng = np.random.default_rng(7)
    pat = np.zeros((N // 32, 32), bool)
    idx = np.argsort(rng.random((N // 32, 32)), axis=1)[:, :keep]
    np.put_along_axis(pat, idx, True, axis=1)
    keepm = np.broadcast_to(pat.reshape(1, N), (K, N))
    pruned = torch.from_numpy(~pat.reshape(N))
    nl = (1 << bits) - 1
    q = rng.integers(0, nl + 1, (K, N)).astype(np.uint8)
    scale = (rng.random((K, N // group)) * 0.01 + 1e-3).astype(np.float16)
    for zmode in ("ongrid", "offgrid"):
        zero = rng.integers(0, nl + 1, (K, N // group)).astype(np.float16) if zmode == "ongrid" \
            else np.full((K, N // group), nl + 37, np.float16)
        pk = R.pack_matrix(R.pack_bits(keepm), q, scale, zero, layout, fix_zero=(zmode == "ongrid"), **kw_of(case))
        pm = packed_from_oracle(case, pk, None, K, N, DEV, tiled=tiled)
        W = R.dequant(pk, K, N, layout, **kw_of(case))
        assert (W[:, ~pat.reshape(N)] == 0).all()
        for dtype in (torch.bfloat16, torch.float16):
            x0 = acts(1, N, dtype, seed=1)
            cmax = x0.float().abs().reshape(N // 128, 128).amax(1, keepdim=True).expand(N // 128, 128).reshape(1, N)
            xm = x0.clone(); xm[0, pruned] = (-cmax).to(dtype)[0, pruned]      # chunk maxima unchanged
            xh = x0.clone(); xh[0, pruned] = 1.0e4
            ref = R.forward_ref(W, _np(x0))
            for M in (1, 4):
                y0 = ops.gemv(pm, x0.expand(M, N).contiguous().to(DEV), out_dtype=torch.float32)
                ym = ops.gemv(pm, xm.expand(M, N).contiguous().to(DEV), out_dtype=torch.float32)
                yh = ops.gemv(pm, xh.expand(M, N).contiguous().to(DEV), out_dtype=torch.float32)
                assert torch.equal(y0, ym), f"{case_id(case)} zero={zmode} {dtype} M={M}"
                assert rel_fro(_np(yh)[0], ref[0]) < TOL, f"{case_id(case)} zero={zmode} {dtype} M={M}"
        assert (_np(ops.dequant(pm))[:, ~pat.reshape(N)] == 0).all()


def test_gemv_rows_are_independent_of_batch_and_run_to_run_identical():
    """The reference's determinism gate: M=4 is bit-exact 4 x M=1 (docs/KERNELS.md:151-155)."""
    case = (F.BLK1632_4, 4, 128, 16)
    K, N = 512, 4096
    pm = F.synth_packed(K, N, *case[:3], case[3], seed=11, device=DEV).to_tiled()
    x = acts(4, N, torch.bfloat16, seed=3).to(DEV)
    y4 = ops.gemv(pm, x, out_dtype=torch.float32)
    for i in range(4):
        assert torch.equal(ops.gemv(pm, x[i:i + 1], out_dtype=torch.float32)[0], y4[i])
    assert torch.equal(ops.gemv(pm, x, out_dtype=torch.float32), y4)


@pytest.mark.parametrize("case", [(F.BLK1632_4, 4, 128, 16), (F.DENSE4, 4, 128, 0), (F.BLKC, 2, 128, 16), (F.BLKC, 4, 64, 23)], ids=case_id)
def test_gemv_five_to_eight_rows_equal_single_rows(case):
    """M = 5..8: where the arrangement allows it (group 128, block code streams of whole bytes) and
    the digits of all rows fit in LDS (N = 4096) the weights are streamed once, with two matrix
    instructions per decoded fragment; elsewhere in passes of at most four rows.  Either way row m
    of the result is the M = 1 result of row m bit for bit, also for a gate/up matrix (two scaled
    copies of every activation row), with a bias, and for a tile split into parts."""
    for (K, N, cs_rows) in ((80, 4096, 1), (48, 4096, 2), (16, 14336, 1)):
        pm, W = _fused(case, K, N, cs_rows, (0, 0), seed=K + N + cs_rows, tiled=True)
        bias = acts(1, K, torch.float32, seed=2)[0].to(DEV)
        for M in (5, 6, 7, 8):
            x = acts(M, N, torch.bfloat16, seed=10 * M).to(DEV)
            y = ops.gemv(pm, x, bias=bias, out_dtype=torch.float32)
            assert rel_fro(_np(y), R.forward_ref(W, _np(x)) + _np(bias)[None, :]) < TOL
            for i in range(M):
                assert torch.equal(ops.gemv(pm, x[i:i + 1], bias=bias, out_dtype=torch.float32)[0], y[i]), (K, N, cs_rows, M, i)
            assert torch.equal(ops.gemv(pm, x, bias=bias, out_dtype=torch.float32), y)


@pytest.mark.parametrize("case", [(F.BLK1632_4, 4, 128, 16), (F.DENSE4, 4, 128, 0), (F.BLKC, 3, 128, 10)], ids=case_id)
def test_gemv_rows_longer_than_the_staging_area(case):
    """Rows whose activation digits do not fit in LDS are staged and multiplied in column slabs, the
    weights still streamed once: one row of 65536 columns, eight rows of 14336, 21504 and 28672
    columns (the deltas of eight rows of 28672 columns are 7 KB of LDS by themselves), and
    a matrix with several 16-row tiles per workgroup (more tiles than reduction slots).  Checked
    against float64 on the dequantised weights and, bit for bit, against the single-row results."""
    for (K, N, Ms) in ((16, 65536, (1, 2)), (48, 21504, (8, 3)), (8208, 14336, (8,)), (24, 28672, (8, 5))):
        pm = F.synth_packed(K, N, case[0], case[1], case[2], case[3], seed=K + N, device=DEV).to_tiled()
        W = ops.dequant(pm, torch.float32).double()
        for M in Ms:
            x = acts(M, N, torch.bfloat16, seed=3 * M).to(DEV)
            y = ops.gemv(pm, x, out_dtype=torch.float32)
            ref = x.double() @ W.t()
            assert float((y.double() - ref).abs().max() / ref.abs().max()) < 2e-5, (K, N, M)
            for i in range(M):
                assert torch.equal(ops.gemv(pm, x[i:i + 1], out_dtype=torch.float32)[0], y[i]), (K, N, M, i)
            # without room for the part sums the same rows are staged slab by slab in every
            # workgroup instead of being split over the workgroups by columns: same bits
            small = torch.empty(256, dtype=torch.uint8, device=DEV)
            assert torch.equal(ops.gemv(pm, x, out_dtype=torch.float32, workspace=small), y), (K, N, M)
    # a gate/up matrix stages two scaled copies of every activation row: four rows of 5376 columns
    # are eight staged rows, more than the staging area holds at once
    K, N = 64, 5376
    pm = F.synth_packed(K, N, case[0], case[1], case[2], case[3], seed=5, device=DEV)
    cs = (torch.rand(2, N, generator=torch.Generator().manual_seed(9)) + 0.5).half().to(DEV)
    pm = F.from_arrays(pm.array("data"), pm.array("scale"), pm.array("zero"), cs, K, N, case[0], case[1], case[2],
                       case[3] or None, device=DEV).to_tiled()
    W = ops.dequant(pm, torch.float32).double()
    for M in (4, 7):
        x = acts(M, N, torch.bfloat16, seed=M).to(DEV)
        y = ops.gemv(pm, x, out_dtype=torch.float32)
        ref = x.double() @ W.t()
        assert float((y.double() - ref).abs().max() / ref.abs().max()) < 2e-5, (K, N, M)
        for i in range(M):
            assert torch.equal(ops.gemv(pm, x[i:i + 1], out_dtype=torch.float32)[0], y[i]), (K, N, M, i)


@pytest.mark.parametrize("case", [(F.BLK1632_4, 4, 128, 16), (F.DENSE4, 4, 128, 0), (F.BLKC, 2, 128, 16), (F.DENSEB, 2, 128, 0)], ids=case_id)
def test_gemv_long_rows_split_by_columns(case):
    """Two to eight activation rows of rows too long for the staging area, with room for the part
    sums (cbk_workspace_bytes says how much): every workgroup takes one column slab of a range of
    tiles and a second kernel adds the parts.  Bias, 16-bit outputs, a gate/up matrix (two col_scale
    vectors by row parity), a row count off the tile, a column count off the 512-column step; row m
    of the result is the M = 1 result bit for bit, and so is the result without a workspace."""
    small = torch.empty(256, dtype=torch.uint8, device=DEV)
    for (K, N, cs_rows, Ms) in ((72, 14336, 1, (8, 5, 4)), (40, 14336, 2, (4, 3)), (16, 28800, 1, (2, 7)), (4112, 8192, 1, (8,))):
        pm, W = _fused(case, K, N, cs_rows, (0, 0), seed=K + N + cs_rows, tiled=True)
        for dt in (torch.float32, torch.bfloat16):
            bias = acts(1, K, dt, seed=2)[0].to(DEV)
            for M in Ms:
                x = acts(M, N, torch.bfloat16, seed=10 * M).to(DEV)
                if M * cs_rows * 3 * N > 140 * 1024:
                    assert _lib.lib().cbk_workspace_bytes(ctypes.byref(pm.desc()), M) >= (K + 15) // 16 * 16 * M * cs_rows * 4
                y = ops.gemv(pm, x, bias=bias, out_dtype=dt)
                if dt == torch.float32:
                    assert rel_fro(_np(y), R.forward_ref(W, _np(x)) + _np(bias)[None, :]) < TOL, (K, N, cs_rows, M)
                for i in range(M):
                    assert torch.equal(ops.gemv(pm, x[i:i + 1], bias=bias, out_dtype=dt)[0], y[i]), (K, N, cs_rows, M, i)
                assert torch.equal(ops.gemv(pm, x, bias=bias, out_dtype=dt, workspace=small), y), (K, N, cs_rows, M)
                assert torch.equal(ops.gemv(pm, x, bias=bias, out_dtype=dt), y)


@pytest.mark.parametrize("case", [(F.BLK1632_4, 4, 128, 16), (F.BLKC, 3, 64, 10), (F.DENSE4, 4, 128, 0)], ids=case_id)
def test_linear_ragged_and_extreme_shapes(case):
    """One row, one chunk, row counts off the 16-row and 256-row tiles, column counts off the
    512-column step, and a row too long for the decode kernel's activation staging: every
    activation count from the decode kernel to the split prefill kernel."""
    for (K, N) in ((1, 128), (17, 384), (33, 640), (257, 128), (300, 1152), (4, 28672)):
        raw = make_raw(case, K, N, seed=K + N)
        pk = oracle_pack(case, raw)
        W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
        for tiled in (False, True):
            pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
            for M in (1, 4, 7, 17, 129, 300):
                x = acts(M, N, torch.float16, seed=M)
                ref = R.forward_ref(W, _np(x))
                err = rel_fro(_np(ops.linear(pm, x.to(DEV), out_dtype=torch.float32)), ref)
                assert err < TOL, f"{case_id(case)} {K}x{N} tiled={tiled} M={M}: {err}"


# ------------------------------------------------------------------ row-fused matrices
FUSED_CASES = [(F.BLK1632_4, 4, 128, 16), (F.BLKC, 3, 128, 10), (F.BLKC, 2, 64, 23), (F.DENSE4, 4, 128, 0),
               (F.BLK1632_6, 6, 128, 16)]


def _fused(case, K, N, cs_rows, splits, seed, tiled):
    raw = make_raw(case, K, N, seed=seed)
    pk = oracle_pack(case, raw)
    rng = np.random.default_rng(seed)
    cs = (rng.random((cs_rows, N)) * 1.5 + 0.5).astype(np.float16)
    pm = packed_from_oracle(case, pk, cs, K, N, DEV, cs_splits=splits, tiled=tiled)
    W = R.dequant(pk, K, N, case[0], col_scale=cs, cs_splits=splits, **kw_of(case))
    return pm, W


@pytest.mark.parametrize("tiled", [False, True], ids=["rowmajor", "tiled"])
@pytest.mark.parametrize("case", FUSED_CASES, ids=case_id)
def test_gemv_fused_col_scale_rows(case, tiled):
    """Fused q|k|v (three col_scale vectors by row range) and gate/up (two by row parity):
    docs/FORMAT.md:126-151, cobalt_format.h:77-99.  Ranges on 16-row tiles go through the MFMA
    kernel range by range; the (40, 8) split does not and takes the row kernel."""
    K, N = 208, 1024
    for cs_rows, splits in ((2, (0, 0)), (3, (96, 48)), (3, (208, 0)), (3, (40, 8))):
        pm, W = _fused(case, K, N, cs_rows, splits, seed=K + cs_rows + splits[0], tiled=tiled)
        for M in (1, 2, 3, 4, 5, 8):
            for dtype in (torch.float16, torch.bfloat16):
                x = acts(M, N, dtype, seed=M)
                bias = acts(1, K, torch.float32, seed=9)[0]
                ref = R.forward_ref(W, _np(x)) + _np(bias)[None, :]
                y = ops.gemv(pm, x.to(DEV), bias=bias.to(DEV), out_dtype=torch.float32)
                err = rel_fro(_np(y), ref)
                assert err < TOL, f"{case_id(case)} cs_rows={cs_rows} splits={splits} M={M} {dtype}: {err}"


def test_gemv_fused_rows_equal_their_unfused_parts_bit_for_bit():
    """A q|k|v matrix gives, row for row, the bits of its three parts run on their own, and a
    gate/up matrix the bits of the even-row and odd-row matrices (same sums, same order; at a
    size where the fused and the separate launches cut the columns into the same parts)."""
    case = (F.BLK1632_4, 4, 128, 16)
    K, N = 256, 4096
    raw = make_raw(case, K, N, seed=77)
    pk = oracle_pack(case, raw)
    rng = np.random.default_rng(5)
    x = acts(2, N, torch.float16, seed=4).to(DEV)
    cs3 = (rng.random((3, N)) * 1.5 + 0.5).astype(np.float16)
    fused = packed_from_oracle(case, pk, cs3, K, N, DEV, cs_splits=(128, 64), tiled=True)
    y = ops.gemv(fused, x, out_dtype=torch.float32)
    for r, (lo, hi) in enumerate(((0, 128), (128, 192), (192, 256))):
        sub = {k: (v[lo:hi] if k != "row_off" else v) for k, v in pk.items() if k in ("scale", "zero")}
        stride = R.row_stride(case[0], N)
        sub["data"] = np.concatenate([pk["data"][lo * stride: hi * stride], np.zeros(64, np.uint8)])
        part = packed_from_oracle(case, sub, cs3[r], hi - lo, N, DEV, tiled=True)
        assert torch.equal(ops.gemv(part, x, out_dtype=torch.float32), y[:, lo:hi])
    cs2 = cs3[:2]
    gu = packed_from_oracle(case, pk, cs2, K, N, DEV, tiled=True)
    y2 = ops.gemv(gu, x, out_dtype=torch.float32)
    whole = [ops.gemv(packed_from_oracle(case, pk, cs2[c], K, N, DEV, tiled=True), x, out_dtype=torch.float32)
             for c in range(2)]
    assert torch.equal(y2[:, 0::2], whole[0][:, 0::2]) and torch.equal(y2[:, 1::2], whole[1][:, 1::2])


@pytest.mark.parametrize("case", FUSED_CASES[:2] + FUSED_CASES[4:], ids=case_id)
def test_gemm_fused_col_scale_rows(case):
    """Prefill on fused matrices: q|k|v ranges run the 256 x 256 kernel range by range, gate/up
    (row parity) as workgroups of one parity; ranges off the 16-row grid the 128 x 128 kernel."""
    K, N = 640, 1024
    # (40, 24): ranges off the 16-row grid, which only the 128 x 128 fallback kernel takes
    for cs_rows, splits in ((3, (256, 128)), (3, (48, 16)), (3, (40, 24)), (2, (0, 0))):
        pm, W = _fused(case, K, N, cs_rows, splits, seed=K + cs_rows + splits[0], tiled=splits[0] % 16 == 0)
        for M, dtype in ((300, torch.bfloat16), (129, torch.float16), (64, torch.float16)):
            x = acts(M, N, dtype, seed=M)
            bias = acts(1, K, torch.float32, seed=9)[0]
            ref = R.forward_ref(W, _np(x)) + _np(bias)[None, :]
            y = ops.gemm(pm, x.to(DEV), bias=bias.to(DEV), out_dtype=torch.float32)
            err = rel_fro(_np(y), ref)
            assert err < TOL, f"{case_id(case)} cs_rows={cs_rows} splits={splits} M={M}: {err}"


def _gated_ref(t, act):
    """act(gate) * up in float64 from t[.., 2i] / t[.., 2i+1]: the tanh-GELU and SiLU formulas of
    cobalt_gemm.cuh:216-220; the reference checks its epilogue against
    torch.nn.functional.gelu(gate, approximate="tanh") * up (test_gemm.py:204-209)."""
    g, u = t[:, 0::2].astype(np.float64), t[:, 1::2].astype(np.float64)
    if act == "gelu_tanh":
        a = 0.5 * g * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (g + 0.044715 * g ** 3)))
    else:
        a = g / (1.0 + np.exp(-g))
    return a * u


@pytest.mark.parametrize("act", ["gelu_tanh", "silu"])
@pytest.mark.parametrize("case", FUSED_CASES[:2], ids=case_id)
def test_linear_act_gated_epilogue(case, act):
    """Gate/up matrix through cbk_linear_act at decode, mid and prefill row counts.  float32 and
    f16 outputs meet the layer tolerance; a bf16 output carries its own 2^-9 rounding (and, above
    128 rows, that of the stored gate and up values), so it is held to 4e-3."""
    K, N = 640, 1024
    pm, W = _fused(case, K, N, 2, (0, 0), seed=K + 5, tiled=True)
    bias = acts(1, K, torch.float16, seed=11)[0]
    for M, dtype, odt, with_bias in ((1, torch.float16, torch.float32, False), (4, torch.bfloat16, torch.bfloat16, False),
                                     (64, torch.float16, torch.float16, True), (129, torch.float16, torch.float32, True),
                                     (300, torch.bfloat16, torch.bfloat16, False), (300, torch.float16, torch.float16, False)):
        x = acts(M, N, dtype, seed=M + 1)
        b = bias.to(odt) if with_bias else None
        t = R.forward_ref(W, _np(x))
        if with_bias:
            t = t + _np(b)[None, :]
        ref = _gated_ref(t, act)
        y = ops.linear_act(pm, x.to(DEV), act, bias=None if b is None else b.to(DEV), out_dtype=odt)
        assert y.shape == (M, K // 2) and y.dtype == odt
        err = rel_fro(_np(y), ref)
        tol = 4e-3 if odt == torch.bfloat16 else TOL
        assert err < tol, f"{case_id(case)} {act} M={M} {dtype}->{odt}: {err}"
    # the first half of an MLP equals the two-step form on the same kernels
    x = acts(8, N, torch.float16, seed=3).to(DEV)
    t = ops.linear(pm, x, out_dtype=torch.float32)
    two = (torch.nn.functional.gelu(t[:, 0::2], approximate="tanh") if act == "gelu_tanh"
           else torch.nn.functional.silu(t[:, 0::2])) * t[:, 1::2]
    one = ops.linear_act(pm, x, act, out_dtype=torch.float32)
    assert rel_fro(_np(one), _np(two)) < 1e-6


@pytest.mark.parametrize("act", ["gelu_tanh", "silu"])
def test_linear_act_for_nine_to_128_rows(act):
    """Between 9 and 128 activation rows (the 64- and 128-token tiles of the matrix kernel, a float32
    intermediate and one rounding of the result).  Row counts on and off the tile sizes, more than
    one row tile with a ragged last one (K = 2 * 331), with and without bias, every output type,
    both byte orders, and a y with a leading dimension beyond K / 2; against the oracle's float64
    gate/up product."""
    for case in (FUSED_CASES[0], (F.BLKC, 3, 64, 10), (F.DENSE4, 4, 128, 0)):
        K, N = 662, 1152
        for tiled in (False, True):
            pm, W = _fused(case, K, N, 2, (0, 0), seed=K + 9, tiled=tiled)
            bias = acts(1, K, torch.float32, seed=13)[0]
            for M, dtype, odt, with_bias in ((9, torch.float16, torch.float32, True), (40, torch.bfloat16, torch.bfloat16, False),
                                             (64, torch.float16, torch.float16, True), (65, torch.bfloat16, torch.float32, False),
                                             (128, torch.float16, torch.float32, True)):
                x = acts(M, N, dtype, seed=M + 2)
                b = bias.to(odt) if with_bias else None
                t = R.forward_ref(W, _np(x))
                if with_bias:
                    t = t + _np(b)[None, :]
                ref = _gated_ref(t, act)
                y = ops.linear_act(pm, x.to(DEV), act, bias=None if b is None else b.to(DEV), out_dtype=odt)
                assert y.shape == (M, K // 2) and y.dtype == odt
                err = rel_fro(_np(y), ref)
                tol = 4e-3 if odt == torch.bfloat16 else TOL
                assert err < tol, f"{case_id(case)} {act} tiled={tiled} M={M} {dtype}->{odt}: {err}"
                assert torch.equal(ops.linear_act(pm, x.to(DEV), act, bias=None if b is None else b.to(DEV), out_dtype=odt), y)
    # through the C ABI into a y with a leading dimension larger than K / 2: the columns beyond stay untouched
    pm, W = _fused(FUSED_CASES[0], 256, 512, 2, (0, 0), seed=3, tiled=True)
    M, ldy = 20, 136
    x = acts(M, 512, torch.float16, seed=5).to(DEV)
    y = torch.full((M, ldy), -7.0, dtype=torch.float32, device=DEV)
    L, d = _lib.lib(), pm.desc()
    need = L.cbk_linear_act_workspace_bytes(ctypes.byref(d), M, F.F32)
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    rc = L.cbk_linear_act(ctypes.byref(d), x.data_ptr(), F.F16, M, 512, y.data_ptr(), F.F32, ldy, None,
                          _lib.ACT_CODE[act], ws.data_ptr(), need, None)
    assert rc == 0
    torch.cuda.synchronize()
    ref = _gated_ref(R.forward_ref(W, _np(x)), act)
    assert rel_fro(_np(y[:, :128]), ref) < TOL and bool((y[:, 128:] == -7.0).all())


def test_linear_act_rejects_bad_calls():
    case = FUSED_CASES[0]
    pm, _ = _fused(case, 64, 256, 2, (0, 0), seed=1, tiled=False)
    x = acts(2, 256, torch.float16, seed=1).to(DEV)
    with pytest.raises(ValueError):
        ops.linear_act(pm, x, "relu")
    L, d = _lib.lib(), pm.desc()
    y = torch.empty(2, 32, dtype=torch.float16, device=DEV)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
    args = lambda act, wsb, ldy: (ctypes.byref(d), x.data_ptr(), 1, 2, 256, y.data_ptr(), 1, ldy, None, act,
                                  ws.data_ptr(), wsb, None)
    assert L.cbk_linear_act(*args(7, ws.numel(), 32)) == -8           # unknown activation
    assert L.cbk_linear_act(*args(0, 16, 32)) == -6                   # workspace too small
    assert L.cbk_linear_act(*args(0, ws.numel(), 16)) == -3           # ldy below K / 2
    assert L.cbk_linear_act(*args(0, ws.numel(), 32)) == 0
    torch.cuda.synchronize()


# ------------------------------------------------------------------ prefill GEMM
@pytest.mark.parametrize("tiled", [False, True], ids=["rowmajor", "tiled"])
@pytest.mark.parametrize("case", FIXED_CASES, ids=case_id)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_gemm_matches_oracle(case, dtype, tiled):
    K, N = 328, 1024
    raw = make_raw(case, K, N, seed=77 + case[0])
    pk = oracle_pack(case, raw)
    pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
    for M in (16, 100, 512):                                # the reference's M set (test_gemm.py:162-195)
        x = acts(M, N, dtype, seed=M)
        ref = R.forward_ref(W, _np(x))
        y = ops.gemm(pm, x.to(DEV), out_dtype=torch.float32)
        err = rel_fro(_np(y), ref)
        assert err < TOL, f"{case_id(case)} M={M}: {err}"


@pytest.mark.parametrize("cs_rows", [1, 2, 3])
def test_gemm_more_tiles_than_one_round_over_the_cus(cs_rows):
    """260 tiles of 256 x 256 (more than the 256 CUs take at once), ragged K and M, plain and
    row-fused: checked against the bit-exact dequantised weights (float64 matmul on the device)
    and for run-to-run identical results."""
    K, N, M = 256 * 130 - 24, 2048, 500                             # 2 x 130 = 260 tiles
    mk = lambda k, seed: F.synth_packed(k, N, F.BLK1632_4, 4, 128, 16, seed=seed, device=DEV)
    if cs_rows == 1:
        pm = mk(K, 1)
    elif cs_rows == 2:
        pm = F.fuse_rows([mk(K // 2, 2), mk(K // 2, 3)], interleave=True)
    else:
        pm = F.fuse_rows([mk(256 * 40, 4), mk(256 * 30, 5), mk(K - 256 * 70, 6)])
    assert pm.cs_rows == cs_rows and pm.K == K
    pm = pm.to_tiled()
    W = ops.dequant(pm, torch.float32).double()
    x = acts(M, N, torch.float16, seed=5).to(DEV)
    bias = torch.randn(K, generator=torch.Generator().manual_seed(1)).to(DEV)
    ref = x.double() @ W.T + bias.double()
    y = ops.gemm(pm, x, bias=bias, out_dtype=torch.float32)
    err = float((y.double() - ref).norm() / ref.norm())
    assert err < TOL, err
    assert torch.equal(ops.gemm(pm, x, bias=bias, out_dtype=torch.float32), y)
    yb = ops.gemm(pm, x.to(torch.bfloat16), out_dtype=torch.bfloat16)
    refb = x.to(torch.bfloat16).double() @ W.T
    assert float((yb.double() - refb).norm() / refb.norm()) < 4e-3


@pytest.mark.parametrize("case", [(F.BLK1632_4, 4, 128, 16), (F.DENSE4, 4, 128, 0), (F.BLKC, 3, 64, 23)], ids=case_id)
def test_gemm_odd_chunk_count_and_ragged_tiles(case):
    """N = 3 chunks of 128 (the kernel works on chunk pairs and pads), K and M not multiples of
    the 256 x 256 tile, every output dtype, strided activations and outputs."""
    K, N, M = 264, 384, 300
    raw = make_raw(case, K, N, seed=31)
    pk = oracle_pack(case, raw)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
    x = acts(M, N, torch.float16, seed=8)
    ref = R.forward_ref(W, _np(x))
    for tiled in (False, True):
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
        for odt in (torch.float32, torch.float16, torch.bfloat16):
            y = ops.gemm(pm, x.to(DEV), out_dtype=odt)
            assert y.dtype == odt and rel_fro(_np(y), ref) < (TOL if odt != torch.bfloat16 else 3e-3)
        xs = torch.zeros(M, N + 8, dtype=torch.float16); xs[:, :N] = x
        assert rel_fro(_np(ops.gemm(pm, xs.to(DEV)[:, :N], out_dtype=torch.float32)), ref) < TOL
        for m in (1, 37, 64, 65):                               # the 64-token tile, ragged, and just past it
            y = ops.gemm(pm, x[:m].to(DEV), out_dtype=torch.float32)
            assert rel_fro(_np(y), ref[:m]) < TOL, (m, tiled)


@pytest.mark.parametrize("case", ALL_MFMA_CASES, ids=case_id)
def test_gemm_every_kernel_configuration(case):
    """Every instantiation of the prefill kernel's byte-permute decoder (code width x survivors
    per block x group size, bitmap and dense), both byte orders, five 128-column chunks so that
    code bits straddle 16-byte units at every skew, run twice."""
    K, N, M = 272, 640, 260
    raw = make_raw(case, K, N, seed=5 * case[1] + case[3])
    pk = oracle_pack(case, raw)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
    x = acts(M, N, torch.bfloat16, seed=3)
    ref = R.forward_ref(W, _np(x))
    for tiled in (False, True):
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
        y = ops.gemm(pm, x.to(DEV), out_dtype=torch.float32)
        err = rel_fro(_np(y), ref)
        assert err < TOL, f"{case_id(case)} tiled={tiled}: {err}"
        assert torch.equal(y, ops.gemm(pm, x.to(DEV), out_dtype=torch.float32))
        y64 = ops.gemm(pm, x[:50].to(DEV), out_dtype=torch.float32)     # the 64-token instantiation
        assert rel_fro(_np(y64), ref[:50]) < TOL, f"{case_id(case)} tiled={tiled} M=50"
        assert torch.equal(y64, ops.gemm(pm, x[:50].to(DEV), out_dtype=torch.float32))


def test_gemm_bias_dtype_and_prune_zero():
    case = (F.BLK1632_4, 4, 128, 16)
    K, N, M = 256, 2048, 300
    raw = make_raw(case, K, N, seed=4)
    pk = oracle_pack(case, raw)
    pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV)
    W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"])
    bias = torch.randn(K).to(torch.bfloat16)
    x = acts(M, N, torch.bfloat16, seed=6)
    y = ops.linear(pm, x.to(DEV), bias=bias.to(DEV))
    assert y.dtype == torch.bfloat16 and rel_fro(_np(y), R.forward_ref(W, _np(x), bias=_np(bias))) < 3e-3
    # prune-zero through the tile (test_gemm.py:223-255): same mask in every row
    pat = np.tile(np.r_[np.ones(16, bool), np.zeros(16, bool)], N // 32)
    rng = np.random.default_rng(1)
    q = rng.integers(0, 16, (K, N)).astype(np.uint8)
    pk = R.pack_matrix(R.pack_bits(np.broadcast_to(pat, (K, N))), q, raw["scale"], np.full((K, N // 128), 52, np.float16),
                       R.BLK1632_4, fix_zero=False)
    pm = packed_from_oracle(case, pk, None, K, N, DEV)
    x0 = acts(M, N, torch.float16, seed=9)
    xh = x0.clone(); xh[:, torch.from_numpy(~pat)] = 1.0e4
    assert torch.equal(ops.gemm(pm, x0.to(DEV), out_dtype=torch.float32), ops.gemm(pm, xh.to(DEV), out_dtype=torch.float32))


def test_gemm_activations_beyond_fp16_range():
    """bf16 activations (and fp16 ones under a column scale) whose products leave fp16's range:
    the prefill kernels feed the fp16 matrix pipe, so such a token is scaled by a power of two on
    the way in and back on the way out.  Tokens 1, 70 and 299 carry values up to 1e36 / 1e9 / 7e4;
    every token, large or not, meets the float64 product to the usual tolerance, and the small
    tokens give the same bits as in a call without the large ones.  Token 200 of the bf16 case holds
    one value of 1.6e38, half of the largest finite bf16, so that its product with a column scale of
    up to 2 is still a finite float32 at the very top of the range."""
    case = (F.BLK1632_4, 4, 128, 16)
    K, N, M = 512, 1024, 300
    for cs_rows, splits in ((1, (0, 0)), (2, (0, 0)), (3, (256, 128)), (3, (40, 24))):
        pm, W = _fused(case, K, N, cs_rows, splits, seed=31 + cs_rows + splits[0], tiled=splits[0] % 16 == 0)
        for dtype, big in ((torch.bfloat16, (1.0e36, 1.0e9, 7.0e4)), (torch.float16, (6.5e4, 4.0e4, 3.3e4))):
            x = acts(M, N, dtype, seed=M + cs_rows)
            small = ops.gemm(pm, x.to(DEV), out_dtype=torch.float32)
            xb = x.clone()
            for tok, top in zip((1, 70, 299), big):
                xb[tok] = (x[tok].float() * (top / float(x[tok].float().abs().max()))).to(dtype)
                xb[tok, 5] = top
            if dtype == torch.bfloat16:
                xb[200, 5] = 1.6e38
            y = ops.gemm(pm, xb.to(DEV), out_dtype=torch.float32)
            assert bool(torch.isfinite(y).all())
            ref = R.forward_ref(W, _np(xb))
            for tok in (0, 1, 70, 150, 200, 299):
                err = rel_fro(_np(y[tok:tok + 1]), ref[tok:tok + 1])
                assert err < TOL, f"cs_rows={cs_rows} splits={splits} {dtype} token {tok}: {err}"
            keep = [t for t in range(M) if t not in (1, 70, 200, 299)]
            assert torch.equal(y[keep], small[keep])
            y64 = ops.gemm(pm, xb[:40].to(DEV), out_dtype=torch.float32)          # the 64-token instantiation
            small64 = ops.gemm(pm, x[:40].to(DEV), out_dtype=torch.float32)
            assert rel_fro(_np(y64[1:2]), ref[1:2]) < TOL and torch.equal(y64[2:], small64[2:])


# ------------------------------------------------------------------ the module seam
def test_cobalt_linear_forward_matches_reference_module_math():
    K, N = 256, 1024
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=2, block=32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    bias = torch.randn(K).half()
    lin = CobaltLinear.from_raw(t(raw["mask"]), t(raw["q"]), t(raw["scale"]), t(raw["zero"]), t(raw["col_scale"]),
                                bias=bias).to(DEV)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.BLK1632_4)
    W = R.dequant(pk, K, N, R.BLK1632_4, col_scale=raw["col_scale"])
    assert np.array_equal(_np(lin.dequantize()), W)
    for tiled in (False, True):
        if tiled:
            lin.to_device_order()
            assert lin.packed().tiled and np.array_equal(_np(lin.dequantize()), W)
        for shape in ((1, N), (3, 5, N), (2, 200, N)):
            x = (torch.randn(*shape) * 1.0).half()
            y = lin(x.to(DEV))
            assert y.shape == shape[:-1] + (K,) and y.dtype == torch.float16
            ref = R.forward_ref(W, _np(x).reshape(-1, N), bias=_np(bias)).reshape(y.shape)
            assert rel_fro(_np(y), ref) < 6e-4


def test_from_linear_single_layer_configuration():
    """The reference's single-layer case: W 4096x4096 ~ N(0, 0.02) with 1 % of the columns
    scaled by 10, calibration activations 128x4096 ~ N(0, 1), column-balanced mask at sparsity
    0.5, OBS, 4-bit RTN group 128, x 1x4096 fp16.  Compressed on the GPU by the product, then
    the HIP forward is compared with the C oracle's forward over the packed bytes."""
    from oracle import cbk_ref_c as RC
    g = torch.Generator().manual_seed(0)
    K = N = 4096
    W = torch.randn(K, N, generator=g) * 0.02
    W[:, torch.randperm(N, generator=g)[:41]] *= 10
    X = torch.randn(128, N, generator=g)
    lin = torch.nn.Linear(N, K, bias=False)
    lin.weight.data.copy_(W)
    m = CobaltLinear.from_linear(lin.to(DEV), X_cal=X.to(DEV), sparsity=0.5, bits=4, group=128)
    pm = m.packed()
    assert pm.layout == F.BLK1632_4 and abs(pm.bpw() - 3.1875) < 1e-9
    cpu = pm.to("cpu")
    pk = dict(data=cpu.array("data").numpy(), scale=cpu.array("scale").numpy().reshape(K, -1),
              zero=cpu.array("zero").numpy().reshape(K, -1))
    cs = cpu.array("col_scale").numpy().reshape(1, N)
    x = torch.randn(1, N, generator=g).half()
    ref = RC.forward(pk, K, N, pm.layout, x.float().numpy(), col_scale=cs)
    for tiled in (False, True):
        if tiled:
            m.to_device_order()
        y = ops.linear(m._pm(), x.to(DEV), out_dtype=torch.float32)
        assert rel_fro(_np(y), ref) < TOL
    # the compressed layer still computes roughly what the dense one did on calibration-like inputs
    dense = (x.float() @ W.T).numpy()
    assert rel_fro(ref, dense) < 0.35


# ------------------------------------------------------------------ full-size properties
@pytest.mark.parametrize("K,N,case", [(14336, 4096, (F.BLK1632_4, 4, 128, 16)), (4096, 14336, (F.BLKC, 3, 128, 10)),
                                      (5376, 21504, (F.BLKC, 2, 64, 23))], ids=["mistral-gate", "mistral-down-b3", "gemma-down-b2g64"])
def test_full_size_properties(K, N, case):
    """Shapes of the benchmark configurations, where the CPU oracle is too slow for a full
    comparison: linearity in x, agreement between the decode and the prefill kernel, agreement
    of both with the dequantised dense weight on sampled rows (oracle on 32 rows)."""
    pm_rm = F.synth_packed(K, N, case[0], case[1], case[2], case[3] or None, seed=K % 97, device=DEV)
    pm = pm_rm.to_tiled()
    x = acts(2, N, torch.bfloat16, seed=5).to(DEV)
    y = ops.gemv(pm, x, out_dtype=torch.float32)
    # linearity: activations scaled by 2 and rows swapped
    y2 = ops.gemv(pm, (x * 2).flip(0), out_dtype=torch.float32)
    assert torch.equal(y2.flip(0), y * 2)
    # decode kernel vs prefill kernel on the same inputs
    yg = ops.gemm(pm, x, out_dtype=torch.float32)
    assert rel_fro(_np(yg), _np(y)) < TOL
    # sampled rows against the oracle
    rows = np.linspace(0, K - 1, 32).astype(int)
    assert torch.equal(ops.gemv(pm_rm, x, out_dtype=torch.float32), y)          # both byte orders, same sums
    pk = dict(data=pm_rm.array("data").cpu().numpy(), scale=pm_rm.array("scale").cpu().numpy().reshape(K, -1),
              zero=pm_rm.array("zero").cpu().numpy().reshape(K, -1), row_off=None)
    stride = R.row_stride(case[0], N, case[1], case[2], case[3] or None)
    sub = dict(data=np.concatenate([pk["data"][r * stride:(r + 1) * stride] for r in rows] + [np.zeros(64, np.uint8)]),
               scale=pk["scale"][rows], zero=pk["zero"][rows], row_off=None)
    Wsub = R.dequant(sub, len(rows), N, case[0], col_scale=pm_rm.array("col_scale").cpu().numpy(), **kw_of(case))
    Wg = _np(ops.dequant(pm, torch.float32))
    assert np.array_equal(Wg[rows], Wsub)
    assert rel_fro(_np(y)[:, rows], R.forward_ref(Wsub, _np(x))) < TOL


@pytest.mark.parametrize("K,N", [(21504, 5376), (5376, 21504)], ids=["gemma-gate", "gemma-down"])
@pytest.mark.parametrize("M,case", [(2048, (F.BLK1632_4, 4, 128, 16)), (4096, (F.BLK1632_4, 4, 128, 16)),
                                    (4096, (F.BLKC, 3, 64, 10))], ids=["m2048-b4g128", "m4096-b4g128", "m4096-b3g64k10"])
def test_prefill_at_the_benchmark_sizes(K, N, M, case):
    """The prefill launches bench.py times (Gemma-3-27B MLP shapes, bf16, M = 2048 and the grid's
    M = 4096: whole rounds of 256 x 256 tiles and the split column range of the long rows), where
    the CPU oracle is too slow: the dequantised rows are bit-exact against the oracle on a
    sample, and sampled output rows match a float64 matmul with the dequantised weights."""
    pm_rm = F.synth_packed(K, N, case[0], case[1], case[2], case[3] or None, seed=11, device=DEV)
    pm = pm_rm.to_tiled()
    x = acts(M, N, torch.bfloat16, seed=M).to(DEV)
    y = ops.gemm(pm, x, out_dtype=torch.float32)
    assert torch.equal(ops.gemm(pm, x, out_dtype=torch.float32), y)              # run-to-run identical
    stride = R.row_stride(case[0], N, case[1], case[2], case[3] or None)
    data = pm_rm.array("data").cpu().numpy()
    scale = pm_rm.array("scale").cpu().numpy().reshape(K, -1)
    zero = pm_rm.array("zero").cpu().numpy().reshape(K, -1)
    cs = pm_rm.array("col_scale").cpu().numpy()
    num = den = 0.0
    for r0 in (0, (K // 2 // 16) * 16 + 3, K - 64):
        W = ops.dequant(pm, torch.float32, row0=r0, nrows=64)
        rows = np.arange(r0, r0 + 64, 9)
        sub = dict(data=np.concatenate([data[r * stride:(r + 1) * stride] for r in rows] + [np.zeros(64, np.uint8)]),
                   scale=scale[rows], zero=zero[rows], row_off=None)
        assert np.array_equal(_np(W)[rows - r0], R.dequant(sub, len(rows), N, case[0], col_scale=cs, **kw_of(case)))
        ref = x.double() @ W.double().T
        num += float((y[:, r0:r0 + 64].double() - ref).pow(2).sum())
        den += float(ref.pow(2).sum())
    assert (num / den) ** 0.5 < TOL, (num / den) ** 0.5
    yb = ops.gemm(pm, x)                                                        # the timed call: output in x's type
    assert float((yb.double() - y.double()).norm() / y.double().norm()) < 4e-3   # bf16 rounding of the output
