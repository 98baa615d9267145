"""Seeded random sweep over shapes, layouts, byte orders, activation counts and types: every call
of the layer (`cbk_linear`: decode kernel up to eight rows, tile kernels above) and of the gated
MLP's first half (`cbk_linear_act`) against the CPU oracle's dequantised weights in float64.
The fixed cases elsewhere pin known corners; this sweep is there for the ones nobody listed
(row counts off the 16-row tiles, column counts off the 512-column step, rows longer than the
decode kernel's staging area, token counts off the 64- and 256-token tiles)."""
import numpy as np
import pytest
import torch

from oracle import cbk_ref as R
from cobalt_amd import format as F
from cobalt_amd import ops
from helpers import FIXED_CASES, SPARSE_CASES, acts, case_id, kw_of, make_raw, oracle_pack, packed_from_oracle, rel_fro

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 1e-3


def _np(t):
    return t.detach().float().cpu().numpy()


def _draws(seed, n):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        K = int(rng.choice([1, 7, 16, 17, 31, 48, 100, 255, 256, 257, 300, 513]))
        N = 128 * int(rng.choice([1, 2, 3, 4, 5, 8, 11, 16, 33, 42, 113]))
        M = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 16, 17, 63, 64, 65, 128, 129, 255, 257, 300]))
        out.append((K, N, M, bool(rng.integers(2)), bool(rng.integers(2)), int(rng.integers(1 << 30))))
    return out


@pytest.mark.parametrize("case", FIXED_CASES + SPARSE_CASES, ids=case_id)
def test_linear_random_shapes(case):
    for (K, N, M, tiled, half, seed) in _draws(1000 + FIXED_CASES.index(case) if case in FIXED_CASES else 77, 6):
        if case in SPARSE_CASES:
            tiled = False
        raw = make_raw(case, K, N, seed=seed % 1000)
        pk = oracle_pack(case, raw)
        W = R.dequant(pk, K, N, case[0], col_scale=raw["col_scale"], **kw_of(case))
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
        dt = torch.float16 if half else torch.bfloat16
        x = acts(M, N, dt, seed=seed % 97)
        ref = R.forward_ref(W, _np(x))
        y = ops.linear(pm, x.to(DEV), out_dtype=torch.float32)
        err = rel_fro(_np(y), ref)
        assert err < TOL, f"{case_id(case)} {K}x{N} M={M} tiled={tiled} {dt}: {err}"


@pytest.mark.parametrize("case", [(F.BLK1632_4, 4, 128, 16), (F.BLKC, 3, 64, 10), (F.DENSE4, 4, 128, 0)], ids=case_id)
def test_linear_act_random_shapes(case):
    """gate/up matrices (rows 2i gate, 2i+1 up, one column-scale vector per parity): act(gate) * up
    from the decode kernel (interleaved float32 intermediate), the 64-token and the 256-token tile
    kernels (intermediate in two halves), tanh-GELU and SiLU, with and without a bias."""
    rng = np.random.default_rng(5)
    for (K2, N, M, act) in ((24, 384, 3, "silu"), (130, 640, 8, "gelu_tanh"), (77, 1152, 9, "silu"), (256, 512, 64, "gelu_tanh"),
                            (300, 256, 65, "silu"), (129, 1408, 300, "gelu_tanh"), (512, 128, 257, "silu")):
        K = 2 * K2
        raw = make_raw(case, K, N, seed=K + N)
        pk = oracle_pack(case, raw)
        cs = (rng.random((2, N)) + 0.5).astype(np.float16)
        W = R.dequant(pk, K, N, case[0], col_scale=cs, **kw_of(case)).astype(np.float64)
        for tiled in (False, True):
            pm = packed_from_oracle(case, pk, cs, K, N, DEV, tiled=tiled)
            x = acts(M, N, torch.bfloat16, seed=M)
            bias = acts(1, K, torch.float32, seed=K)[0] if M % 2 else None
            t = _np(x).astype(np.float64) @ W.T
            if bias is not None:
                t = t + _np(bias).astype(np.float64)[None, :]
            g, u = t[:, 0::2], t[:, 1::2]
            if act == "silu":
                a = g / (1.0 + np.exp(-g))
            else:
                a = 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
            ref = a * u
            y = ops.linear_act(pm, x.to(DEV), act, bias=None if bias is None else bias.to(DEV), out_dtype=torch.float32)
            assert y.shape == (M, K2)
            err = rel_fro(_np(y), ref.astype(np.float32))
            # above 128 rows the intermediate is rounded to the output type before the activation
            assert err < (4e-3 if M > 128 else TOL), f"{case_id(case)} {K}x{N} M={M} tiled={tiled} {act}: {err}"


def test_gemv_between_one_and_two_tiles_per_workgroup():
    """257..512 row tiles: where at least 192 workgroups still get work, two tiles go to each of
    half as many workgroups; below that (and above 512 tiles) the tiles are dealt over 256.  Same
    results either way: against float64 on the dequantised weights, and batched against single calls."""
    for K in (4112, 5376, 6144, 8192, 8208):
        N = 384
        pm = F.synth_packed(K, N, F.BLK1632_4, 4, 128, 16, seed=K, device=DEV).to_tiled()
        W = ops.dequant(pm, torch.float32).double()
        x = acts(2, N, torch.float16, seed=K % 89).to(DEV)
        y = ops.gemv(pm, x, out_dtype=torch.float32)
        ref = x.double() @ W.t()
        assert float((y.double() - ref).abs().max() / ref.abs().max()) < 2e-5, K
        assert torch.equal(ops.gemv(pm, x[1:2], out_dtype=torch.float32)[0], y[1])


@pytest.mark.parametrize("layout", [F.SPARSE4, F.SPARSE4X, F.SPARSE4E], ids=lambda l: F.LAYOUT_NAME[l])
def test_synthetic_survivor_streams(layout):
    """The synthetic variable-length matrices the benchmark times: the device dequantiser reads them
    as the oracle does (bit for bit), and the decode kernel agrees with float64 on those weights."""
    K, N = 200, 1152
    pm = F.synth_packed(K, N, layout, seed=2, device=DEV)
    W = ops.dequant(pm, torch.float32)
    pk = dict(data=pm.array("data").cpu().numpy(), scale=pm.array("scale").cpu().numpy().reshape(K, -1),
              zero=pm.array("zero").cpu().numpy().reshape(K, -1), row_off=pm.array("row_off").cpu().numpy().view(np.uint32))
    cs = pm.array("col_scale").cpu().numpy().reshape(1, N)
    assert np.array_equal(_np(W), R.dequant(pk, K, N, layout, col_scale=cs[0]))
    for M in (1, 5):
        x = acts(M, N, torch.float16, seed=M).to(DEV)
        y = ops.gemv(pm, x, out_dtype=torch.float32)
        ref = x.double() @ W.double().t()
        assert float((y.double() - ref).abs().max() / ref.abs().max()) < 2e-5, M
