"""The producer side on the GPU: the library's packing kernel (RAW arrays -> CBK1 rows, row-major
or tiled) bit for bit against the oracle's packer, the torch packer and the reference's own bytes;
the compressor run on the GPU against the reference's vectors."""
import ctypes
import os
import time

import numpy as np
import pytest
import torch

from cobalt_amd import _lib, compress as C, format as F, ops
from cobalt_amd.linear import CobaltLinear
from oracle import cbk_ref as R
from helpers import FIXED_CASES, case_id, make_raw, oracle_pack

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _same_arrays(a, b, names=("data", "scale", "zero", "col_scale")):
    for n in names:
        if n == "col_scale" and not a.cs_rows:
            continue
        assert torch.equal(a.array(n), b.array(n)), n


@pytest.mark.parametrize("case", FIXED_CASES, ids=case_id)
def test_hip_packer_writes_the_oracle_bytes(case):
    """K not a multiple of 16 (tile padding), N an odd and an even multiple of 128 (a last
    128-column unit), zero points off the grid (the repair path), two column-scale rows."""
    layout, bits, group, keep = case
    for K, N, seed in ((37, 384, 1), (48, 1024, 2)):
        raw = make_raw(case, K, N, seed=seed)
        zero = raw["zero"].astype(np.float16).copy()
        if seed == 1:
            zero[3, 0] = -2.0
            zero[5, -1] = float((1 << bits) + 1)
        pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], zero, layout,
                           **({"bits": bits, "group": group, "keep_per_block": keep or None} if layout in (F.BLKC, F.DENSEB) else {}))
        cs = np.stack([raw["col_scale"], raw["col_scale"][::-1]], 0) if seed == 2 else raw["col_scale"]
        host = (raw["mask"], raw["q"], raw["scale"], zero, cs)
        args = tuple(_t(a) for a in host) + (layout, bits, group, keep or None)
        # the torch packer on the CPU: its divisions on the GPU round differently in the zero-point repair
        torch_pm = F.pack_raw(*[torch.from_numpy(np.ascontiguousarray(a)) for a in host], layout, bits, group, keep or None).to(DEV)
        rm = ops.pack_raw(*args, tiled=False)
        a, c = rm.array("data").cpu().numpy(), pk["data"]
        assert np.array_equal(a, c), f"row bytes against the oracle: {np.nonzero(a != c)[0][:8]} of {(a != c).sum()}, K={K} N={N}"
        assert np.array_equal(rm.array("scale").cpu().numpy().reshape(K, -1), pk["scale"])
        assert np.array_equal(rm.array("zero").cpu().numpy().reshape(K, -1), pk["zero"])
        assert (rm.offs, rm.data_bytes, rm.flags, rm.n_survivors, rm.n_zero_fixed, rm.cs_rows) == \
               (torch_pm.offs, torch_pm.data_bytes, torch_pm.flags, torch_pm.n_survivors, torch_pm.n_zero_fixed, torch_pm.cs_rows)
        assert torch.equal(rm.blob, torch_pm.blob)
        tl, want = ops.pack_raw(*args, tiled=True), torch_pm.to_tiled()
        assert (tl.offs, tl.data_bytes, tl.flags) == (want.offs, want.data_bytes, want.flags) and torch.equal(tl.blob, want.blob)
        W = R.dequant(pk, K, N, layout, col_scale=np.asarray(cs, np.float16).reshape(-1, N),
                      **({"bits": bits, "group": group, "keep_per_block": keep or None} if layout in (F.BLKC, F.DENSEB) else {}))
        assert np.array_equal(ops.dequant(tl, torch.float32).cpu().numpy() + np.float32(0), W + np.float32(0))


def test_hip_packer_writes_the_reference_bytes():
    """tests/golden/fixed_stride.npz: bytes of the reference's own pack_matrix."""
    fix = np.load(os.path.join(GOLD, "fixed_stride.npz"))
    for name in ("DENSE4", "DENSE8", "BLK1632_4", "BLK1632_6"):
        p = name + "_"
        pm = ops.pack_raw(_t(fix[p + "mask"]), _t(fix[p + "q"]), _t(fix[p + "scale_in"]), _t(fix[p + "zero_in"]),
                          _t(fix[p + "col_scale"]), getattr(F, name), tiled=False)
        assert np.array_equal(pm.array("data").cpu().numpy(), fix[p + "data"]), name
        assert np.array_equal(pm.array("scale").cpu().numpy().reshape(6, -1), fix[p + "scale"])
        assert np.array_equal(pm.array("zero").cpu().numpy().reshape(6, -1), fix[p + "zero"])
        assert pm.n_zero_fixed == 2


def test_hip_packer_refuses_a_mask_with_the_wrong_block_count():
    raw = make_raw((F.BLK1632_4, 4, 128, 16), 32, 256, seed=3)
    mask = raw["mask"].copy()
    mask[7, 4] ^= 1
    with pytest.raises(ValueError):
        ops.pack_raw(_t(mask), _t(raw["q"]), _t(raw["scale"]), _t(raw["zero"]), _t(raw["col_scale"]), F.BLK1632_4)
    with pytest.raises(Exception):
        ops.pack_raw(torch.from_numpy(mask), torch.from_numpy(raw["q"]), torch.from_numpy(raw["scale"]),
                     torch.from_numpy(raw["zero"]), None, F.BLK1632_4)                       # CPU tensors: not this packer


def test_modules_built_on_the_gpu_use_the_hip_packer_and_match_the_cpu_build():
    raw = make_raw((F.BLK1632_4, 4, 128, 16), 80, 512, seed=4)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    cpu = CobaltLinear.from_raw(t(raw["mask"]), t(raw["q"]), t(raw["scale"]), t(raw["zero"]), t(raw["col_scale"]))
    gpu = CobaltLinear.from_raw(*[_t(raw[k]) for k in ("mask", "q", "scale", "zero", "col_scale")])
    assert gpu.blob.is_cuda and torch.equal(gpu.blob.cpu(), cpu.blob) and torch.equal(gpu.cbk_meta, cpu.cbk_meta)
    tiled = CobaltLinear.from_raw(*[_t(raw[k]) for k in ("mask", "q", "scale", "zero", "col_scale")], tiled=True)
    assert tiled._pm().tiled and torch.equal(tiled.blob.cpu(), cpu._pm().to_tiled().blob)


def _golden_case(fix, i):
    p = f"c{i}_"
    c = {k[len(p):]: fix[k] for k in fix.files if k.startswith(p)}
    X = c["X"].astype(np.float64)
    c["H"] = (X.T @ X).astype(np.float32)
    sp, beta, bits, group, mb = c["cfg"]
    c["args"] = (float(sp), float(beta), int(bits), int(group), int(mb))
    c["keep"] = np.unpackbits(c["mask"], axis=-1, bitorder="little")[:, : c["W"].shape[1]].astype(bool)
    return c


def test_compressor_on_the_gpu_against_the_reference_vectors():
    """`cobalt_compress` with its tensors on the GPU against the vectors the reference's
    `cobalt_math.cobalt_quantize` wrote (tests/golden/cobalt_quantize.npz; bit for bit on the CPU).
    The mask is computed before any matrix product and has to be identical.  The Cholesky inverse
    and the compensation matmul are other libraries on the GPU and sum in another order, so what
    follows them agrees to rounding: scales and column scales within one fp16 step, zero points
    within one code, at most 2 % of the codes differ and never by more than one, and the
    reconstruction error equals the reference's to 1e-3 of itself."""
    fix = np.load(os.path.join(GOLD, "cobalt_quantize.npz"))
    for i in range(4):
        c = _golden_case(fix, i)
        sp, beta, bits, group, mb = c["args"]
        r = C.cobalt_compress(_t(c["W"]), _t(c["H"]), sp, bits, group, beta, mb)
        assert r["q"].is_cuda
        keep = c["keep"]
        assert np.array_equal(r["mask"].cpu().numpy(), c["mask"]), f"case {i}: mask bytes"
        q = r["q"].cpu().numpy().astype(np.int32)
        dq = np.abs(q[keep] - c["q"][keep].astype(np.int32))
        assert dq.max() <= 1 and (dq != 0).mean() <= 0.02, f"case {i}: {(dq != 0).mean():.4f} of the codes differ, max {dq.max()}"
        assert (q[~keep] == 0).all()
        for name in ("scale", "col_scale"):
            a, b = r[name].cpu().numpy().astype(np.float32), c[name].astype(np.float16).astype(np.float32)
            assert np.all(np.abs(a - b) <= np.abs(b) * 2.0 ** -10), f"case {i}: {name}"
            assert (a != b).mean() <= 0.05, f"case {i}: {name} differs in {(a != b).mean():.3f} of its entries"
        assert np.abs(r["zero"].float().cpu().numpy() - c["zero"]).max() <= 1
        W_hat = r["W_hat"].cpu().numpy()
        rel = np.linalg.norm(W_hat - c["W"]) / np.linalg.norm(c["W"])
        assert abs(rel - float(c["relerr"])) < 1e-3 * float(c["relerr"]), f"case {i}: {rel} vs {float(c['relerr'])}"


def test_compress_and_pack_one_full_size_matrix_on_the_gpu():
    """14336 x 4096 (the reference's bandwidth-test shape) through the whole producer path on the
    GPU: Hessian, compressor, HIP packer; the packed module multiplies like its own W_hat.  Prints
    the seconds each stage took."""
    K, N = 14336, 4096
    g = torch.Generator(device=DEV).manual_seed(0)
    W = torch.randn(K, N, device=DEV, generator=g) * 0.02
    X = torch.randn(2048, N, device=DEV, generator=g)
    torch.cuda.synchronize(); t0 = time.time()
    H = C.hessian(X)
    raw = C.cobalt_compress(W, H, 0.5, 4, 128, 0.5, 32)
    torch.cuda.synchronize(); t1 = time.time()
    pm = ops.pack_raw(raw["mask"], raw["q"], raw["scale"], raw["zero"], raw["col_scale"], F.BLK1632_4, tiled=True)
    torch.cuda.synchronize(); t2 = time.time()
    ref = F.pack_raw(*[raw[k].cpu() for k in ("mask", "q", "scale", "zero", "col_scale")], F.BLK1632_4).to_tiled()
    t3 = time.time()
    print(f"\n14336x4096: compress {t1 - t0:.3f} s, HIP pack {t2 - t1:.4f} s ({pm.n_zero_fixed} zero points re-derived), "
          f"torch pack + tile on the CPU {t3 - t2:.2f} s", flush=True)
    assert torch.equal(pm.blob.cpu(), ref.blob) and abs(pm.bpw() - 3.1875) < 1e-9 and pm.n_zero_fixed == ref.n_zero_fixed
    x = torch.randn(2, N, device=DEV, generator=g).half()
    y = ops.gemv(pm, x, out_dtype=torch.float32).double()
    want = x.double() @ ops.dequant(pm, torch.float32).double().T
    assert float((y - want).abs().max() / want.abs().max()) < 2e-5
    loose = x.double() @ raw["W_hat"].double().T                        # scales not yet rounded to fp16
    assert float((y - loose).norm() / loose.norm()) < 1e-3


# ------------------------------------------------------------------ the way back, and re-packing
from helpers import SPARSE_CASES, packed_from_oracle, kw_of, rel_fro, acts


@pytest.mark.parametrize("case", FIXED_CASES + SPARSE_CASES, ids=case_id)
def test_unpack_returns_the_codes_and_the_bitmap(case):
    """cbk_unpack on every layout, both byte orders, against the oracle's decoder: the codes of
    the kept columns, zeros (bitmap / survivor-stream layouts) or the zero point (dense layouts)
    at the pruned ones, and the keep bitmap."""
    layout, bits, group, keep = case
    K, N = 37, 640
    raw = make_raw(case, K, N, seed=9)
    pk = oracle_pack(case, raw)
    q_ref, keep_ref = R.unpack_codes(pk, K, N, layout, bits, group, keep or None)
    for tiled in ((False, True) if layout not in (F.SPARSE4, F.SPARSE4X, F.SPARSE4E) else (False,)):
        pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
        mask, q = ops.unpack(pm)
        q, keepm = q.cpu().numpy(), F.unpack_mask(mask.cpu(), N).numpy()
        dense = layout in (F.DENSE4, F.DENSE8, F.DENSEB)
        assert np.array_equal(keepm, np.ones_like(keepm) if dense else keep_ref != 0), tiled
        assert np.array_equal(q[keep_ref != 0], np.asarray(q_ref)[keep_ref != 0]), tiled
        if not dense:
            assert (q[keep_ref == 0] == 0).all()


@pytest.mark.parametrize("case", SPARSE_CASES, ids=case_id)
def test_survivor_streams_repacked_as_dense_rows(case):
    """A survivor-stream matrix re-packed as DENSE4 (`ops.transcode`) dequantises to the same
    values bit for bit and runs on the matrix-core kernels; and `ops.linear` above 16 rows, which
    re-packs inside the call's workspace, meets the oracle like every other layout."""
    layout = case[0]
    K, N = 300, 1152
    raw = R.synth_raw_matrix(K, N, 0.55, 4, seed=21)
    pk = oracle_pack(case, raw)
    W = R.dequant(pk, K, N, layout, col_scale=raw["col_scale"])
    pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV)
    d4 = ops.transcode(pm, F.DENSE4)
    assert d4.tiled and d4.layout == F.DENSE4 and abs(d4.bpw() - (4 + 24 / 128) * (304 / 300)) < 1e-9
    assert np.array_equal(ops.dequant(d4, torch.float32).cpu().numpy() + np.float32(0), W + np.float32(0))
    for M in (1, 8, 17, 64, 300):
        x = acts(M, N, torch.bfloat16, seed=M)
        ref = R.forward_ref(W, x.float().numpy())
        for p in (pm, d4):
            y = ops.linear(p, x.to(DEV), out_dtype=torch.float32).cpu().numpy()
            assert rel_fro(y, ref) < 1e-3, (case_id(case), M, p.layout)
    y = ops.gemm(pm, acts(5, N, torch.float16, seed=5).to(DEV), out_dtype=torch.float32)       # few rows: the row kernel
    assert rel_fro(y.cpu().numpy(), R.forward_ref(W, acts(5, N, torch.float16, seed=5).float().numpy())) < 1e-3


def test_survivor_stream_with_zero_points_off_the_code_grid():
    """A survivor-stream image may carry zero points that are no 4-bit codes (packed without the
    repair).  A dense layout cannot hold such a matrix (a pruned column stores the zero point as
    its code), so above 16 rows the call must not re-pack it: it runs as 16-row slices on the row
    kernel and meets the oracle at every row count; re-packing it on request is refused; and the
    packing kernel never lets a wide zero point spill into the neighbouring code."""
    case = (F.SPARSE4X, 4, 128, 0)
    K, N = 200, 1024
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=33)
    raw["zero"] = raw["zero"].copy()
    raw["zero"][::3, ::2] = 20                                   # off the grid, below 128
    pk = oracle_pack(case, raw, fix_zero=False)
    assert int(pk["zero"].max()) == 20
    W = R.dequant(pk, K, N, F.SPARSE4X, col_scale=raw["col_scale"])
    pm = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV)
    assert pm.flags & F.FLAG_ZERO_LE_128 and not pm.flags & F.FLAG_ZERO_ON_GRID
    assert _lib.lib().cbk_workspace_bytes(ctypes.byref(pm.desc()), 64) == 0
    assert np.array_equal(ops.dequant(pm, torch.float32).cpu().numpy() + np.float32(0), W + np.float32(0))
    for M in (1, 16, 17, 40):
        x = acts(M, N, torch.bfloat16, seed=M)
        y = ops.linear(pm, x.to(DEV), out_dtype=torch.float32).cpu().numpy()
        assert rel_fro(y, R.forward_ref(W, x.float().numpy())) < 1e-3, M
    with pytest.raises(ValueError, match="zero point"):
        ops.transcode(pm, F.DENSE4)
    # the same matrix with a workspace that would hold the dense image: still the row kernel
    x = acts(17, N, torch.float16, seed=2)
    ws = torch.empty(8 << 20, dtype=torch.uint8, device=DEV)
    y = ops.gemm(pm, x.to(DEV), out_dtype=torch.float32, workspace=ws).cpu().numpy()
    assert rel_fro(y, R.forward_ref(W, x.float().numpy())) < 1e-3


def test_module_with_sparse4_rows_gets_group_offsets_in_device_order():
    """to_device_order on a SPARSE4 matrix (the packer's default, pack_cobalt.py:561): the same codes
    as SPARSE4X, which the matrix-core stream kernel takes; values and results unchanged."""
    case = (F.SPARSE4, 4, 128, 0)
    K, N = 4112, 3072
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=8)
    pk = oracle_pack(case, raw)
    W = R.dequant(pk, K, N, F.SPARSE4, col_scale=raw["col_scale"])
    lin = CobaltLinear(packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV))
    x = acts(5, N, torch.float16, seed=1).to(DEV)
    y4 = ops.gemv(lin._pm(), x, out_dtype=torch.float32)
    lin.to_device_order()
    pm = lin._pm()
    assert pm.layout == F.SPARSE4X and not pm.tiled
    px = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.SPARSE4X)
    assert np.array_equal(pm.array("data").cpu().numpy(), px["data"])
    assert np.array_equal(lin.dequantize().cpu().numpy() + np.float32(0), W + np.float32(0))
    yx = ops.gemv(pm, x, out_dtype=torch.float32)
    ref = R.forward_ref(W, x.float().cpu().numpy())
    assert rel_fro(yx.cpu().numpy(), ref) < 1e-5 and rel_fro(y4.cpu().numpy(), ref) < 1e-5
    assert lin.to_device_order()._pm().layout == F.SPARSE4X                     # and stays


def test_module_with_a_survivor_stream_matrix_can_be_repacked_at_load():
    case = (F.SPARSE4E, 4, 128, 0)
    K, N = 96, 1024
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=4)
    pk = oracle_pack(case, raw)
    W = R.dequant(pk, K, N, F.SPARSE4E, col_scale=raw["col_scale"])
    lin = CobaltLinear(packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV))
    assert lin.to_device_order()._pm().layout == F.SPARSE4E                      # unchanged unless asked
    lin.to_device_order(repack_sparse=True)
    pm = lin._pm()
    assert (pm.layout, pm.tiled) == (F.DENSE4, True)
    assert np.array_equal(lin.dequantize().cpu().numpy() + np.float32(0), W + np.float32(0))
    x = acts(3, N, torch.float16, seed=1)
    y = lin(x.to(DEV)).float().cpu().numpy()
    assert rel_fro(y, R.forward_ref(W, x.float().numpy())) < 2e-3               # fp16 output
    sd = lin.state_dict()
    back = CobaltLinear.from_state(sd["blob"], sd["cbk_meta"])
    assert torch.equal(back.dequantize(), lin.dequantize())


def test_pack_and_unpack_at_the_smallest_and_ragged_shapes():
    """One row of one 128-column group; 17 rows (a tile and one row) of 128 and 384 columns: the
    packing kernel's half unit, the tile padding and the unpacker, both byte orders."""
    for case in ((F.BLK1632_4, 4, 128, 16), (F.BLKC, 3, 64, 10), (F.DENSE4, 4, 128, 0), (F.BLK1632_6, 6, 128, 16)):
        layout, bits, group, keep = case
        for K, N in ((1, 128), (17, 128), (17, 384)):
            raw = make_raw(case, K, N, seed=K + N)
            pk = oracle_pack(case, raw)
            args = tuple(_t(raw[k]) for k in ("mask", "q", "scale", "zero", "col_scale")) + (layout, bits, group, keep or None)
            for tiled in (False, True):
                pm = ops.pack_raw(*args, tiled=tiled)
                want = packed_from_oracle(case, pk, raw["col_scale"], K, N, DEV, tiled=tiled)
                assert torch.equal(pm.blob, want.blob), (case_id(case), K, N, tiled)
                mask, q = ops.unpack(pm)
                back = ops.pack_raw(None if keep == 0 else mask, q, pm.to_rowmajor().array("scale").view(K, -1),
                                    pm.to_rowmajor().array("zero").view(K, -1), _t(raw["col_scale"]), layout, bits, group,
                                    keep or None, fix_zero=False, tiled=tiled)
                assert torch.equal(back.blob, pm.blob), (case_id(case), K, N, tiled)
