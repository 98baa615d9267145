"""CPU-side checks of the product package: its packer against the oracle's bytes, the C-ABI
library's exports and host-side validation, and the nn.Module plumbing.  No kernel runs here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import cbk_ref as R
from cobalt_amd import _lib, format as F
from cobalt_amd.linear import CobaltLinear, patch_model
from helpers import FIXED_CASES, case_id, kw_of, make_raw, oracle_pack, product_pack

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("case", FIXED_CASES, ids=case_id)
def test_product_packer_matches_oracle_bytes(case):
    K, N = 12, 640
    raw = make_raw(case, K, N, seed=7)
    raw["zero"][0, 0] = -3        # one off-grid group, exercises the zero repair
    raw["zero"][5, 1] = 99 if case[1] < 8 else 300
    pk = oracle_pack(case, raw)
    pm = product_pack(case, raw)
    assert np.array_equal(pm.array("data").numpy(), pk["data"])
    assert np.array_equal(pm.array("scale").numpy(), pk["scale"].reshape(-1))
    assert np.array_equal(pm.array("zero").numpy(), pk["zero"].reshape(-1))
    assert pm.n_zero_fixed == pk["n_zero_fixed"] == 2 and pm.n_survivors == pk["n_survivors"]
    assert pm.data_bytes == K * R.row_stride(case[0], N, *case[1:]) and pm.stream_bytes() == R.stream_bytes(pk)
    assert abs(pm.bpw() - R.bpw(pk, K, N)) < 1e-12
    assert all(o % 256 == 0 for o in pm.offs.values())


@pytest.mark.parametrize("case", FIXED_CASES, ids=case_id)
def test_synth_packed_is_valid(case):
    layout, bits, group, keep = case
    K, N = 8, 384
    pm = F.synth_packed(K, N, layout, bits, group, keep or None, seed=3)
    pk = dict(data=pm.array("data").numpy(), scale=pm.array("scale").numpy().reshape(K, -1),
              zero=pm.array("zero").numpy().reshape(K, -1), row_off=None)
    q, kp = R.unpack_codes(pk, K, N, layout, **kw_of(case))
    if keep:
        assert (kp.reshape(K, N // 32, 32).sum(-1) == keep).all()
    assert q.max() <= (1 << bits) - 1
    # padding bits of the stream are zero, so re-packing the decoded codes reproduces the bytes
    pk2 = R.pack_matrix(R.pack_bits(kp), q, pk["scale"], pk["zero"], layout, fix_zero=False, **kw_of(case))
    assert np.array_equal(pk2["data"], pk["data"])


@pytest.mark.parametrize("layout", [F.SPARSE4, F.SPARSE4X, F.SPARSE4E], ids=lambda l: F.LAYOUT_NAME[l])
def test_synth_packed_survivor_streams_are_valid(layout):
    """The synthetic rows have the structure the oracle's reader checks (stored group offsets equal
    the bitmap's prefix sums, rows padded to 16 bytes) and, random padding nibbles aside, are the
    bytes the oracle's packer makes from the decoded codes."""
    K, N = 9, 640
    pm = F.synth_packed(K, N, layout, seed=5)
    pm.validate(deep=True)
    ro = pm.array("row_off").numpy().view(np.uint32)
    pk = dict(data=pm.array("data").numpy(), scale=pm.array("scale").numpy().reshape(K, -1),
              zero=pm.array("zero").numpy().reshape(K, -1), row_off=ro)
    q, kp = R.unpack_codes(pk, K, N, layout)
    assert int(kp.sum()) == pm.n_survivors and q.max() <= 15 and (q[~kp] == 0).all()
    pk2 = R.pack_matrix(R.pack_bits(kp), q, pk["scale"], pk["zero"], layout, fix_zero=False)
    assert np.array_equal(pk2["row_off"], ro) and pk2["data"].size == pk["data"].size
    q2, kp2 = R.unpack_codes(pk2, K, N, layout)
    assert np.array_equal(q2, q) and np.array_equal(kp2, kp)


def test_stream_helpers_roundtrip():
    g = torch.Generator().manual_seed(0)
    for bits in (2, 3, 4, 6, 8):
        for n in (8, 40, 92, 250):
            c = torch.randint(0, 1 << bits, (5, n), generator=g, dtype=torch.int32)
            s = F.pack_stream(c, bits)
            assert s.shape[1] == (n * bits + 7) // 8
            assert torch.equal(F.unpack_stream(s, n, bits), c)
            assert np.array_equal(s.numpy(), R._pack_stream(c.numpy(), bits))


# ------------------------------------------------------------------ C ABI
def test_group_offsets_turn_sparse4_rows_into_the_oracles_sparse4x_bytes():
    """ops.with_group_offsets: the SPARSE4 image of a matrix plus the offset tables is, byte for
    byte, the SPARSE4X image the packer writes for the same matrix (pack_cobalt.py:201-250);
    groups with no, one and all survivors, a row count off the 16-row grid."""
    from cobalt_amd import ops
    from helpers import packed_from_oracle
    K, N = 37, 1024
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=21)
    rng = np.random.default_rng(3)
    keep = R.unpack_bits(raw["mask"], N)
    keep[3, :256] = False
    keep[4, 128:384] = True
    keep[5] = False
    keep[5, 700] = True
    raw["q"] = (rng.integers(0, 16, (K, N), dtype=np.uint8) * keep).astype(np.uint8)
    raw["mask"] = R.pack_bits(keep)
    p4 = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.SPARSE4)
    px = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.SPARSE4X)
    pm4 = packed_from_oracle((F.SPARSE4, 4, 128, 0), p4, raw["col_scale"], K, N, "cpu")
    pmx = ops.with_group_offsets(pm4)
    assert pmx.layout == F.SPARSE4X and pmx.validate(deep=True) is pmx
    assert np.array_equal(pmx.array("row_off").numpy().view(np.uint32), px["row_off"])
    assert np.array_equal(pmx.array("data").numpy(), px["data"])
    assert np.array_equal(pmx.array("scale").numpy().view(np.uint16), np.asarray(px["scale"]).view(np.uint16).reshape(-1))
    assert np.array_equal(pmx.array("zero").numpy(), np.asarray(px["zero"]).reshape(-1))
    assert torch.equal(pmx.array("col_scale"), pm4.array("col_scale"))
    with pytest.raises(ValueError):
        ops.with_group_offsets(pmx)


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "cbk.h")).read()
    names = set(re.findall(r"\b(cbk_[a-z_]+)\s*\(", hdr))
    assert {"cbk_gemv", "cbk_gemm", "cbk_linear", "cbk_dequant", "cbk_workspace_bytes"} <= names
    L = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(L, n), n
    assert set(_lib.SIGNATURES) == names
    assert _lib.lib().cbk_abi_version() == 1


def test_bench_helper_library_loads():
    """libcbk_bench.so (the measured-ceiling probes of bench.py) is built beside the C-ABI library
    and exports its two entry points; nothing is launched here."""
    path = os.path.join(ROOT, "cobalt_amd", "libcbk_bench.so")
    if not os.path.exists(path):
        pytest.skip("libcbk_bench.so is not built (python -m cobalt_amd.build)")
    L = ctypes.CDLL(path)
    assert hasattr(L, "cbk_bench_mfma_f16") and hasattr(L, "cbk_bench_read")


def test_descriptor_validation_and_strides():
    L = _lib.lib()
    for case in FIXED_CASES:
        layout, bits, group, keep = case
        for N in (128, 4096, 5376, 14336, 21504):
            d = F.CbkDesc(K=16, N=N, layout=layout, bits=bits, group=group, keep=keep)
            assert L.cbk_row_stride(ctypes.byref(d)) == R.row_stride(layout, N, bits, group, keep or None)
    d = F.CbkDesc(K=16, N=4096, layout=F.BLK1632_4)
    o = F.CbkDesc()
    assert L.cbk_desc_check(ctypes.byref(d), ctypes.byref(o)) == 0 and (o.bits, o.group, o.keep) == (4, 128, 16)
    assert L.cbk_stream_bytes(ctypes.byref(d), 0) == 16 * 4096 * 3 // 8 + 16 * 32 * 3
    bad = [F.CbkDesc(K=16, N=4096, layout=11), F.CbkDesc(K=16, N=4096, layout=F.BLKC, bits=5, group=128, keep=16),
           F.CbkDesc(K=16, N=4096, layout=F.BLKC, bits=4, group=32, keep=16),
           F.CbkDesc(K=16, N=4096, layout=F.BLKC, bits=4, group=64, keep=33),
           F.CbkDesc(K=16, N=4096, layout=F.BF16)]
    for b in bad:
        assert L.cbk_desc_check(ctypes.byref(b), ctypes.byref(o)) == -2
    assert L.cbk_desc_check(ctypes.byref(F.CbkDesc(K=16, N=4000, layout=F.DENSE4)), ctypes.byref(o)) == -3
    assert L.cbk_desc_check(ctypes.byref(F.CbkDesc(K=0, N=4096, layout=F.DENSE4)), ctypes.byref(o)) == -3
    assert L.cbk_desc_check(None, ctypes.byref(o)) == -1


def test_workspace_sizes_of_the_decode_path():
    """cbk_workspace_bytes at decode sizes (host arithmetic only, nothing is launched): two to eight
    activation rows of a long row (8192 columns and more, digits beyond LDS) leave room for the
    part sums of the column-split kernel, K * M * parts * 4 bytes with 14 parts at 21504 columns;
    the figure is a multiple of 256, grows with M, and a batch asks for the sum of its matrices."""
    L = _lib.lib()
    flags = F.zero_flags(15, 4)
    long_row = F.CbkDesc(K=5376, N=21504, layout=F.BLK1632_4, flags=flags)
    short_row = F.CbkDesc(K=21504, N=5376, layout=F.BLK1632_4, flags=flags)
    last = 0
    for M in (2, 4, 8):
        need = L.cbk_workspace_bytes(ctypes.byref(long_row), M)
        assert need >= 5376 * M * 14 * 4 and need % 256 == 0 and need >= last
        last = need
    descs = (F.CbkDesc * 2)(long_row, short_row)
    assert L.cbk_gemv_batch_workspace_bytes(2, descs, 8) == \
        L.cbk_workspace_bytes(ctypes.byref(long_row), 8) + L.cbk_workspace_bytes(ctypes.byref(short_row), 8)


def test_entry_points_reject_bad_arguments_before_any_launch():
    L = _lib.lib()
    d = F.CbkDesc(K=16, N=256, layout=F.BLK1632_4)
    # NULL device arrays
    assert L.cbk_gemv(ctypes.byref(d), None, 1, 1, 256, None, 0, 16, None, None, 0, None) == -1
    assert L.cbk_dequant(ctypes.byref(d), 0, 16, 1, None, 0, 256, None) == -1
    d.data, d.scale, d.zero = 0x1000, 0x2000, 0x3000           # never dereferenced: checks fail first
    assert L.cbk_gemv(ctypes.byref(d), None, 1, 1, 256, None, 0, 16, None, None, 0, None) == -1
    assert L.cbk_gemv(ctypes.byref(d), 0x4000, 0, 1, 256, 0x5000, 0, 16, None, None, 0, None) == -5
    assert L.cbk_gemv(ctypes.byref(d), 0x4000, 1, 17, 256, 0x5000, 0, 16, None, None, 0, None) == -3
    assert L.cbk_gemv(ctypes.byref(d), 0x4000, 1, 1, 128, 0x5000, 0, 16, None, None, 0, None) == -3
    assert L.cbk_gemv(ctypes.byref(d), 0x4004, 1, 1, 256, 0x5000, 0, 16, None, None, 0, None) == -4
    assert L.cbk_gemm(ctypes.byref(d), 0x4000, 2, 300, 260, 0x5000, 2, 16, None, None, 0, None) == -4
    assert L.cbk_dequant(ctypes.byref(d), 8, 16, 1, 0x5000, 0, 256, None) == -3
    d.data = 0x1004
    assert L.cbk_gemv(ctypes.byref(d), 0x4000, 1, 1, 256, 0x5000, 0, 16, None, None, 0, None) == -4
    d.data, d.cs_rows = 0x1000, 1
    assert L.cbk_gemv(ctypes.byref(d), 0x4000, 1, 1, 256, 0x5000, 0, 16, None, None, 0, None) == -1
    assert b"aligned" in L.cbk_strerror(-4)
    # the packing and the static-scratch entry points check before they launch, too
    d = F.CbkDesc(K=16, N=256, layout=F.BLK1632_4)
    assert L.cbk_pack(ctypes.byref(d), None, 0x4000, 0x5000, 0x6000, 1, 1, None, None) == -1      # no destination arrays
    d.data, d.scale, d.zero = 0x1000, 0x2000, 0x3000
    assert L.cbk_pack(ctypes.byref(d), None, None, 0x5000, 0x6000, 1, 1, None, None) == -1
    assert L.cbk_pack(ctypes.byref(d), None, 0x4000, 0x5000, 0x6000, 0, 1, None, None) == -5      # zero points are fp16 or uint8
    assert L.cbk_pack(ctypes.byref(d), None, 0x4004, 0x5000, 0x6000, 1, 1, None, None) == -4
    assert L.cbk_pack(ctypes.byref(d), 0x7001, 0x4000, 0x5000, 0x6000, 3, 1, None, None) == -4
    ds = F.CbkDesc(K=16, N=256, layout=F.SPARSE4, data=0x1000, scale=0x2000, zero=0x3000, row_off=0x8000)
    assert L.cbk_pack(ctypes.byref(ds), None, 0x4000, 0x5000, 0x6000, 1, 1, None, None) == -8     # variable-length layouts are not produced
    big = F.CbkDesc(K=256, N=21504, layout=F.BLK1632_4, data=0x1000, scale=0x2000, zero=0x3000)
    assert L.cbk_gemm_static(ctypes.byref(big), 0x4000, 2, 4096, 21504, 0x5000, 2, 256, None, None) == -6


def test_ops_refuse_to_run_without_gpu_tensors():
    from cobalt_amd import ops
    pm = F.synth_packed(16, 256, F.BLK1632_4, seed=1)
    with pytest.raises(_lib.CbkError):
        ops.linear(pm, torch.zeros(1, 256, dtype=torch.float16))
    with pytest.raises(_lib.CbkError):
        ops.dequant(pm)


# ------------------------------------------------------------------ module plumbing
class _FakeSQL(torch.nn.Module):
    """Same buffers as the reference's SparseQuantLinear (benchmark_suite.py:1178-1198)."""

    def __init__(self, W_q, scales, zeros, mask, scale2, bias, meta):
        super().__init__()
        for n, v in dict(W_q=W_q, scales=scales, zeros=zeros, mask=mask, scale2=scale2).items():
            self.register_buffer(n, v)
        self.bias = torch.nn.Parameter(bias) if bias is not None else None
        self.meta = meta


def _fake_sql(K, N, bits, group, block, seed):
    raw = R.synth_raw_matrix(K, N, 0.5, bits, seed=seed, block=block, group=group)
    keep = torch.from_numpy(R.unpack_bits(raw["mask"], N))
    m = _FakeSQL(torch.from_numpy(raw["q"]).half(), torch.from_numpy(raw["scale"]).reshape(K, -1, 1),
                 torch.from_numpy(raw["zero"]).reshape(K, -1, 1), keep.half(),
                 torch.from_numpy(raw["col_scale"]).reshape(1, N), torch.randn(K).half(),
                 {"nbits": bits, "group_size": group})
    return m, raw


def test_from_sparse_quant_linear_layout_choice_and_bytes():
    m, raw = _fake_sql(16, 256, 4, 128, 32, 1)
    cl = CobaltLinear.from_sparse_quant_linear(m)
    p = cl.packed()
    assert (p.layout, p.bits, p.group, p.keep) == (F.BLK1632_4, 4, 128, 16)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.BLK1632_4)
    assert np.array_equal(p.array("data").numpy(), pk["data"])
    assert np.array_equal(p.array("col_scale").numpy(), raw["col_scale"])
    m2, _ = _fake_sql(16, 256, 3, 64, 0, 2)               # unconstrained mask -> dense stream
    p2 = CobaltLinear.from_sparse_quant_linear(m2).packed()
    assert (p2.layout, p2.bits, p2.group) == (F.DENSEB, 3, 64)
    m3, _ = _fake_sql(16, 256, 2, 64, 32, 3)
    p3 = CobaltLinear.from_sparse_quant_linear(m3).packed()
    assert (p3.layout, p3.bits, p3.group, p3.keep) == (F.BLKC, 2, 64, 16)
    assert cl.bias is not None and cl.in_features == 256 and cl.out_features == 16
    assert "BLK1632_4" in repr(cl)
    with pytest.raises(ValueError):
        cl.set_forward_backend("pytorch")


def test_state_dict_roundtrip_and_patch_model():
    m, _ = _fake_sql(16, 256, 4, 128, 32, 4)
    cl = CobaltLinear.from_sparse_quant_linear(m)
    sd = cl.state_dict()
    assert set(sd) == {"blob", "cbk_meta", "bias"}
    cl2 = CobaltLinear(F.synth_packed(16, 256, F.BLK1632_4, seed=9), bias=torch.zeros(16).half())
    cl2.load_state_dict(sd)
    assert torch.equal(cl2.blob, cl.blob) and cl2.packed().offs == cl.packed().offs

    net = torch.nn.Sequential(torch.nn.Linear(256, 16), torch.nn.ReLU())
    net.add_module("inner", torch.nn.Sequential(torch.nn.Linear(256, 16)))
    done = patch_model(net, lambda name, mod: cl if isinstance(mod, torch.nn.Linear) and name == "inner.0" else None)
    assert done == ["inner.0"] and net.inner[0] is cl
    done = patch_model(net, {"0": cl2})
    assert done == ["0"] and net[0] is cl2
    with pytest.raises(TypeError):
        F.dtype_code(torch.float64)


def test_packed_matrix_validate_refuses_descriptions_that_do_not_fit_the_image():
    """A description from a state dict or a manifest is outside input: offsets past the image,
    misaligned arrays, a byte count that is not rows x stride, row ranges beyond K, parameters the
    layout does not take and row offsets that are not increasing multiples of 16 all raise."""
    import dataclasses
    pm = F.synth_packed(48, 256, F.BLK1632_4, seed=1)
    assert pm.validate() is pm and pm.to_tiled().validate().tiled
    for change in (dict(offs={**pm.offs, "scale": pm.blob.numel()}), dict(offs={**pm.offs, "data": 8}),
                   dict(offs={k: v for k, v in pm.offs.items() if k != "zero"}), dict(data_bytes=pm.data_bytes - 96),
                   dict(K=pm.K + 1), dict(cs_rows=4), dict(cs_rows=3, cs_splits=(40, 16)), dict(bits=3), dict(keep=8),
                   dict(layout=4), dict(N=192), dict(blob=pm.blob[:-256])):
        with pytest.raises(ValueError):
            dataclasses.replace(pm, **change).validate()
    import os
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sparse_stream.npz"))
    sp = F.from_arrays(z["c0_SPARSE4X_data"], z["c0_SPARSE4X_scale"], z["c0_SPARSE4X_zero"], None, 5, 256, F.SPARSE4X,
                       row_off=z["c0_SPARSE4X_row_off"].astype(np.int32))
    assert sp.validate(deep=True) is sp
    ro = sp.array("row_off").clone()
    ro[3] += 8
    broken = sp.clone()
    broken.array("row_off")[:] = ro
    with pytest.raises(ValueError):
        broken.validate(deep=True)
    cl = CobaltLinear(pm)
    meta = cl.cbk_meta.clone()
    meta[12] = pm.blob.numel()                                         # off_scale past the image
    with pytest.raises(ValueError):
        CobaltLinear.from_state(pm.blob, meta)
