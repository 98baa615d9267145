"""Pins oracle/cbk_ref.py: hand vectors, the reference documentation's known answers,
an independent per-position decoder, round trips and the exact-zero invariants."""
import numpy as np
import pytest

from oracle import cbk_ref as R

LAYOUT_CASES = [
    (R.DENSE4, {}), (R.DENSE8, {}), (R.BLK1632_4, {}), (R.BLK1632_6, {}),
    (R.SPARSE4, {}), (R.SPARSE4X, {}), (R.SPARSE4E, {}),
    (R.BLKC, dict(bits=4, group=128, keep_per_block=16)),
    (R.BLKC, dict(bits=3, group=128, keep_per_block=10)),
    (R.BLKC, dict(bits=2, group=64, keep_per_block=23)),
    (R.BLKC, dict(bits=3, group=64, keep_per_block=23)),
    (R.BLKC, dict(bits=4, group=64, keep_per_block=10)),
    (R.BLKC, dict(bits=2, group=64, keep_per_block=16)),
    (R.DENSEB, dict(bits=3, group=128)), (R.DENSEB, dict(bits=2, group=64)),
    (R.DENSEB, dict(bits=4, group=64)),
]


def _raw_for(layout, kw, K, N, seed):
    bits, group, kpb = R.canon(layout, kw.get("bits"), kw.get("group"), kw.get("keep_per_block"))
    if layout in R.BLK_FAMILY:
        sp = 1.0 - kpb / 32.0
        raw = R.synth_raw_matrix(K, N, sparsity=sp, bits=bits, seed=seed, block=32, group=group)
    else:
        raw = R.synth_raw_matrix(K, N, sparsity=0.5, bits=bits, seed=seed, group=group)
    return raw, bits, group, kpb


# ------------------------------------------------------------------ hand vectors
def test_hand_blk1632_4_block():
    # one row, N=128: block 0 keeps columns 0..15 with codes 0..15; blocks 1-3 keep the
    # odd columns with code 5.  docs/FORMAT.md:96-107: survivor 2j is the low nibble of byte j.
    N = 128
    keep = np.zeros((1, N), bool); keep[0, :16] = True; keep[0, 33::2] = True
    q = np.zeros((1, N), np.uint8); q[0, :16] = np.arange(16); q[0, 33::2] = 5
    pk = R.pack_matrix(R.pack_bits(keep), q, np.ones((1, 1), np.float16), np.zeros((1, 1), np.uint8), R.BLK1632_4)
    d = pk["data"]
    assert d.size == 3 * N // 8 + 64
    assert list(d[0:4]) == [0xFF, 0xFF, 0x00, 0x00]
    assert list(d[4:16]) == [0xAA] * 12
    assert list(d[16:24]) == [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]
    assert list(d[24:48]) == [0x55] * 24
    assert (d[48:] == 0).all()


def test_hand_dense4_nibble_order():
    N = 128
    q = (np.arange(N) % 16).astype(np.uint8)[None]
    pk = R.pack_matrix(None, q, np.ones((1, 1), np.float16), np.zeros((1, 1), np.uint8), R.DENSE4)
    # column j lives in byte j>>1, low nibble for even j (docs/FORMAT.md:85-87)
    assert list(pk["data"][:8]) == [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]
    assert pk["data"].size == N // 2 + 64


def test_hand_blk1632_6_hi2_word():
    # survivors i=0..15 of block 0 carry code 16*(i%4) + i  -> high-2-bits i%4, low nibble i.
    N = 128
    keep = np.zeros((1, N), bool); keep[0, 0:32:2] = True; keep[0, 32:] = np.tile([True, False], 48)
    q = np.zeros((1, N), np.uint8)
    q[0, 0:32:2] = [16 * (i % 4) + i for i in range(16)]
    pk = R.pack_matrix(R.pack_bits(keep), q, np.ones((1, 1), np.float16), np.zeros((1, 1), np.uint8), R.BLK1632_6)
    d = pk["data"]
    assert d.size == N // 2 + 64
    assert list(d[16:24]) == [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]
    # hi2 plane (docs/FORMAT.md:102-106): bits [0,16) even survivors (hi = 0,2,0,2,...), bits
    # [16,32) odd survivors (hi = 1,3,1,3,...), slot e at bits [2e, 2e+2).
    he = sum((([0, 2] * 4)[e]) << (2 * e) for e in range(8))
    ho = sum((([1, 3] * 4)[e]) << (2 * e) for e in range(8))
    word = int.from_bytes(bytes(d[48:52]), "little")
    assert word == (he | (ho << 16)) == 0xDDDD8888


def test_hand_3bit_stream_straddles_words():
    # codes j%8 at 3 bits each: every 8 codes are the 24-bit value 0o76543210 = 0xFAC688, so
    # the byte stream is 88 C6 FA repeating, and code 10 (bits 30..32) straddles a dword.
    N = 128
    q = (np.arange(N) % 8).astype(np.uint8)[None]
    pk = R.pack_matrix(None, q, np.ones((1, 1), np.float16), np.zeros((1, 1), np.uint8), R.DENSEB, bits=3, group=128)
    assert list(pk["data"][:48]) == [0x88, 0xC6, 0xFA] * 16
    w0, w1 = int.from_bytes(bytes(pk["data"][0:4]), "little"), int.from_bytes(bytes(pk["data"][4:8]), "little")
    assert ((w0 >> 30) | ((w1 & 1) << 2)) == 10 % 8
    assert pk["data"].size == 48 + 64


def test_hand_2bit_stream():
    N = 128
    q = (np.arange(N) % 4).astype(np.uint8)[None]
    pk = R.pack_matrix(None, q, np.ones((1, 2), np.float16), np.zeros((1, 2), np.uint8), R.DENSEB, bits=2, group=64)
    assert list(pk["data"][:32]) == [0xE4] * 32


def test_hand_blkc_3bit_10of32():
    # 10 survivors per block at 3 bits = 30 bits per block: block 1 starts at bit 30.
    N = 128
    keep = np.zeros((1, N), bool)
    for t in range(4):
        keep[0, 32 * t: 32 * t + 10] = True
    q = np.zeros((1, N), np.uint8)
    for t in range(4):
        q[0, 32 * t: 32 * t + 10] = (np.arange(10) + t) % 8
    pk = R.pack_matrix(R.pack_bits(keep), q, np.ones((1, 1), np.float16), np.zeros((1, 1), np.uint8),
                       R.BLKC, bits=3, group=128, keep_per_block=10)
    d = pk["data"]
    assert R.row_stride(R.BLKC, N, 3, 128, 10) == 16 + 16 and d.size == 32 + 64
    stream = int.from_bytes(bytes(d[16:32]), "little")
    for t in range(4):
        for i in range(10):
            assert (stream >> ((t * 10 + i) * 3)) & 7 == (i + t) % 8
    assert stream >> 120 == 0          # zero padding
    assert list(d[0:4]) == [0xFF, 0x03, 0, 0]


def test_hand_dequant_values():
    # W = (q - z) * s * cs * keep with s=0.5, z=3, cs=2 -> (q-3)
    N = 128
    keep = np.tile([True, False], N // 2)[None]
    q = (np.arange(N) % 16).astype(np.uint8)[None]
    pk = R.pack_matrix(R.pack_bits(keep), q, np.full((1, 1), 0.5, np.float16), np.full((1, 1), 3, np.uint8), R.BLK1632_4)
    W = R.dequant(pk, 1, N, R.BLK1632_4, col_scale=np.full(N, 2.0, np.float16))
    exp = np.where(keep, (np.arange(N) % 16) - 3.0, 0.0).astype(np.float32)
    assert np.array_equal(W, exp)


# ------------------------------------------------------------------ documented sizes
def test_known_bpw_and_sizes():
    assert R.bpw_formula(R.DENSE4) == 4.1875
    assert R.bpw_formula(R.BLK1632_4) == 3.1875
    assert R.bpw_formula(R.BLK1632_6) == 4.1875
    # docs/FORMAT.md:197-220
    assert round(25_598_361_600 * 4.1875 / 8 / 1e9, 3) == 13.399
    assert round(25_598_361_600 * 3.1875 / 8 / 1e9, 3) == 10.199
    assert round(6_979_321_856 * 4.1875 / 8 / 1e9, 3) == 3.653
    assert round(6_979_321_856 * 3.1875 / 8 / 1e9, 3) == 2.781
    # docs/FORMAT.md:29-34 manifest example: 4096 x 5376 BLK1632_4
    K, N = 4096, 5376
    assert K * R.row_stride(R.BLK1632_4, N) == 8257536
    assert K * (N // 128) * 2 == 344064 and K * (N // 128) == 172032 and N * 2 == 10752
    # extension table (bitmap + b*keep/32 + 24/g)
    assert R.bpw_formula(R.BLKC, 3, 128, 10) == 1 + 30 / 32 + 0.1875
    assert R.bpw_formula(R.BLKC, 2, 64, 23) == 1 + 46 / 32 + 0.375
    assert R.bpw_formula(R.DENSEB, 3, 128) == 3.1875


@pytest.mark.parametrize("layout,kw", LAYOUT_CASES)
def test_packed_bpw_matches_formula(layout, kw):
    K, N = 8, 512
    raw, bits, group, kpb = _raw_for(layout, kw, K, N, 3)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], layout, **kw)
    if layout in R.SPARSE_FAMILY:
        keep = R.unpack_bits(raw["mask"], N)
        G = N // group
        hdr = R._align(N // 8 + (R._align(2 * G, 16) if layout != R.SPARSE4 else 0), 16)
        cnt = keep.reshape(K, G, group).sum(-1)
        rb = R._align_arr(hdr + ((cnt + 1) // 2).sum(1), 16)
        assert pk["data"].size == rb.sum() + 64 and pk["row_off"][-1] == rb.sum()
    else:
        got = R.bpw(pk, K, N)
        want = R.bpw_formula(layout, bits, group, kpb)
        pad = 8.0 * (R.row_stride(layout, N, bits, group, kpb) * K) / (K * N) - (want - 24.0 / group)
        assert abs(got - want - pad) < 1e-12 and 0 <= pad < 0.26


# ------------------------------------------------------------------ round trip + cross-check
@pytest.mark.parametrize("layout,kw", LAYOUT_CASES)
def test_roundtrip_and_scalar_decoder(layout, kw):
    K, N = 6, 384
    raw, bits, group, kpb = _raw_for(layout, kw, K, N, 11 + layout)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], layout, return_ref=True, **kw)
    q, keep = R.unpack_codes(pk, K, N, layout, **kw)
    keep_in = R.unpack_bits(raw["mask"], N)
    if layout in R.DENSE_FAMILY:
        zi = np.repeat(pk["zero"].astype(np.int32), group, axis=1)
        assert np.array_equal(q, np.where(keep_in, raw["q"], zi))
    else:
        assert np.array_equal(keep, keep_in)
        assert np.array_equal(q, raw["q"].astype(np.int32) * keep_in)
    W = R.dequant(pk, K, N, layout, **kw)
    assert np.array_equal(W, pk["W_ref"])
    Wc = R.dequant(pk, K, N, layout, col_scale=raw["col_scale"], **kw)
    Ws = R.dequant_scalar(pk, K, N, layout, col_scale=raw["col_scale"], **kw)
    assert np.array_equal(Wc, Ws)
    # float64 witness rounded once to float32
    G = N // group
    w64 = (q.astype(np.float64) - np.repeat(pk["zero"].astype(np.float64), group, 1)) * \
        np.repeat(pk["scale"].astype(np.float64), group, 1) * raw["col_scale"].astype(np.float64)[None]
    if layout not in R.DENSE_FAMILY:
        w64 = w64 * keep
    assert np.array_equal(Wc, w64.astype(np.float32))


def test_fused_col_scale_rows():
    K, N = 8, 256
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=5, block=32)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.BLK1632_4)
    rng = np.random.default_rng(0)
    cs2 = (rng.random((2, N)) + 0.5).astype(np.float16)
    cs3 = (rng.random((3, N)) + 0.5).astype(np.float16)
    W0 = R.dequant(pk, K, N, R.BLK1632_4)
    W2 = R.dequant(pk, K, N, R.BLK1632_4, col_scale=cs2)
    assert np.array_equal(W2[0::2], W0[0::2] * cs2[0].astype(np.float32))
    assert np.array_equal(W2[1::2], W0[1::2] * cs2[1].astype(np.float32))
    W3 = R.dequant(pk, K, N, R.BLK1632_4, col_scale=cs3, cs_splits=(4, 2))
    for r, c in zip(range(8), [0, 0, 0, 0, 1, 1, 2, 2]):
        assert np.array_equal(W3[r], W0[r] * cs3[c].astype(np.float32))
    assert np.array_equal(W2, R.dequant_scalar(pk, K, N, R.BLK1632_4, col_scale=cs2))
    assert np.array_equal(W3, R.dequant_scalar(pk, K, N, R.BLK1632_4, col_scale=cs3, cs_splits=(4, 2)))


# ------------------------------------------------------------------ exact zeros / zero repair
def test_pruned_positions_exactly_zero_even_off_grid():
    # restates prod/verify.py:137-145 and test_gemv.py:403-455 on the dequantised weight
    K, N = 8, 256
    raw = R.synth_raw_matrix(K, N, 0.5, 4, seed=9, block=32)
    keep = R.unpack_bits(raw["mask"], N)
    off = np.full((K, N // 128), 15 + 37, np.float16)
    for layout in (R.BLK1632_4, R.BLKC):
        kw = {} if layout == R.BLK1632_4 else dict(bits=4, group=128, keep_per_block=16)
        pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], off, layout, fix_zero=False, **kw)
        assert (pk["zero"] == 52).all()
        W = R.dequant(pk, K, N, layout, col_scale=raw["col_scale"], **kw)
        assert (W[~keep] == 0).all() and (W[keep] != 0).any()
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.DENSE4)
    W = R.dequant(pk, K, N, R.DENSE4, col_scale=raw["col_scale"])
    assert (W[~keep] == 0).all()


def test_fix_zero_range_invariants():
    K, N, G = 16, 256, 2
    rng = np.random.default_rng(4)
    keep = rng.random((K, N)) > 0.5
    q = rng.integers(0, 16, (K, N)).astype(np.float32)
    scale = (rng.random((K, G)) * 0.01 + 0.001).astype(np.float16)
    zero = rng.integers(0, 16, (K, G)).astype(np.float16)
    zero[0, 0], zero[3, 1], zero[7, 0] = -6, 40, -1      # off-grid groups
    keep[7, :128] = False                                # an empty off-grid group
    qf, sc, zi, n = R.fix_zero_range(q, scale, zero, keep, 15)
    assert n == 3 and zi.min() >= 0 and zi.max() <= 15
    good = ~((np.rint(zero.astype(np.float32)) < 0) | (np.rint(zero.astype(np.float32)) > 15))
    g3 = np.repeat(good, 128, axis=1)
    assert np.array_equal(qf[g3], q[g3]) and np.array_equal(sc[good], scale.astype(np.float32)[good])
    assert np.array_equal(zi[good], zero.astype(np.int32)[good])
    # the repaired groups still reproduce their survivors to within half a (new) step
    v_old = (q - np.repeat(np.rint(zero.astype(np.float32)), 128, 1)) * np.repeat(scale.astype(np.float32), 128, 1)
    v_new = (qf - np.repeat(zi.astype(np.float32), 128, 1)) * np.repeat(sc, 128, 1)
    err = np.abs(v_new - v_old)[keep & ~g3]
    assert err.max() <= 0.5001 * sc[~good].max()
    assert zi[7, 0] == 0 and sc[7, 0] == np.float32(1e-12)
    # packing after the repair gives exact zeros in the dense layout
    pk = R.pack_matrix(R.pack_bits(keep), q, scale, zero, R.DENSE4)
    assert pk["n_zero_fixed"] == 3
    W = R.dequant(pk, K, N, R.DENSE4)
    assert (W[~keep] == 0).all()


def test_blk_rejects_wrong_cardinality():
    raw = R.synth_raw_matrix(4, 256, 0.5, 4, seed=1, block=0)
    with pytest.raises(ValueError):
        R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.BLK1632_4)


def test_synth_mask_cardinality():
    for s, want in ((0.3, 23), (0.5, 16), (0.7, 10)):
        raw = R.synth_raw_matrix(8, 256, s, 3, seed=2, block=32)
        cnt = R.unpack_bits(raw["mask"], 256).reshape(8, 8, 32).sum(-1)
        assert (cnt == want).all()
    raw = R.synth_raw_matrix(64, 512, 0.5, 4, seed=2)
    keep = R.unpack_bits(raw["mask"], 512)
    assert abs(keep.mean() - 0.5) < 1e-3
    assert (raw["q"][~keep] == 0).all()


def test_rtn_dense_zero_inclusive():
    rng = np.random.default_rng(1)
    W = rng.normal(0, 0.02, (4, 256)).astype(np.float32) + 0.05
    q, s, z = R.rtn_dense(W, 4)
    assert z.min() >= 0 and z.max() <= 15
    deq = (q.reshape(4, 2, 128) - z[..., None].astype(np.float32)) * s[..., None].astype(np.float32)
    assert np.abs(deq.reshape(4, 256) - W).max() <= 0.51 * s.astype(np.float32).max() + 1e-6


def test_blob_alignment():
    raw = R.synth_raw_matrix(4, 256, 0.5, 4, seed=1, block=32)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], R.BLK1632_4)
    blob, offs = R.make_blob(pk, raw["col_scale"])
    assert all(o % 256 == 0 for o in offs.values()) and blob.size % 256 == 0
    assert np.array_equal(blob[offs["data"]: offs["data"] + pk["data"].size], pk["data"])
    assert R.stream_bytes(pk) == 4 * 96 + 4 * 2 * 2 + 4 * 2


# ------------------------------------------------------------------ tile-interleaved order
@pytest.mark.parametrize("layout,kw", [c for c in LAYOUT_CASES if c[0] not in R.SPARSE_FAMILY])
def test_tile16_is_a_byte_permutation(layout, kw):
    K, N = 40, 384                       # 2.5 tiles: exercises the zero padding rows
    raw, bits, group, kpb = _raw_for(layout, kw, K, N, 21)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], layout, **kw)
    t = R.tile16(pk, K, N, layout, **kw)
    stride = R.row_stride(layout, N, bits, group, kpb)
    G = N // group
    assert t["data"].size == 48 * stride + 512 and t["scale"].size == 48 * G and t["zero"].size == 48 * G
    rng = np.random.default_rng(0)
    for _ in range(200):                 # the closed-form index map, element by element
        k, o, g = int(rng.integers(K)), int(rng.integers(stride)), int(rng.integers(G))
        assert t["data"][(k // 16) * 16 * stride + ((o // 16) * 16 + k % 16) * 16 + o % 16] == pk["data"][k * stride + o]
        assert t["scale"][((k // 16) * G + g) * 16 + k % 16] == pk["scale"].reshape(K, G)[k, g]
        assert t["zero"][((k // 16) * G + g) * 16 + k % 16] == pk["zero"].reshape(K, G)[k, g]
    assert sorted(t["data"][: 48 * stride].tolist()) == sorted(pk["data"][: K * stride].tolist() + [0] * (8 * stride))
    u = R.untile16(t, K, N, layout, **kw)
    assert np.array_equal(u["data"], pk["data"]) and np.array_equal(u["scale"], pk["scale"].reshape(K, G))
    assert np.array_equal(u["zero"], pk["zero"].reshape(K, G))
    assert np.array_equal(R.dequant(u, K, N, layout, **kw), R.dequant(pk, K, N, layout, **kw))
