"""CBK1 directory write/read round trip and the offset-driven handling of row-fused matrices
with `alias_of` entries (CPU)."""
import json
import os

import numpy as np
import torch

from cobalt_amd import container as Ct, format as F
from oracle import cbk_ref as R


def _pk(pm):
    return dict(data=pm.array("data").numpy(), scale=pm.array("scale").numpy().reshape(pm.K, -1),
                zero=pm.array("zero").numpy().reshape(pm.K, -1))


def test_container_round_trip(tmp_path):
    layers = []
    for li in range(2):
        layers.append({"q_proj": F.synth_packed(64, 256, F.BLK1632_4, seed=10 * li),
                       "o_proj": F.synth_packed(48, 384, F.BLKC, 3, 64, 10, seed=10 * li + 1),
                       "down_proj": F.synth_packed(32, 512, F.DENSE4, seed=10 * li + 2)})
    man = Ct.write_container(str(tmp_path), layers, config={"hidden_size": 256})
    assert man["format"] == "CBK1" and man["version"] == 1 and len(man["layers"]) == 2
    # the reference's layer record and entry fields (pack_cobalt.py:414-434, :601-602, :672)
    rec = man["layers"][0]
    assert rec["file"] == "layer_00.bin" and rec["norms"] == {} and set(rec["matrices"]) == {"q_proj", "o_proj", "down_proj"}
    assert rec["bytes"] == os.path.getsize(os.path.join(str(tmp_path), "layer_00.bin")) and rec["bytes"] % 256 == 0
    e = rec["matrices"]["q_proj"]
    assert e["layout"] == 6 and e["layout_name"] == "BLK1632_4" and e["G"] == 2 and e["cs_rows"] == 1
    assert e["stream_bytes"] == 64 * (3 * 256 // 8) + 64 * 2 * 3 and abs(e["bpw"] - 3.1875) < 1e-12
    assert e["arrays"]["data"]["bytes"] == 64 * 96 + 64 and all(a["off"] % 256 == 0 for a in e["arrays"].values())
    assert "n_zero_fixed" in e and "bits" not in e and "blob" not in e
    x = rec["matrices"]["o_proj"]
    assert (x["layout_name"], x["bits"], x["group"], x["keep"]) == ("BLKC", 3, 64, 10)
    man2, back = Ct.read_container(str(tmp_path))
    assert man2 == json.loads(json.dumps(man))
    for li in range(2):
        for name, pm in layers[li].items():
            b = back[li][name]
            assert (b.K, b.N, b.layout, b.bits, b.group, b.keep, b.cs_rows, b.flags) == \
                   (pm.K, pm.N, pm.layout, pm.bits, pm.group, pm.keep, pm.cs_rows, pm.flags)
            for an in ("data", "scale", "zero", "col_scale"):
                assert torch.equal(b.array(an), pm.array(an)), (name, an)
            # both dequantise to the same matrix under the oracle
            kw = dict(bits=pm.bits, group=pm.group, keep_per_block=pm.keep or None)
            cs = pm.array("col_scale").numpy().reshape(1, pm.N)
            assert np.array_equal(R.dequant(_pk(b), b.K, b.N, b.layout, col_scale=cs, **kw),
                                  R.dequant(_pk(pm), pm.K, pm.N, pm.layout, col_scale=cs, **kw))
    # one blob tensor per layer, shared by its matrices
    assert back[0]["q_proj"].blob.data_ptr() == back[0]["o_proj"].blob.data_ptr()
    assert Ct.total_stream_bytes(man) == sum(pm.stream_bytes() for l in layers for pm in l.values())
    assert man["bpw"]["packed_bytes"] == Ct.total_stream_bytes(man)


GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _canon_hash(W):
    import hashlib
    return hashlib.sha256((np.ascontiguousarray(W, dtype=np.float32) + np.float32(0.0)).tobytes()).hexdigest()


def test_reads_a_directory_the_reference_wrote():
    """tests/golden/cbk1_dir is the output of the reference's `pack_artifact` (--fuse-qkv,
    --fuse-gateup, o_proj overridden to DENSE4); cbk1_dir_expect.npz holds the reference's own
    decode of each matrix (hash of all values, four rows in full).  The reader takes the blob from
    `file`, the entries from `matrices`, the three row ranges of qkv from `row_ranges`/`cs_row_of`,
    and the tail-less `data.bytes` of the alias entries as rows only."""
    exp = np.load(os.path.join(GOLD, "cbk1_dir_expect.npz"))
    man, layers = Ct.read_container(os.path.join(GOLD, "cbk1_dir"))
    mats = layers[0]
    assert set(mats) == {"qkv", "q_proj", "k_proj", "v_proj", "o_proj", "down_proj", "gateup"}
    qkv = mats["qkv"]
    assert (qkv.K, qkv.N, qkv.cs_rows, qkv.cs_splits, qkv.layout) == (256, 256, 3, (128, 64), F.BLK1632_4)
    assert mats["gateup"].cs_rows == 2 and mats["o_proj"].layout == F.DENSE4
    for name in ("q_proj", "k_proj", "v_proj"):
        a, e = mats[name], man["layers"][0]["matrices"][name]
        assert a.data_bytes == e["arrays"]["data"]["bytes"] == a.K * 96            # no tail in an alias
        assert a.offs["data"] == qkv.offs["data"] + e["alias_row_start"] * 96
        assert a.stream_bytes() == e["stream_bytes"]
    for name in ("qkv", "o_proj", "down_proj", "gateup"):
        assert mats[name].stream_bytes() == man["layers"][0]["matrices"][name]["stream_bytes"], name
    assert Ct.total_stream_bytes(man) == man["bpw"]["packed_bytes"]
    for name, pm in mats.items():
        cs = pm.array("col_scale").numpy().reshape(pm.cs_rows, pm.N)
        W = R.dequant(_pk(pm), pm.K, pm.N, pm.layout, col_scale=cs, cs_splits=pm.cs_splits)
        assert np.array_equal(W[exp[f"{name}.rows"]] + np.float32(0), exp[f"{name}.values"] + np.float32(0)), name
        assert _canon_hash(W) == bytes(exp[f"{name}.sha256"]).decode(), name
    rep = Ct.check_container(os.path.join(GOLD, "cbk1_dir"))
    assert rep["ok"] and abs(rep["bpw"] - man["bpw"]["bpw_packed"]) < 1e-9
    assert "0:q_proj" not in rep["matrices"] and rep["matrices"]["0:qkv"]["block_survivors"] == [16, 16]


def test_writer_emits_the_reference_schema_for_fused_matrices(tmp_path):
    """Rewriting the matrices of the reference's directory gives a manifest whose entries carry
    the same fields and the same values as the reference's, offsets included."""
    ref_man, layers = Ct.read_container(os.path.join(GOLD, "cbk1_dir"), include_aliases=False)
    man = Ct.write_container(str(tmp_path), layers)
    ref_mats, mats = ref_man["layers"][0]["matrices"], man["layers"][0]["matrices"]
    assert list(mats) == list(ref_mats)
    for name, e in ref_mats.items():
        m = mats[name]
        assert set(m) == set(e), (name, set(m) ^ set(e))
        for k in e:
            if k == "n_survivors" and e.get("alias_of"):
                continue                                              # apportioned by rows when written from a fused matrix
            assert m[k] == e[k], (name, k, m[k], e[k])
    assert man["layers"][0]["bytes"] == ref_man["layers"][0]["bytes"]
    a = open(os.path.join(GOLD, "cbk1_dir", "layer_00.bin"), "rb").read()
    assert open(os.path.join(str(tmp_path), "layer_00.bin"), "rb").read() == a
    for k in ("format", "version", "group_size", "bits", "layout", "fuse_gateup", "fuse_qkv", "mixed_layout"):
        assert man[k] == ref_man[k], k
    assert set(ref_man) - set(man) == set()


def test_alias_entries_point_into_the_fused_matrix(tmp_path):
    """qkv rows concatenated (docs/FORMAT.md:134-151): data / scale / zero written once, the
    q / k / v entries carry alias_of and byte ranges inside the fused arrays, own col_scale each."""
    Kq, Kk, N = 64, 32, 256
    q = F.synth_packed(Kq, N, F.BLK1632_4, seed=1)
    k = F.synth_packed(Kk, N, F.BLK1632_4, seed=2)
    v = F.synth_packed(Kk, N, F.BLK1632_4, seed=3)
    fused = F.fuse_rows([q, k, v])
    man = Ct.write_container(str(tmp_path), [{"qkv": fused}])
    ent = man["layers"][0]["matrices"]
    f = ent["qkv"]
    assert f["cs_rows"] == 3 and f["row_ranges"] == {"q_proj": [0, Kq], "k_proj": [Kq, Kq + Kk], "v_proj": [Kq + Kk, Kq + 2 * Kk]}
    assert f["cs_row_of"] == {"q_proj": 0, "k_proj": 1, "v_proj": 2} and f["fused_from"] == ["q_proj", "k_proj", "v_proj"]
    assert ent["k_proj"]["alias_of"] == "qkv" and ent["k_proj"]["alias_row_start"] == Kq
    assert ent["k_proj"]["arrays"]["data"] == {"off": f["arrays"]["data"]["off"] + Kq * 96, "bytes": Kk * 96}
    man2, layers = Ct.read_container(str(tmp_path))
    assert layers[0]["qkv"].cs_splits == (Kq, Kk)
    for name, p in (("q_proj", q), ("k_proj", k), ("v_proj", v)):
        a = layers[0][name]
        cs = p.array("col_scale").numpy().reshape(1, N)
        assert np.array_equal(R.dequant(_pk(a), a.K, N, 6, col_scale=a.array("col_scale").numpy().reshape(1, N)),
                              R.dequant(_pk(p), p.K, N, 6, col_scale=cs))
    # totals skip the aliases
    assert Ct.total_stream_bytes(man2) == fused.stream_bytes()
    assert "q_proj" not in Ct.read_container(str(tmp_path), include_aliases=False)[1][0]


def test_entries_that_do_not_fit_are_refused(tmp_path):
    """A manifest entry is outside input: an array past the blob, a byte count that is not rows x
    stride, row ranges that do not tile the rows and a layer record without `matrices` each raise."""
    import pytest
    Ct.write_container(str(tmp_path), [{"qkv": F.fuse_rows([F.synth_packed(32, 256, F.BLK1632_4, seed=s) for s in (1, 2, 3)])}])
    mp = os.path.join(str(tmp_path), "manifest.json")
    good = json.load(open(mp))

    def with_change(fn):
        man = json.loads(json.dumps(good))
        fn(man["layers"][0]["matrices"], man)
        json.dump(man, open(mp, "w"))
        with pytest.raises(ValueError):
            Ct.read_container(str(tmp_path))

    with_change(lambda m, _: m["q_proj"]["arrays"]["data"].update(off=10 ** 9))
    with_change(lambda m, _: m["qkv"]["arrays"]["data"].update(bytes=m["qkv"]["arrays"]["data"]["bytes"] - 16))
    with_change(lambda m, _: m["k_proj"]["arrays"]["data"].update(bytes=m["k_proj"]["arrays"]["data"]["bytes"] + 64))
    with_change(lambda m, _: m["qkv"]["row_ranges"].update(k_proj=[40, 64]))
    with_change(lambda m, _: m["qkv"].pop("cs_row_of"))
    with_change(lambda m, _: m["v_proj"]["arrays"]["zero"].update(bytes=5))
    with_change(lambda m, man: man["layers"].__setitem__(0, man["layers"][0]["matrices"]))
    json.dump(good, open(mp, "w"))
    Ct.read_container(str(tmp_path))


def test_check_container_finds_what_is_wrong(tmp_path):
    """The structural half of the checker (the role of src/prod/verify.py:64-152) on the CPU:
    a good directory passes; a truncated blob, a wrong byte count and a block with the wrong
    number of survivors are each reported."""
    import pytest
    import shutil
    layers = [{"q_proj": F.synth_packed(64, 256, F.BLK1632_4, seed=1),
               "down_proj": F.synth_packed(32, 512, F.BLKC, 3, 64, 10, seed=2)}]
    good = str(tmp_path / "good")
    Ct.write_container(good, layers)
    rep = Ct.check_container(good)
    assert rep["ok"] and abs(rep["bpw"] - Ct.total_stream_bytes(json.load(open(good + "/manifest.json"))) * 8.0 / (64 * 256 + 32 * 512)) < 1e-9
    assert rep["matrices"]["0:q_proj"]["block_survivors"] == [16, 16] and rep["matrices"]["0:down_proj"]["block_survivors"] == [10, 10]

    def variant(name):
        d = str(tmp_path / name)
        shutil.copytree(good, d)
        return d

    d = variant("short")
    with open(d + "/layer_00.bin", "r+b") as f:
        f.truncate(1000)
    rep = Ct.check_container(d, strict=False)
    assert not rep["ok"] and any("runs past the blob" in p for p in rep["problems"])
    with pytest.raises(ValueError):
        Ct.check_container(d)

    d = variant("bytes")
    man = json.load(open(d + "/manifest.json"))
    man["layers"][0]["matrices"]["q_proj"]["stream_bytes"] += 64
    json.dump(man, open(d + "/manifest.json", "w"))
    assert any("bytes per weight" in p for p in Ct.check_container(d, strict=False)["problems"])

    d = variant("mask")
    man = json.load(open(d + "/manifest.json"))
    off = man["layers"][0]["matrices"]["q_proj"]["arrays"]["data"]["off"]
    with open(d + "/layer_00.bin", "r+b") as f:
        f.seek(off)
        b = f.read(1)
        f.seek(off)
        f.write(bytes([b[0] ^ 1]))                                   # one more or one fewer survivor in block 0 of row 0
    assert any("survivors per 32-column block" in p for p in Ct.check_container(d, strict=False)["problems"])
