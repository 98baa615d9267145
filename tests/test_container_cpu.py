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
    assert man["format"] == "CBK1" and len(man["layers"]) == 2
    e = man["layers"][0]["q_proj"]
    # the reference's manifest fields and their known values for this shape (docs/FORMAT.md:26-35)
    assert e["layout"] == 6 and e["layout_name"] == "BLK1632_4" and e["G"] == 2 and e["cs_rows"] == 1
    assert e["stream_bytes"] == 64 * (3 * 256 // 8) + 64 * 2 * 3 and abs(e["bpw"] - 3.1875) < 1e-12
    assert e["arrays"]["data"]["bytes"] == 64 * 96 + 64 and all(a["off"] % 256 == 0 for a in e["arrays"].values())
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


def test_alias_entries_point_into_the_fused_matrix(tmp_path):
    """qkv rows concatenated (docs/FORMAT.md:134-151): data / scale / zero written once, the
    q / k / v entries carry alias_of and offsets into the fused arrays, own col_scale each."""
    Kq, Kk, N = 64, 32, 256
    q = F.synth_packed(Kq, N, F.BLK1632_4, seed=1)
    k = F.synth_packed(Kk, N, F.BLK1632_4, seed=2)
    v = F.synth_packed(Kk, N, F.BLK1632_4, seed=3)
    stride = F.row_stride(F.BLK1632_4, N)
    G = N // 128
    rows = lambda p: p.array("data")[: p.K * stride]
    fused = F.from_arrays(torch.cat([rows(q), rows(k), rows(v), torch.zeros(64, dtype=torch.uint8)]),
                          torch.cat([p.array("scale") for p in (q, k, v)]), torch.cat([p.array("zero") for p in (q, k, v)]),
                          torch.cat([p.array("col_scale") for p in (q, k, v)]).reshape(3, N), Kq + 2 * Kk, N, F.BLK1632_4,
                          cs_splits=(Kq, Kk))
    man = Ct.write_container(str(tmp_path), [{"qkv": fused}])
    ent = man["layers"][0]
    f = ent["qkv"]
    assert f["cs_rows"] == 3 and f["cs_splits"] == [Kq, Kk]
    row0 = 0
    for name, p, csr in (("q_proj", q, 0), ("k_proj", k, 1), ("v_proj", v, 2)):
        ent[name] = {"K": p.K, "N": N, "G": G, "layout": 6, "layout_name": "BLK1632_4", "cs_rows": 1, "alias_of": "qkv",
                     "n_survivors": 0, "stream_bytes": p.stream_bytes(), "bpw": p.bpw(), "blob": f["blob"],
                     "arrays": {"data": {"off": f["arrays"]["data"]["off"] + row0 * stride, "bytes": p.K * stride + 64},
                                "scale": {"off": f["arrays"]["scale"]["off"] + row0 * G * 2, "bytes": p.K * G * 2},
                                "zero": {"off": f["arrays"]["zero"]["off"] + row0 * G, "bytes": p.K * G},
                                "col_scale": {"off": f["arrays"]["col_scale"]["off"] + csr * N * 2, "bytes": N * 2}}}
        row0 += p.K
    with open(os.path.join(str(tmp_path), "manifest.json"), "w") as fh:
        json.dump(man, fh)
    man2, layers = Ct.read_container(str(tmp_path))
    for name, p in (("q_proj", q), ("k_proj", k), ("v_proj", v)):
        a = layers[0][name]
        cs = p.array("col_scale").numpy().reshape(1, N)
        assert np.array_equal(R.dequant(_pk(a), a.K, N, 6, col_scale=a.array("col_scale").numpy().reshape(1, N)),
                              R.dequant(_pk(p), p.K, N, 6, col_scale=cs))
    # totals skip the aliases
    assert Ct.total_stream_bytes(man2) == fused.stream_bytes()
    assert "q_proj" not in Ct.read_container(str(tmp_path), include_aliases=False)[1][0]


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
    man["layers"][0]["q_proj"]["stream_bytes"] += 64
    json.dump(man, open(d + "/manifest.json", "w"))
    assert any("bytes per weight" in p for p in Ct.check_container(d, strict=False)["problems"])

    d = variant("mask")
    man = json.load(open(d + "/manifest.json"))
    off = man["layers"][0]["q_proj"]["arrays"]["data"]["off"]
    with open(d + "/layer_00.bin", "r+b") as f:
        f.seek(off)
        b = f.read(1)
        f.seek(off)
        f.write(bytes([b[0] ^ 1]))                                   # one more or one fewer survivor in block 0 of row 0
    assert any("survivors per 32-column block" in p for p in Ct.check_container(d, strict=False)["problems"])
