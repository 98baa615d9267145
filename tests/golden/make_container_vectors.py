"""Writes tests/golden/cbk1_dir/ (manifest.json + layer_00.bin) and tests/golden/cbk1_dir_expect.npz:
a tiny CBK1 directory produced by the reference's own writer
(src/cobaltkernel/pack_cobalt.py:561-714 `pack_artifact`, with --fuse-qkv and --fuse-gateup and a
DENSE4 override for o_proj) and the reference's own decode of every matrix in it
(`dequant_reference`, :277-334).

What it pins is the directory schema, which no other fixture of the reference holds: the layer
records (`file`, `matrices`, `norms`, `bytes`), the fused `qkv` entry with `row_ranges` and
`cs_row_of`, the `alias_of` entries whose `data.bytes` carries no tail, and the row-interleaved
`gateup` with its [2, N] column scales.  Run in the development container only (needs the
reference checkout); the committed files are what the tests read.

    python tests/golden/make_container_vectors.py [/root/reference]
"""
import hashlib
import importlib.util
import json
import os
import shutil
import sys
import tempfile

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
HIDDEN, Q_OUT, KV_OUT, INTER = 256, 128, 64, 128
SHAPES = {"q_proj": (Q_OUT, HIDDEN), "k_proj": (KV_OUT, HIDDEN), "v_proj": (KV_OUT, HIDDEN), "o_proj": (HIDDEN, Q_OUT),
          "gate_proj": (INTER, HIDDEN), "up_proj": (INTER, HIDDEN), "down_proj": (HIDDEN, INTER)}


def canon_hash(W):
    """sha256 of the fp32 bytes with -0.0 folded into +0.0 (a pruned weight under a non-zero
    zero point decodes to -0.0 in the reference's arithmetic)."""
    W = np.ascontiguousarray(W, dtype=np.float32) + np.float32(0.0)
    return hashlib.sha256(W.tobytes()).hexdigest()


def sample_rows(K):
    return sorted({0, 1, K // 2, K - 1})


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec = importlib.util.spec_from_file_location("ref_pack_cobalt", os.path.join(ref, "src/cobaltkernel/pack_cobalt.py"))
    P = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(P)
    from safetensors.torch import save_file

    out = os.path.join(HERE, "cbk1_dir")
    shutil.rmtree(out, ignore_errors=True)
    cwd = os.getcwd()
    with tempfile.TemporaryDirectory() as tmp:
        os.chdir(tmp)
        try:
            os.makedirs("raw")
            raws, tensors = {}, {}
            for i, (name, (K, N)) in enumerate(SHAPES.items()):
                raws[name] = P.synth_raw_matrix(K, N, sparsity=0.5, bits=4, seed=100 + i, block=32)
                for f, t in raws[name].items():
                    tensors[f"model.layers.0.{name}.{f}"] = t.contiguous()
            save_file(tensors, "raw/layer_00.safetensors")
            json.dump({"config": {"group_size": 128, "bits": 4}}, open("raw/manifest.json", "w"))
            man = P.pack_artifact("raw", out, layout=P.BLK1632_4, fuse_gateup=True, fuse_qkv=True, bits=4, device="cpu",
                                  layout_over={"o_proj": P.DENSE4})
        finally:
            os.chdir(cwd)

    # the reference's decode of what it wrote, matrix by matrix, from the bytes in the blob
    blob = np.fromfile(os.path.join(out, "layer_00.bin"), dtype=np.uint8)
    mats = man["layers"][0]["matrices"]

    def arrays_of(e):
        a = e["arrays"]
        take = lambda n: blob[a[n]["off"]: a[n]["off"] + a[n]["bytes"]]
        return dict(data=take("data"), scale=take("scale").view(np.float16).reshape(e["K"], e["G"]),
                    zero=take("zero").reshape(e["K"], e["G"])), (take("col_scale").view(np.float16) if "col_scale" in a else None)

    expect = {}
    for name in ("q_proj", "k_proj", "v_proj", "o_proj", "down_proj"):
        e = mats[name]
        pk, cs = arrays_of(e)
        assert cs is not None and cs.size == e["N"]
        expect[name] = P.dequant_reference(pk, e["K"], e["N"], e["layout"], col_scale=cs.astype(np.float32)).numpy()
    # fused matrices: the reference decodes them part by part, each part with its own column scale
    expect["qkv"] = np.concatenate([expect[n] for n in ("q_proj", "k_proj", "v_proj")], 0)
    parts = []
    for n in ("gate_proj", "up_proj"):
        r = raws[n]
        pk = P.pack_matrix(r["mask"], r["q"].float(), r["scale"], r["zero"], P.BLK1632_4, bits=4, device=torch.device("cpu"))
        parts.append(P.dequant_reference(pk, *SHAPES[n], P.BLK1632_4, col_scale=r["col_scale"].float()).numpy())
    expect["gateup"] = np.stack(parts, 1).reshape(2 * INTER, HIDDEN)

    save = {}
    for name, W in expect.items():
        K = W.shape[0]
        assert (K, W.shape[1]) == (mats[name]["K"], mats[name]["N"]), name
        save[f"{name}.sha256"] = np.frombuffer(canon_hash(W).encode(), dtype=np.uint8)
        save[f"{name}.rows"] = np.array(sample_rows(K), dtype=np.int64)
        save[f"{name}.values"] = W[sample_rows(K)].astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "cbk1_dir_expect.npz"), **save)
    print("wrote", out, os.path.getsize(os.path.join(out, "layer_00.bin")), "bytes;",
          {k: (v["K"], v["N"], v["layout_name"], v.get("alias_of")) for k, v in mats.items()})


if __name__ == "__main__":
    main()
