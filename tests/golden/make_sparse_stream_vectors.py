"""Writes tests/golden/sparse_stream.npz: bytes of the reference's packer
(src/cobaltkernel/pack_cobalt.py:98-250 `pack_matrix`) and its own decode of them
(`dequant_reference`, :277-334) for the variable-length layouts SPARSE4, SPARSE4X and SPARSE4E
on small seeded RAW matrices.

The fixed-stride layouts are pinned by hand-computed byte vectors; for the survivor streams
(per-row offsets, per-group offsets, even-nibble group padding, 16-byte row alignment) this
build's packer and decoder were written from one reading of the same text and only check each
other, so the bytes are taken from the reference itself.  Run in the development container
only (needs the reference checkout); the committed .npz is what the tests read.

    python tests/golden/make_sparse_stream_vectors.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def raw(seed, K, N, density):
    g = torch.Generator().manual_seed(seed)
    G = N // 128
    keep = torch.rand(K, N, generator=g) < density
    keep[0, :128] = False                                     # an empty group
    keep[1, 128:256] = True                                   # a full group
    keep[2 % K] = False                                       # an empty row
    q = torch.randint(0, 16, (K, N), generator=g).float()
    scale = (torch.rand(K, G, generator=g) * 0.01 + 0.001).half()
    zero = torch.randint(0, 16, (K, G), generator=g).half()
    mask = torch.from_numpy(np.packbits(keep.numpy(), axis=-1, bitorder="little"))
    return mask, q, scale, zero


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec = importlib.util.spec_from_file_location("ref_pack_cobalt", os.path.join(ref, "src/cobaltkernel/pack_cobalt.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = {}
    cases = [(0, 5, 256, 0.5), (1, 4, 384, 0.3), (2, 6, 256, 0.8)]
    for seed, K, N, dens in cases:
        mask, q, scale, zero = raw(seed, K, N, dens)
        p = f"c{seed}_"
        out[p + "mask"] = mask.numpy(); out[p + "q"] = q.numpy().astype(np.uint8)
        out[p + "scale"] = scale.numpy(); out[p + "zero"] = zero.numpy()
        for name in ("SPARSE4", "SPARSE4X", "SPARSE4E"):
            layout = getattr(mod, name)
            pk = mod.pack_matrix(mask, q.clone(), scale, zero, layout, return_ref=True)
            out[p + name + "_data"] = np.asarray(pk["data"]); out[p + name + "_row_off"] = np.asarray(pk["row_off"])
            out[p + name + "_scale"] = np.asarray(pk["scale"]); out[p + name + "_zero"] = np.asarray(pk["zero"])
            out[p + name + "_nsurv"] = np.int64(pk["n_survivors"])
            W = mod.dequant_reference(pk, K, N, layout)
            out[p + name + "_W"] = np.asarray(W.cpu().numpy() if hasattr(W, "cpu") else W, np.float32)
            print(p, name, "data bytes", len(pk["data"]), "survivors", pk["n_survivors"], "keys", sorted(pk.keys()))
    path = os.path.join(HERE, "sparse_stream.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
