"""Writes tests/golden/fixed_stride.npz: bytes of the reference's packer
(src/cobaltkernel/pack_cobalt.py:98-250 `pack_matrix`) and its own decode of them
(`dequant_reference`, :277-334) for the fixed-stride layouts DENSE4, DENSE8, BLK1632_4 and
BLK1632_6 on small seeded RAW matrices with a 16-of-32 mask, one off-grid zero point per matrix
(the 0-inclusive-hull repair, :55-87) and a column scale; plus a row-interleaved gate/up pair
packed the way `pack_artifact` does it (:654-667) with its [2, N] column scales, whose expected
decode is the reference's decode of gate and of up, each under its own column scale, interleaved.

Run in the development container only (needs the reference checkout); the committed .npz is what
the tests read.

    python tests/golden/make_fixed_stride_vectors.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = [("DENSE4", 4), ("DENSE8", 8), ("BLK1632_4", 4), ("BLK1632_6", 6)]


def raw(seed, K, N, bits):
    g = torch.Generator().manual_seed(seed)
    G = N // 128
    imp = torch.rand(K, N // 32, 32, generator=g)
    keep = torch.zeros(K, N // 32, 32, dtype=torch.bool).scatter_(-1, imp.topk(16, -1).indices, True).reshape(K, N)
    q = torch.randint(0, 1 << bits, (K, N), generator=g).to(torch.uint8) * keep.to(torch.uint8)
    scale = (torch.rand(K, G, generator=g) * 0.01 + 0.001).half()
    zero = torch.randint(0, 1 << bits, (K, G), generator=g).half()
    zero[1, 0] = -3.0                                          # off the grid: survivors all positive
    zero[2 % K, G - 1] = float((1 << bits) + 2)                # off the grid: survivors all negative
    cs = (torch.rand(N, generator=g) * 1.5 + 0.5).half()
    mask = torch.from_numpy(np.packbits(keep.numpy(), axis=-1, bitorder="little"))
    return mask, q, scale, zero, cs


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec = importlib.util.spec_from_file_location("ref_pack_cobalt", os.path.join(ref, "src/cobaltkernel/pack_cobalt.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = {}
    for ci, (name, bits) in enumerate(CASES):
        K, N = 6, 256 + 128 * (ci % 2)
        mask, q, scale, zero, cs = raw(10 + ci, K, N, bits)
        layout = getattr(mod, name)
        p = name + "_"
        out[p + "mask"] = mask.numpy(); out[p + "q"] = q.numpy(); out[p + "scale_in"] = scale.numpy()
        out[p + "zero_in"] = zero.numpy(); out[p + "col_scale"] = cs.numpy()
        pk = mod.pack_matrix(mask, q.float(), scale, zero, layout, bits=bits)
        out[p + "data"] = np.asarray(pk["data"]); out[p + "scale"] = np.asarray(pk["scale"]); out[p + "zero"] = np.asarray(pk["zero"])
        out[p + "nsurv"] = np.int64(pk["n_survivors"]); out[p + "nfixed"] = np.int64(pk["n_zero_fixed"])
        out[p + "W"] = mod.dequant_reference(pk, K, N, layout, col_scale=cs.float(), bits=bits).numpy().astype(np.float32)
        print(name, "K,N", (K, N), "data bytes", len(pk["data"]), "survivors", pk["n_survivors"], "zeros repaired", pk["n_zero_fixed"])

    # gate/up: rows interleaved before packing, column scales stacked [2, N]
    K, N = 5, 256
    gm, gq, gs, gz, gcs = raw(30, K, N, 4)
    um, uq, us, uz, ucs = raw(31, K, N, 4)
    il = lambda a, b: torch.stack([a, b], 1).reshape(2 * K, -1)
    pk = mod.pack_matrix(il(gm, um), il(gq, uq).float(), il(gs, us), il(gz, uz), mod.BLK1632_4, bits=4)
    parts = []
    for (m, q, s, z, cs) in ((gm, gq, gs, gz, gcs), (um, uq, us, uz, ucs)):
        one = mod.pack_matrix(m, q.float(), s, z, mod.BLK1632_4, bits=4)
        parts.append(mod.dequant_reference(one, K, N, mod.BLK1632_4, col_scale=cs.float()).numpy())
    for nm, (m, q, s, z, cs) in (("gate", (gm, gq, gs, gz, gcs)), ("up", (um, uq, us, uz, ucs))):
        out[f"gateup_{nm}_mask"] = m.numpy(); out[f"gateup_{nm}_q"] = q.numpy(); out[f"gateup_{nm}_scale_in"] = s.numpy()
        out[f"gateup_{nm}_zero_in"] = z.numpy()
    out["gateup_col_scale"] = torch.stack([gcs, ucs], 0).numpy()
    out["gateup_data"] = np.asarray(pk["data"]); out["gateup_scale"] = np.asarray(pk["scale"]); out["gateup_zero"] = np.asarray(pk["zero"])
    out["gateup_W"] = np.stack(parts, 1).reshape(2 * K, N).astype(np.float32)
    path = os.path.join(HERE, "fixed_stride.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
