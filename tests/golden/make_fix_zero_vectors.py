"""Writes tests/golden/fix_zero_range.npz: inputs and outputs of the reference's zero-point
repair (src/cobaltkernel/pack_cobalt.py:55-87 `_fix_zero_range`) on small seeded cases.

The exact re-derived (q, scale, zero) of an off-grid group is the one function of the packer
that no hand vector, closed form or invariant fixes bit for bit, so its vectors are taken from
the reference itself.  Run in the development container only (needs the reference checkout);
the committed .npz is what the tests read.

    python tests/golden/make_fix_zero_vectors.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec = importlib.util.spec_from_file_location("ref_pack_cobalt", os.path.join(ref, "src/cobaltkernel/pack_cobalt.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = {}
    cases = [(0, 6, 256, 15), (1, 5, 384, 15), (2, 4, 256, 63)]          # (seed, K, N, nlevels)
    for seed, K, N, nlevels in cases:
        g = torch.Generator().manual_seed(seed)
        G = N // 128
        keep = torch.rand(K, N, generator=g) < 0.5
        keep[0, :128] = False                                              # an empty group
        qf = torch.randint(0, nlevels + 1, (K, N), generator=g).float()
        scale = (torch.rand(K, G, generator=g) * 0.01 + 0.001).half()
        zero = torch.randint(0, nlevels + 1, (K, G), generator=g).float()
        # off-grid zero points on both sides, as fp16 (rounded integers) like the RAW schema
        zero[0, 0] = -3.0; zero[1, 1] = nlevels + 7.0; zero[2, 0] = -40.0; zero[3, G - 1] = nlevels + 1.0
        zero = zero.half()
        q2, s2, z2, n = mod._fix_zero_range(qf.clone(), scale, zero, keep, nlevels)
        p = f"c{seed}_"
        out[p + "keep"] = keep.numpy(); out[p + "q"] = qf.numpy(); out[p + "scale"] = scale.numpy()
        out[p + "zero"] = zero.numpy(); out[p + "nlevels"] = np.int32(nlevels)
        out[p + "q_out"] = q2.numpy(); out[p + "scale_out"] = s2.numpy().astype(np.float32)
        out[p + "zero_out"] = z2.numpy().astype(np.int32); out[p + "n_fixed"] = np.int32(n)
    np.savez_compressed(os.path.join(HERE, "fix_zero_range.npz"), **out)
    print("wrote", os.path.join(HERE, "fix_zero_range.npz"), {k: v.shape for k, v in out.items() if k.startswith("c0_")})


if __name__ == "__main__":
    main()
