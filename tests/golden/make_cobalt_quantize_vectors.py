"""Writes tests/golden/cobalt_quantize.npz: inputs and outputs of the reference's compressor
(src/cobaltkernel/cobalt_math.py:336-394 `cobalt_quantize`, shipped path: quant_mode 'rtn',
clip 'none') on small seeded matrices.

What `torch.kthvalue` / `torch.topk` do with near-ties, which of the Cholesky and inverse paths
the OBS step takes and how the float32 roundings of the whole chain fall is fixed by no closed
form, so the vectors of this one function are taken from the reference itself.  Run in the
development container only (needs the reference checkout); the committed .npz is what the
tests read.

    python tests/golden/make_cobalt_quantize_vectors.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

# (seed, K, N, calibration rows, sparsity, beta, bits, group, mask_block)
CASES = [(0, 24, 256, 32, 0.5, 0.5, 4, 128, 0),
         (1, 16, 256, 48, 0.5, 0.5, 4, 128, 32),
         (2, 16, 256, 32, 0.6875, 0.5, 3, 64, 32),
         (3, 12, 128, 64, 0.3, 0.3, 2, 64, 0)]


def inputs(seed, K, N, T):
    """W ~ N(0, 0.02) with a few heavy columns, X ~ N(0, 1) with a few loud channels; H = X^T X
    accumulated in float64 and rounded once, so that every machine forms the same H."""
    g = torch.Generator().manual_seed(seed)
    W = torch.randn(K, N, generator=g) * 0.02
    W[:, torch.randperm(N, generator=g)[:3]] *= 10.0
    X = torch.randn(T, N, generator=g)
    X[:, torch.randperm(N, generator=g)[:4]] *= 6.0
    H = (X.double().T @ X.double()).float()
    return W, X, H


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec = importlib.util.spec_from_file_location("ref_cobalt_math", os.path.join(ref, "src/cobaltkernel/cobalt_math.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = {}
    for seed, K, N, T, sp, beta, bits, group, mb in CASES:
        W, X, H = inputs(seed, K, N, T)
        q, scale, zero, c, mask, W_hat, stats = mod.cobalt_quantize(W, H, sp, beta, bits, group, mask_block=mb)
        p = f"c{seed}_"
        out[p + "W"] = W.numpy(); out[p + "X"] = X.numpy()
        out[p + "cfg"] = np.array([sp, beta, bits, group, mb], np.float64)
        out[p + "q"] = q.numpy().astype(np.uint8); out[p + "scale"] = scale.numpy().astype(np.float32)
        out[p + "zero"] = zero.numpy().astype(np.float32); out[p + "col_scale"] = c.numpy().astype(np.float32)
        out[p + "mask"] = np.packbits(mask.numpy() != 0, axis=-1, bitorder="little")
        out[p + "relerr"] = np.float64(stats["relerr"]); out[p + "damping"] = np.float64(stats["damping"])
        print(p, {k: stats[k] for k in ("sparsity_achieved", "relerr", "eout_ratio", "damping", "inv_method", "zero_oor")},
              "q dtype", q.dtype, "scale dtype", scale.dtype, "zero dtype", zero.dtype)
    path = os.path.join(HERE, "cobalt_quantize.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
