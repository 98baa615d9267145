"""TEST INFRASTRUCTURE, not product code: torch restatement of the reference's CPU forward of a
packed layer, the path `SparseQuantLinear.forward` takes in its low-memory mode
(benchmarks/benchmark_suite.py:1200-1209): dequantise the whole matrix to float32, then matmul.

Only tests and the `cpu_baseline` leg of bench.py import this module; nothing under cobalt_amd/
does.  It follows the torch oracle of the reference (src/cobaltkernel/dequant_ref.py:36-103:
unpack the planes with integer tensor ops, scatter the survivors into their columns in column
order, `((q - zero) * scale) * keep * col_scale` in float32) and is generalised to the code
widths and survivor counts of the extension layouts (one LSB-first bit stream per row).
It is pinned against the numpy oracle (oracle/cbk_ref.py) in tests/test_oracle_torch.py.
"""
import torch

BLOCK = 32
DENSE4, DENSE8, BLK1632_4, BLK1632_6, BLKC, DENSEB = 1, 2, 6, 7, 8, 9      # layout ids of docs/FORMAT.md:65-71 + extensions


def _unpack_bits_lsb(by: torch.Tensor) -> torch.Tensor:
    """uint8 [K, B] -> uint8 [K, 8 B], bit i of byte j at position 8 j + i."""
    sh = torch.arange(8, dtype=torch.uint8, device=by.device)
    return ((by.unsqueeze(-1) >> sh) & 1).reshape(by.shape[0], -1)


def _codes_from_stream(by: torch.Tensor, n: int, bits: int) -> torch.Tensor:
    """First n codes of `bits` bits of an LSB-first bit stream, uint8 [K, *] -> float32 [K, n]."""
    K = by.shape[0]
    if bits == 8:
        return by[:, :n].to(torch.float32)
    if bits == 4:                                        # dequant_ref.py:43-47, :58-59: low nibble first
        b = by[:, : (n + 1) // 2]
        return torch.stack([b & 0xF, b >> 4], dim=2).reshape(K, -1)[:, :n].to(torch.float32)
    nbytes = (n * bits + 7) // 8
    bit = _unpack_bits_lsb(by[:, :nbytes])[:, : n * bits].reshape(K, n, bits).to(torch.int32)
    w = (1 << torch.arange(bits, dtype=torch.int32, device=by.device))
    return (bit * w).sum(-1).to(torch.float32)


def dequant(rows: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, col_scale, K: int, N: int, layout: int,
            bits: int = 4, group: int = 128, keep: int = 16) -> torch.Tensor:
    """rows uint8 [K, stride] (row-major packed rows), scale float16 [K, G], zero uint8 [K, G],
    col_scale float16 [cs_rows, N] or None -> W_hat float32 [K, N]."""
    G = N // group
    if layout in (DENSE4, DENSE8, DENSEB):
        b = 4 if layout == DENSE4 else 8 if layout == DENSE8 else bits
        q = _codes_from_stream(rows, N, b)
        kept = None
    else:
        if layout == BLK1632_4:
            bits, keep = 4, 16
        if layout == BLK1632_6:
            raise NotImplementedError("the 6-bit plane layout is not part of the timed baseline")
        NB = N // BLOCK
        kept = _unpack_bits_lsb(rows[:, : N // 8]).bool()                     # dequant_ref.py:56-57
        codes = _codes_from_stream(rows[:, N // 8:], NB * keep, bits)
        q = torch.zeros(K, N, dtype=torch.float32)
        q[kept] = codes.reshape(-1)                                            # survivors in column order, :68
    s = scale.reshape(K, G).to(torch.float32)
    z = zero.reshape(K, G).to(torch.float32)
    w = ((q.view(K, G, group) - z[:, :, None]) * s[:, :, None]).reshape(K, N)  # :69-72, :87-90
    if kept is not None:
        w = w * kept.to(torch.float32)                                         # pruned positions exactly 0, :73
    if col_scale is not None:
        cs = col_scale.to(torch.float32).reshape(-1, N)
        if cs.shape[0] == 2:                                                   # fused gate/up, :76-79
            w[0::2] *= cs[0][None, :]
            w[1::2] *= cs[1][None, :]
        else:
            w = w * cs[0][None, :]
    return w


def forward(w_hat: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """y = x.float() @ W_hat.T (benchmarks/benchmark_suite.py:1205-1209 with float32 weights)."""
    return x.to(torch.float32) @ w_hat.t()
