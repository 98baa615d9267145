"""Headline benchmark: decode GEMV over a Mistral-7B-shaped layer set in CBK1 form.

One "step" is one pass of the hot path over one layer set: the seven M=1 GEMVs of a decoder
layer (q, k, v, o, gate, up, down) at sparsity 0.5, 4-bit codes, group 128 (layout BLK1632_4,
3.1875 bits per weight).  The packed weights of several distinct layer sets are resident in
HBM before the timed region; successive steps rotate through them so that the streamed set
exceeds twice the 256 MB Infinity Cache.  `value` is packed bytes streamed per second.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mistral7b|gemma27b] [--m M]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SHAPES = {
    "mistral7b": [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
                  ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)],
    "gemma27b": [("q", 4096, 5376), ("k", 2048, 5376), ("v", 2048, 5376), ("o", 5376, 4096),
                 ("gate", 21504, 5376), ("up", 21504, 5376), ("down", 5376, 21504)],
}
HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(pm, M, e_x=2, e_y=2):
    """Packed rows + scale + zero + col_scale + activations in + outputs out, per GEMV."""
    return pm.stream_bytes() + pm.cs_rows * pm.N * 2 + M * pm.N * e_x + M * pm.K * e_y


def cpu_baseline(shape, layout, bits, group, keep, M, seed=0, budget_s=20.0):
    """The oracle's dequantise-then-matmul forward on the host cores, on ONE matrix of the layer set."""
    import numpy as np
    from oracle import cbk_ref as R
    name, K, N = shape
    raw = R.synth_raw_matrix(K, N, 1.0 - keep / 32.0, bits, seed=seed, block=32, group=group)
    kw = {} if layout == R.BLK1632_4 else dict(bits=bits, group=group, keep_per_block=keep)
    pk = R.pack_matrix(raw["mask"], raw["q"], raw["scale"], raw["zero"], layout, **kw)
    x = np.random.default_rng(1).standard_normal((M, N)).astype(np.float16).astype(np.float32)
    times = []
    t_end = time.time() + budget_s
    while len(times) < 5 and (time.time() < t_end or len(times) < 2):
        t0 = time.perf_counter()
        W = R.dequant(pk, K, N, layout, col_scale=raw["col_scale"], **kw)
        y = x @ W.T
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    nbytes = R.stream_bytes(pk) + N * 2 + M * N * 2 + M * K * 2
    return dict(value=nbytes / t / 1e9, unit="GB/s", cores=os.cpu_count(), kind="port",
                sample=f"{name}_proj {K}x{N} only (1 of 7 matrices), numpy dequant+matmul per call, "
                       f"median of {len(times)} runs, {t * 1e3:.0f} ms per call")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="mistral7b", choices=list(SHAPES))
    ap.add_argument("--m", type=int, default=1)
    ap.add_argument("--dtype", default="f16", choices=["f16", "bf16"])
    ap.add_argument("--bits", type=int, default=4)
    ap.add_argument("--keep", type=int, default=16)
    ap.add_argument("--group", type=int, default=128)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--launch", default="phase", choices=["matrix", "phase", "layer"],
                    help="GEMVs per launch: one matrix, one dependency phase (qkv | o | gate,up | down), or the layer set")
    ap.add_argument("--no-graph", action="store_true", help="launch from the host instead of replaying HIP graphs")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    from cobalt_amd import format as F, ops
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    layout = F.BLK1632_4 if (a.bits, a.keep, a.group) == (4, 16, 128) else F.BLKC
    dt = torch.float16 if a.dtype == "f16" else torch.bfloat16
    shapes = SHAPES[a.workload]
    M = a.m

    set_bytes = sum(K * F.row_stride(layout, N, a.bits, a.group, a.keep) + K * (N // a.group) * 3 for _, K, N in shapes)
    n_copies = max(2, -(-2 * 256 * 2**20 // set_bytes))
    sets = []
    for c in range(n_copies):
        sets.append([F.synth_packed(K, N, layout, a.bits, a.group, a.keep, seed=1000 * c + i, device=dev).to_tiled()
                     for i, (_, K, N) in enumerate(shapes)])
    xs = {N: torch.randn(M, N, device=dev, generator=torch.Generator(device=dev).manual_seed(N)).to(dt)
          for _, _, N in shapes}
    ys = [torch.empty(M, K, dtype=dt, device=dev) for _, K, _ in shapes]
    step_bytes = sum(algorithmic_bytes(pm, M) for pm in sets[0])

    import ctypes
    from cobalt_amd import _lib
    L = _lib.lib()
    stream = torch.cuda.Stream(dev)
    sp = stream.cuda_stream
    xdt = F.dtype_code(dt)
    groups = {"matrix": [[i] for i in range(len(shapes))],
              "phase": [[0, 1, 2], [3], [4, 5], [6]],          # qkv | o | gate,up | down
              "layer": [list(range(len(shapes)))]}[a.launch]
    P = ctypes.c_void_p
    calls = []                                                  # per layer set: list of batched calls
    keep_alive = []
    for s in sets:
        cs = []
        for g in groups:
            n = len(g)
            descs = (F.CbkDesc * n)(*[s[i].desc() for i in g])
            xp = (P * n)(*[xs[shapes[i][2]].data_ptr() for i in g])
            yp = (P * n)(*[ys[i].data_ptr() for i in g])
            ldx = (ctypes.c_int64 * n)(*[shapes[i][2] for i in g])
            ldy = (ctypes.c_int64 * n)(*[shapes[i][1] for i in g])
            need = L.cbk_gemv_batch_workspace_bytes(n, descs, M)
            w = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
            keep_alive.append((descs, xp, yp, ldx, ldy, w))
            cs.append((n, descs, xp, ldx, yp, ldy, w.data_ptr(), w.numel()))
        calls.append(cs)

    def step(i):
        for n, descs, xp, ldx, yp, ldy, wp, wn in calls[i % n_copies]:
            rc = L.cbk_gemv_batch(n, descs, xp, ldx, xdt, M, yp, ldy, xdt, None, wp, wn, sp)
            if rc:
                raise RuntimeError(L.cbk_strerror(rc).decode())

    launches = len(groups)
    with torch.cuda.stream(stream):
        for i in range(n_copies):
            step(i)
        stream.synchronize()
        graphs = None
        if not a.no_graph:                                      # one HIP graph per distinct layer set
            graphs = []
            for i in range(n_copies):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    step(i)
                graphs.append(g)
        run = (lambda i: graphs[i % n_copies].replay()) if graphs else step
        for i in range(a.warmup):
            run(i)
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(a.steps):
            run(a.warmup + i)
        e1.record(stream)
        stream.synchronize()
    ms = e0.elapsed_time(e1)
    ms_per_step = ms / a.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    us_per_launch = ms_per_step * 1e3 / launches
    bytes_per_launch = step_bytes / launches
    achieved = bytes_per_launch / (us_per_launch * 1e-6) / 1e9
    bpw = sets[0][0].bpw()
    out = {
        "metric": "decode GEMV HBM GB/s at M=1 (packed CBK1 bytes streamed per second)" if M == 1
                  else f"decode GEMV HBM GB/s at M={M}",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8xi8->i32 mfma, f32 scale" if False else ("f16" if a.dtype == "f16" else "bf16"),
        "data": "synthetic",
        "config": {"workload": f"{a.workload} decode layer set, 7 GEMVs, M={M}, sparsity {1 - a.keep / 32:.4g}, "
                               f"{a.bits}-bit, group {a.group}, layout {F.LAYOUT_NAME[layout]}, {bpw:.4f} bpw",
                   "layer_set_bytes": step_bytes, "distinct_layer_sets": n_copies,
                   "launches_per_step": launches, "launch_grouping": a.launch,
                   "hip_graph": not a.no_graph},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "decode GEMV", "avg_launch_us": round(us_per_launch, 3),
                     "bytes_per_launch": int(bytes_per_launch)},
    }
    if not a.no_cpu:
        from oracle import cbk_ref as R
        out["cpu_baseline"] = cpu_baseline(shapes[0], layout if layout == F.BLK1632_4 else R.BLKC, a.bits, a.group,
                                           a.keep, M)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
