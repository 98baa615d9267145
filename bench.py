"""Headline benchmark of the CBK1 sparse low-bit linear layer on one MI355X.

Decode (the `value` of the JSON line).  One "step" is one pass of the hot path over one
decoder-layer set: the seven M-row GEMVs of a layer (q, k, v, o, gate, up, down) at sparsity
0.5, 4-bit codes, group 128 (layout BLK1632_4, 3.1875 bits per weight), launched as the four
dependency phases of a decoder layer (q,k,v | o | gate,up | down), one batched kernel launch
per phase, replayed from HIP graphs: one graph holds about 32 steps in a row, as a decoder
replays all its layers for a token in one graph (a replay boundary costs several microseconds
on the GPU; single-step graphs serve the remainder, so that exactly K steps are timed).  The
packed weights of several distinct layer sets are resident in HBM before the timed region;
successive steps rotate through them so that the streamed set exceeds twice the 256 MB
Infinity Cache.  `value` is algorithmic bytes (packed
rows + scales + zeros + col_scale + activations in + outputs out) streamed per second.

`roofline` describes the decode kernel: algorithmic bytes per launch over the average launch
duration, which is the timed region (HIP events recorded on the launch stream) divided by
the number of launches in it; the gaps between launches are therefore counted as kernel time.

`prefill_gemm` reports the prefill kernel at the Gemma-3-27B MLP shapes (M=2048, bf16 by
default; --prefill-workload / --prefill-m / --prefill-dtype choose others) in TFLOP/s against
the 2.5 PFLOP/s dense bf16/f16 MFMA peak.

`gemm_m64` is the same kernel's 64-token tile at 64 activation rows (batched decoding) on the
decode workload's MLP shapes; `measured_ceilings` are this GPU's dense f16 MFMA rate and plain
read rate from two probe kernels.

`lm_head_gemv` is the decode kernel on one large matrix, the model's output projection
(vocabulary x hidden, dense 4-bit): what the kernel streams when a launch is long enough for
its fixed costs not to matter.

`cpu_baseline` is the C oracle (dequantise-then-matmul, OpenMP over rows) timed on the host
cores on the SAME packed bytes as the first layer set, and doubles as a last parity check of
the GPU outputs.

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
MFMA_PEAK_TFLOPS = 2500.0          # dense bf16 / f16 MFMA peak of MI355X

# HBM bytes per launch of the decode kernel (FETCH_SIZE + WRITE_SIZE of rocprofv3 --pmc, scaled by
# the same counters read for a device-to-device copy of known size), keyed by
# (workload, launch grouping, M); filled from the runs summarised under profiles/.
MEASURED_TRAFFIC = {("mistral7b", "phase", 1): 22311131}


def algorithmic_bytes(pm, M, e_x=2, e_y=2):
    """Packed rows + scale + zero + col_scale + activations in + outputs out, per GEMV."""
    return pm.stream_bytes() + pm.cs_rows * pm.N * 2 + M * pm.N * e_x + M * pm.K * e_y


def cpu_baseline(pms, shapes, xs, ys, M, budget_s=20.0):
    """C oracle forward over the layer set on the host cores, on the bytes the GPU used."""
    import numpy as np
    from oracle import cbk_ref_c as C
    nthreads = min(16, os.cpu_count() or 1)
    C.set_threads(nthreads)
    total_bytes, total_t, worst, done, calls = 0, 0.0, 0.0, [], []
    t_stop = time.time() + budget_s
    for pm, (name, K, N) in zip(pms, shapes):
        if done and time.time() > t_stop:
            break
        pk = dict(data=pm.array("data").cpu().numpy(), scale=pm.array("scale").cpu().numpy().reshape(K, -1),
                  zero=pm.array("zero").cpu().numpy().reshape(K, -1))
        cs = pm.array("col_scale").cpu().numpy().reshape(pm.cs_rows, N) if pm.cs_rows else None
        x = xs[N].float().cpu().numpy()
        call = lambda pk=pk, K=K, N=N, pm=pm, x=x, cs=cs: C.forward(
            pk, K, N, pm.layout, x, col_scale=cs, bits=pm.bits, group=pm.group, keep_per_block=pm.keep or None)
        t0 = time.perf_counter()
        y = call()
        total_t += time.perf_counter() - t0
        total_bytes += algorithmic_bytes(pm, M)
        got = ys[name].float().cpu().numpy()
        worst = max(worst, float(np.linalg.norm(got - y) / np.linalg.norm(y)))
        done.append(name)
        calls.append((call, algorithmic_bytes(pm, M)))
    # further passes over the same matrices until about one second of wall time on all threads
    # (10-30 s of CPU work); the first, checked pass counts too
    passes = 1
    more = max(0, min(40, int(1.0 / max(total_t, 1e-3))))
    for _ in range(more):
        if time.time() > t_stop:
            break
        for call, nbytes in calls:
            t0 = time.perf_counter()
            call()
            total_t += time.perf_counter() - t0
            total_bytes += nbytes
        passes += 1
    return dict(value=round(total_bytes / total_t / 1e9, 3), unit="GB/s", cores=nthreads, kind="port",
                sample=f"C oracle dequantise-then-matmul (OpenMP, {nthreads} threads) over {'+'.join(done)} of the first "
                       f"layer set, {passes} passes, {total_t:.2f} s wall = {total_t * nthreads:.0f} core-seconds; "
                       f"same packed bytes as the GPU run",
                gpu_vs_oracle_rel_fro=worst)


def measured_ceilings(torch, dev):
    """What this GPU reaches on back-to-back dense f16 MFMAs and on a plain streaming read of
    1 GiB (libcbk_bench.so, built by `python -m cobalt_amd.build`): ceilings to read the kernels'
    figures against, beside the published peaks.  None if the helper library is not built."""
    import ctypes
    path = os.path.join(ROOT, "cobalt_amd", "libcbk_bench.so")
    if not os.path.exists(path):
        return None
    L = ctypes.CDLL(path)
    L.cbk_bench_mfma_f16.restype = ctypes.c_int
    L.cbk_bench_mfma_f16.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    L.cbk_bench_read.restype = ctypes.c_int
    L.cbk_bench_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    st = torch.cuda.current_stream(dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(fn, reps):
        for _ in range(3):
            fn()
        e0.record(st)
        for _ in range(reps):
            fn()
        e1.record(st)
        st.synchronize()
        return e0.elapsed_time(e1) / reps

    blocks, iters = 2 * cus, 4000
    sink = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
    ms = timed(lambda: L.cbk_bench_mfma_f16(blocks, iters, sink.data_ptr(), st.cuda_stream), 5)
    mfma = blocks * 4 * iters * 16 * 2.0 * 32 * 32 * 16 / ms / 1e9
    buf = torch.empty(2**30, dtype=torch.uint8, device=dev)
    buf.random_(0, 256)
    sink4 = torch.zeros(1, dtype=torch.int32, device=dev)
    read = 0.0
    for per_cu in (8, 16, 32):                                    # the best of three grid sizes
        ms = timed(lambda: L.cbk_bench_read(buf.data_ptr(), buf.numel(), per_cu * cus, sink4.data_ptr(), st.cuda_stream), 10)
        read = max(read, buf.numel() / ms / 1e6)
    del buf, sink, sink4
    return {"mfma_f16_dense_tflops": round(mfma, 1), "hbm_read_gbs": round(read, 1),
            "how": "libcbk_bench.so: 16 independent v_mfma_f32_32x32x16_f16 per wavefront, one wavefront per SIMD; "
                   "grid-stride 16-byte reads of 1 GiB, eight in flight per lane, best of three grid sizes"}


VOCAB = {"mistral7b": 32000, "gemma27b": 262144}


def lm_head_gemv(torch, F, ops, dev, workload, M, dt, reps=20):
    """Decode kernel on the output projection of the model the workload is shaped after: dense
    4-bit codes (DENSE4, the reference packer's default for the tied embedding,
    src/cobaltkernel/pack_cobalt.py:561-563), vocabulary x hidden, one launch."""
    N = SHAPES[workload][0][2]
    K = VOCAB[workload]
    pm = F.synth_packed(K, N, F.DENSE4, seed=3, device=dev).to_tiled()
    # successive calls rotate over as many copies of the matrix as exceed twice the 256 MB Infinity Cache
    copies = [pm]
    while len(copies) * pm.stream_bytes() < 2 * 256 * 2**20:
        copies.append(F.synth_packed(K, N, F.DENSE4, seed=3 + len(copies), device=dev).to_tiled())
    x = torch.randn(M, N, device=dev, generator=torch.Generator(device=dev).manual_seed(1)).to(dt)
    for i in range(2 * len(copies)):
        y = ops.gemv(copies[i % len(copies)], x)
    st = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = -(-reps // len(copies)) * len(copies)
    e0.record(st)
    for i in range(reps):
        y = ops.gemv(copies[i % len(copies)], x)
    e1.record(st)
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    nbytes = algorithmic_bytes(pm, M)
    out = {"matrix": f"{K}x{N} DENSE4 ({pm.bpw():.4f} bpw), M={M}", "distinct_copies": len(copies), "ms": round(ms, 4), "bytes": nbytes,
           "gbs": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    del pm, copies, x, y
    return out


def prefill_gemm(torch, F, ops, dev, workload, layout, bits, group, keep, M, dt, reps=20, warm=10):
    """Prefill kernel on the MLP matrices (gate, up, down) of a layer set."""
    shapes = {n: (K, N) for n, K, N in SHAPES[workload]}
    rows = []
    tot_flop, tot_ms = 0.0, 0.0
    for name in ("gate", "down"):
        K, N = shapes[name]
        pm = F.synth_packed(K, N, layout, bits, group, keep, seed=7, device=dev).to_tiled()
        x = torch.randn(M, N, device=dev, generator=torch.Generator(device=dev).manual_seed(N)).to(dt)
        ws = ops.workspace_for(pm, M)                             # the caller's scratch, allocated once
        for _ in range(warm):                                     # the first launches run at a lower clock
            y = ops.gemm(pm, x, workspace=ws)
        torch.cuda.synchronize()
        st = torch.cuda.current_stream()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(st)
        for _ in range(reps):
            y = ops.gemm(pm, x, workspace=ws)
        e1.record(st)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        flop = 2.0 * M * K * N
        tot_flop += flop * (2 if name == "gate" else 1)         # gate and up have the same shape
        tot_ms += ms * (2 if name == "gate" else 1)
        rows.append({"matrix": f"{name} {K}x{N}", "ms": round(ms, 4), "tflops": round(flop / ms / 1e9, 1)})
        bpw = pm.bpw()
        del pm, x, y, ws
    ach = tot_flop / tot_ms / 1e9
    return {"workload": f"{workload} MLP (gate, up, down), M={M}, {str(dt)[6:]} activations, {F.LAYOUT_NAME[layout]} "
                        f"{bits}-bit keep {keep}/32 group {group}, {bpw:.4f} bpw; time includes the activation "
                        "pre-scaling kernel (and the reduction kernel of a split column range)",
            "tflops": round(ach, 1), "per_matrix": rows,
            "roofline": {"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(ach / MFMA_PEAK_TFLOPS, 4), "traffic": None,
                         "kernel": "cbk::gemm_big_kernel"}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--workload", default="mistral7b", choices=list(SHAPES))
    ap.add_argument("--m", type=int, default=1)
    ap.add_argument("--dtype", default="f16", choices=["f16", "bf16"])
    ap.add_argument("--bits", type=int, default=4)
    ap.add_argument("--keep", type=int, default=16)
    ap.add_argument("--group", type=int, default=128)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-core baseline")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill GEMM measurement")
    ap.add_argument("--no-lm-head", action="store_true", help="skip the output-projection GEMV measurement")
    ap.add_argument("--prefill-workload", default="gemma27b", choices=list(SHAPES))
    ap.add_argument("--prefill-m", type=int, default=2048)
    ap.add_argument("--prefill-dtype", default="bf16", choices=["f16", "bf16"])
    ap.add_argument("--launch", default="phase", choices=["matrix", "phase", "layer"],
                    help="GEMVs per launch: one matrix, one dependency phase (qkv | o | gate,up | down), or the layer set")
    ap.add_argument("--no-graph", action="store_true", help="launch from the host instead of replaying HIP graphs")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 1 GiB device-to-device copy (reference reading for the HBM traffic counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    from cobalt_amd import format as F, ops
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    layout = F.BLK1632_4 if (a.bits, a.keep, a.group) == (4, 16, 128) else \
        F.BLK1632_6 if (a.bits, a.keep, a.group) == (6, 16, 128) else F.BLKC
    dt = torch.float16 if a.dtype == "f16" else torch.bfloat16
    shapes = SHAPES[a.workload]
    M = a.m

    set_bytes = sum(K * F.row_stride(layout, N, a.bits, a.group, a.keep) + K * (N // a.group) * 3 for _, K, N in shapes)
    n_copies = max(2, -(-2 * 256 * 2**20 // set_bytes))
    sets, first_rowmajor = [], None
    for c in range(n_copies):
        rm = [F.synth_packed(K, N, layout, a.bits, a.group, a.keep, seed=1000 * c + i, device=dev)
              for i, (_, K, N) in enumerate(shapes)]
        if c == 0 and not a.no_cpu:
            first_rowmajor = [p.to("cpu") for p in rm]
        sets.append([p.to_tiled() for p in rm])
        del rm
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

    def launch(c):
        n, descs, xp, ldx, yp, ldy, wp, wn = c
        rc = L.cbk_gemv_batch(n, descs, xp, ldx, xdt, M, yp, ldy, xdt, None, wp, wn, sp)
        if rc:
            raise RuntimeError(L.cbk_strerror(rc).decode())

    def step(i):
        for c in calls[i % n_copies]:
            launch(c)

    launches = len(groups)
    torch.cuda.synchronize()                                    # the weights were made on the default stream
    with torch.cuda.stream(stream):
        step(0)
        stream.synchronize()
        y_first = {name: y.clone() for (name, _, _), y in zip(shapes, ys)}   # outputs of layer set 0, for the parity check
        for i in range(1, n_copies):
            step(i)
        stream.synchronize()
        graphs = None
        per_graph = 0
        if not a.no_graph:                                      # one HIP graph per distinct layer set
            graphs = []
            for i in range(n_copies):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    step(i)
                graphs.append(g)
            # and one graph of about 32 layer sets in a row (whole rotations of the distinct sets),
            # as a decoder replays all its layers per token
            per_graph = -(-32 // n_copies) * n_copies
            g_all = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g_all, stream=stream):
                for i in range(per_graph):
                    step(i)
        run = (lambda i: graphs[i % n_copies].replay()) if graphs else step

        def run_steps(first, count):                             # exactly `count` steps, layer sets in rotation
            i = first
            while count > 0:
                if graphs and i % n_copies == 0 and count >= per_graph:
                    g_all.replay()
                    i += per_graph
                    count -= per_graph
                else:
                    run(i)
                    i += 1
                    count -= 1
            return i

        nxt = run_steps(0, a.warmup)
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        run_steps(nxt, a.steps)
        e1.record(stream)
        stream.synchronize()
        ms_per_step = e0.elapsed_time(e1) / a.steps

        if a.copy_calibration:
            src = torch.empty(2**30, dtype=torch.uint8, device=dev)
            dst = torch.empty_like(src)
            for _ in range(3):
                dst.copy_(src)
            stream.synchronize()
            del src, dst

    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    # average launch of the decode kernel over the timed region (HIP events on the launch stream);
    # it contains the gap between consecutive launches, so it is an upper bound of the kernel time
    us_per_launch = ms_per_step * 1e3 / launches
    bytes_per_launch = step_bytes / launches
    achieved = bytes_per_launch / (us_per_launch * 1e-6) / 1e9
    bpw = sets[0][0].bpw()
    out = {
        "metric": "decode GEMV HBM GB/s (% of 8 TB/s) at M=1; prefill GEMM TFLOP/s at M=2048",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8 (int8 MFMA on integer codes and 3-digit block-fixed-point activations, f32 scales)",
        "data": "synthetic",
        "config": {"workload": f"{a.workload} decode layer set, 7 GEMVs, M={M}, {a.dtype} activations, sparsity "
                               f"{1 - a.keep / 32:.4g}, {a.bits}-bit, group {a.group}, layout {F.LAYOUT_NAME[layout]}, "
                               f"{bpw:.4f} bpw",
                   "layer_set_bytes": step_bytes, "distinct_layer_sets": n_copies,
                   "launches_per_step": launches, "launch_grouping": a.launch,
                   "hip_graph": not a.no_graph,
                   "steps_per_graph_replay": (per_graph if not a.no_graph else 0), "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC.get((a.workload, a.launch, M)),
                     "kernel": "cbk::gemv_mfma_kernel", "avg_launch_us": round(us_per_launch, 3),
                     "launches_timed": a.steps * launches, "bytes_per_launch": int(bytes_per_launch)},
    }
    g_all = None
    del graphs, sets, calls, keep_alive
    torch.cuda.empty_cache()
    if not a.no_prefill:
        out["prefill_gemm"] = prefill_gemm(torch, F, ops, dev, a.prefill_workload, layout, a.bits, a.group, a.keep,
                                           a.prefill_m, torch.float16 if a.prefill_dtype == "f16" else torch.bfloat16)
        # the same kernel's 64-token tile at a batched-decoding row count, on the decode workload's shapes
        mid = prefill_gemm(torch, F, ops, dev, a.workload, layout, a.bits, a.group, a.keep, 64,
                           torch.float16 if a.dtype == "f16" else torch.bfloat16)
        out["gemm_m64"] = {"workload": mid["workload"], "tflops": mid["tflops"], "per_matrix": mid["per_matrix"]}
    if not a.no_lm_head:
        out["lm_head_gemv"] = lm_head_gemv(torch, F, ops, dev, a.workload, M, dt)
    ceil = measured_ceilings(torch, dev)
    if ceil:
        out["measured_ceilings"] = ceil
        out["roofline"]["frac_of_measured_read"] = round(achieved / ceil["hbm_read_gbs"], 4)
        if "prefill_gemm" in out:
            out["prefill_gemm"]["roofline"]["frac_of_measured_mfma"] = round(
                out["prefill_gemm"]["tflops"] / ceil["mfma_f16_dense_tflops"], 4)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(first_rowmajor, shapes, xs, y_first, M)
        # outputs are rounded to the activation dtype (2^-11 relative) on top of the kernel's own error
        assert out["cpu_baseline"]["gpu_vs_oracle_rel_fro"] < 1e-3, "GPU outputs disagree with the oracle"
    print(json.dumps(out))


if __name__ == "__main__":
    main()
