"""Headline benchmark of the CBK1 sparse low-bit linear layer on one MI355X.

Decode (the `value` of the JSON line).  One "step" is one pass of the hot path over one
decoder-layer set: the seven M-row GEMVs of a layer (q, k, v, o, gate, up, down), launched as the
four dependency phases of a decoder layer (q,k,v | o | gate,up | down), one batched kernel launch
per phase.  The headline workload is the Gemma-3-27B-shaped layer set at sparsity 0.5, 4-bit
codes, group 128 (layout BLK1632_4, 3.1875 bits per weight), bf16 activations, M=1; the
Mistral-7B-shaped set (f16) is reported beside it as `decode_mistral7b`.  The packed weights of
several distinct layer sets are resident in HBM before the timed region and successive steps
rotate through them, so that the streamed set exceeds twice the 256 MB Infinity Cache.

Launches are replayed from HIP graphs of many steps in a row, as a decoder replays all its layers
for a token in one graph (a replay boundary costs the GPU several microseconds).  `--steps K` is
honoured exactly and inside such graphs: K // P replays of a graph of P steps (whole rotations over
the distinct layer sets, about 32 steps) plus one replay of a graph holding the K % P steps that
remain.  Warm-up is `--warmup` steps, and never less than 50 ms of replays (the first launches
of a process run at a lower clock), both graphs included; the start event of the timed region is
enqueued behind one more untimed replay, so that the host's graph-launch latency stays outside
the region (exactly K steps between the two events).  The JSON says what was replayed.

`value` is algorithmic bytes (packed rows + scales + zeros + col_scale + activations in + outputs
out) streamed per second.  `roofline` describes the decode kernel: algorithmic bytes per launch
over the average launch duration, which is the timed region (HIP events recorded on the launch
stream) divided by the number of launches in it; the gaps between launches are therefore counted
as kernel time.  `per_matrix` times each distinct matrix of the set on its own (one launch per
matrix, distinct copies of at least 512 MB in rotation): the kernel's rate without the other
phases of the step.

`prefill_gemm` reports the prefill kernel at the Gemma-3-27B MLP shapes (M=2048, bf16 by default)
in TFLOP/s against the 2.5 PFLOP/s dense bf16/f16 MFMA peak, and checks sampled output rows of
the timed configuration against a float64 matmul with the bit-exact dequantised weights.

The other benchmark configurations ride in the same JSON line unless `--no-configs` is given:
`config0_single_layer` (one Mistral-7B MLP up-projection, M=1 and a 256-token prefill, checked
against the C oracle), `config1_mistral7b_m4/_m8` and `config3_gemma27b_m4/_m8` (the decode step
at four and eight activation rows), `config2_mistral7b_b3_keep10` (3-bit codes, 10 survivors per
32 columns, group 64: decode step and MLP prefill) and `config4_grid`, the nine-cell sweep
(Gemma-3-27B shapes x 62 layers, sparsity 0.3/0.5/0.7 as 23/16/10 survivors per 32 columns,
2/3/4-bit codes, group 64): per-token linear time of a decode step (M=1) and of a 4096-token
prefill, and bits per weight, per cell.  `--grid` runs that sweep alone, at more repetitions.

`cpu_baseline` is the torch restatement of the reference's CPU forward (dequantise the packed
bytes to float32, then matmul: oracle/torch_ref.py) on the host cores, on the same packed bytes
as the first layer set: the median of five passes over as many matrices of the set as fit the
time budget, and a 256-token prefill leg on the MLP shapes extrapolated linearly in M to the
2048 tokens the GPU leg runs; the C oracle checks the GPU outputs of that set.

`--only per-matrix|row-kernels` runs one leg with host launches or graphs (`--no-graph`) and
prints a progress line per matrix on stderr: the form a counter-collecting profiler run takes,
with the profiler's kernel filter set to this library's kernels.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gemma27b|mistral7b] [--m M]
                [--grid] [--no-configs] [--only LEG] [--no-graph] [--copy-calibration]
"""
import argparse
import ctypes
import json
import os
import platform
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
WORKLOAD_DTYPE = {"mistral7b": "f16", "gemma27b": "bf16"}          # the activation types the configurations name
VOCAB = {"mistral7b": 32000, "gemma27b": 262144}
GEMMA_LAYERS = 62
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0          # dense bf16 / f16 MFMA peak of MI355X
INFINITY_CACHE = 256 * 2**20
MIN_WARM_MS = 50.0

# HBM bytes per launch of the decode kernel (FETCH_SIZE + WRITE_SIZE of rocprofv3 --pmc, scaled by
# the same counters read for a device-to-device copy of known size), keyed by
# (workload, launch grouping, M).  Stored figures from the runs summarised under profiles/, not
# counters read during a bench run.
MEASURED_TRAFFIC = {("mistral7b", "phase", 1): 22366413, ("gemma27b", "phase", 1): 43134566}


def algorithmic_bytes(pm, M, e_x=2, e_y=2):
    """Packed rows + scale + zero + col_scale + activations in + outputs out, per GEMV."""
    return pm.stream_bytes() + pm.cs_rows * pm.N * 2 + M * pm.N * e_x + M * pm.K * e_y


def layout_of(F, bits, keep, group):
    return F.BLK1632_4 if (bits, keep, group) == (4, 16, 128) else \
        F.BLK1632_6 if (bits, keep, group) == (6, 16, 128) else F.BLKC


def torch_dtype(torch, name):
    return torch.float16 if name == "f16" else torch.bfloat16


# ------------------------------------------------------------------ decode: layer-set step
def make_sets(torch, F, dev, shapes, layout, bits, group, keep, min_bytes, keep_first_rowmajor=False):
    """Distinct layer sets (device order) whose packed bytes add up to at least `min_bytes`."""
    set_bytes = sum(K * F.row_stride(layout, N, bits, group, keep) + K * (N // group) * 3 for _, K, N in shapes)
    n_copies = max(2, -(-min_bytes // set_bytes))
    sets, first = [], None
    for c in range(n_copies):
        rm = [F.synth_packed(K, N, layout, bits, group, keep, seed=1000 * c + i, device=dev)
              for i, (_, K, N) in enumerate(shapes)]
        if c == 0 and keep_first_rowmajor:
            first = [p.to("cpu") for p in rm]
        sets.append([p.to_tiled() for p in rm])
        del rm
    return sets, first


class GraphTimer:
    """Replays `step(i)` (i = running step index) from HIP graphs and times exactly K steps."""

    def __init__(self, torch, stream, step, rotation, use_graph=True, target_steps=32):
        self.torch, self.stream, self.step, self.use_graph = torch, stream, step, use_graph
        self.per_graph = -(-target_steps // rotation) * rotation       # whole rotations over the distinct sets
        self.g_all = None
        self._rem = {}
        if use_graph:
            self.g_all = self._capture(self.per_graph)

    def _capture(self, n):
        g = self.torch.cuda.CUDAGraph()
        with self.torch.cuda.graph(g, stream=self.stream):
            for i in range(n):
                self.step(i)
        return g

    def _run(self, full, rem):
        if not self.use_graph:
            for i in range(full * self.per_graph + rem):
                self.step(i)
            return
        for _ in range(full):
            self.g_all.replay()
        if rem:
            self._rem[rem].replay()

    def measure(self, steps, warmup):
        torch, stream = self.torch, self.stream
        full, rem = divmod(steps, self.per_graph)
        if self.use_graph and rem and rem not in self._rem:
            self._rem[rem] = self._capture(rem)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        # first replay of every graph (uploads it), then an estimate of a replay's duration
        self._run(1, rem)
        stream.synchronize()
        e0.record(stream)
        self._run(1, 0)
        e1.record(stream)
        stream.synchronize()
        t_replay = max(e0.elapsed_time(e1), 1e-3)
        n_warm = max(-(-warmup // self.per_graph), int(MIN_WARM_MS / t_replay) + 1)
        self._run(n_warm, rem)
        stream.synchronize()
        # One more untimed replay goes out in front of the start event, with no synchronisation
        # behind it: while the GPU runs it the host enqueues the event and the timed replays, so
        # the host's graph-launch latency (tens of microseconds, several per cent of a 20-step
        # region) does not sit inside the timed region.  The region itself is exactly `steps` steps.
        lead = 1 if self.use_graph else 0
        self._run(lead, 0)
        e0.record(stream)
        self._run(full, rem)
        e1.record(stream)
        stream.synchronize()
        return {"ms_per_step": e0.elapsed_time(e1) / steps, "warmup_steps_run": (n_warm + 2 + lead) * self.per_graph + 2 * rem,
                "untimed_lead_replays": lead,
                "graph_replays_timed": (full + (1 if rem else 0)) if self.use_graph else 0,
                "steps_per_full_graph": self.per_graph if self.use_graph else 0,
                "steps_in_remainder_graph": rem if self.use_graph else 0}


def decode_layer_sets(torch, F, L, dev, shapes, sets, M, dt, launch, steps, warmup, use_graph=True):
    """Times `steps` layer-set steps over the distinct `sets` in rotation."""
    n_copies = len(sets)
    xs = {N: torch.randn(M, N, device=dev, generator=torch.Generator(device=dev).manual_seed(N)).to(dt)
          for _, _, N in shapes}
    ys = [torch.empty(M, K, dtype=dt, device=dev) for _, K, _ in shapes]
    step_bytes = sum(algorithmic_bytes(pm, M) for pm in sets[0])
    stream = torch.cuda.Stream(dev)
    sp = stream.cuda_stream
    xdt = F.dtype_code(dt)
    groups = {"matrix": [[i] for i in range(len(shapes))],
              "phase": [[0, 1, 2], [3], [4, 5], [6]],          # qkv | o | gate,up | down
              "layer": [list(range(len(shapes)))]}[launch]
    P = ctypes.c_void_p
    calls, keep_alive = [], []
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

    torch.cuda.synchronize()                                    # the weights were made on the default stream
    with torch.cuda.stream(stream):
        # outputs of layer set 0 in float32, for the parity check (untimed; the timed steps write x's type)
        y32 = [torch.empty(M, K, dtype=torch.float32, device=dev) for _, K, _ in shapes]
        for (n, descs, xp, ldx, _, ldy, wp, wn), g in zip(calls[0], groups):
            yp32 = (P * n)(*[y32[i].data_ptr() for i in g])
            rc = L.cbk_gemv_batch(n, descs, xp, ldx, xdt, M, yp32, ldy, F.F32, None, wp, wn, sp)
            if rc:
                raise RuntimeError(L.cbk_strerror(rc).decode())
        stream.synchronize()
        y_first = {name: y for (name, _, _), y in zip(shapes, y32)}
        for i in range(n_copies):
            step(i)
        stream.synchronize()
        timer = GraphTimer(torch, stream, step, n_copies, use_graph)
        res = timer.measure(steps, warmup)
    del timer, calls, keep_alive
    res.update(step_bytes=step_bytes, launches=len(groups), distinct_layer_sets=n_copies,
               gbs=step_bytes / (res["ms_per_step"] * 1e-3) / 1e9)
    return res, xs, y_first


def per_matrix(torch, F, L, dev, shapes, layout, bits, group, keep, M, dt, iters=24, tiled=True, use_graph=True):
    """Each distinct matrix of the layer set on its own: one launch per matrix, distinct copies of
    at least 512 MB in rotation (the protocol of src/cobaltkernel/test_gemv.py:201-202, :521-522),
    one HIP graph per rotation, or launches from the host with use_graph=False (counter runs:
    the profiler's counter collection is kept away from graph capture and replay).  tiled=False
    keeps the row-major order (the survivor-stream layouts have no other)."""
    rows, seen = [], set()
    stream = torch.cuda.Stream(dev)
    xdt = F.dtype_code(dt)
    P = ctypes.c_void_p
    for name, K, N in shapes:
        if (K, N) in seen:
            continue
        seen.add((K, N))
        order = (lambda p: p.to_tiled()) if tiled else (lambda p: p)
        pm0 = order(F.synth_packed(K, N, layout, bits, group, keep, seed=7000, device=dev))
        copies = max(2, -(-2 * INFINITY_CACHE // pm0.stream_bytes()))
        pms = [pm0] + [order(F.synth_packed(K, N, layout, bits, group, keep, seed=7000 + c, device=dev)) for c in range(1, copies)]
        x = torch.randn(M, N, device=dev, generator=torch.Generator(device=dev).manual_seed(N)).to(dt)
        y = torch.empty(M, K, dtype=dt, device=dev)
        args = []
        for pm in pms:
            d = (F.CbkDesc * 1)(pm.desc())
            args.append((d, (P * 1)(x.data_ptr()), (ctypes.c_int64 * 1)(N), (P * 1)(y.data_ptr()), (ctypes.c_int64 * 1)(K)))
        w = torch.empty(max(L.cbk_gemv_batch_workspace_bytes(1, args[0][0], M), 256), dtype=torch.uint8, device=dev)

        def rotation():
            for d, xp, ldx, yp, ldy in args:
                rc = L.cbk_gemv_batch(1, d, xp, ldx, xdt, M, yp, ldy, xdt, None, w.data_ptr(), w.numel(), stream.cuda_stream)
                if rc:
                    raise RuntimeError(L.cbk_strerror(rc).decode())

        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            rotation()
            stream.synchronize()
            g = None
            if use_graph:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    rotation()
            once = g.replay if use_graph else rotation
            for _ in range(3):
                once()
            stream.synchronize()
            reps = max(1, -(-iters // copies))
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            if use_graph:
                once()                                            # untimed, in front of the start event (see GraphTimer.measure)
            e0.record(stream)
            for _ in range(reps):
                once()
            e1.record(stream)
            stream.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * copies)
        nbytes = algorithmic_bytes(pms[0], M)
        rows.append({"matrix": f"{name} {K}x{N}", "bytes": nbytes, "distinct_copies": copies, "launches_timed": reps * copies,
                     "hip_graph": use_graph, "us": round(us, 2), "gbs": round(nbytes / us / 1e3, 1),
                     "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
        print(f"per_matrix {name} {K}x{N}: {us:.2f} us", file=sys.stderr, flush=True)
        del pms, args, g, x, y, w
        torch.cuda.empty_cache()
    return rows


def lm_head_gemv(torch, F, ops, dev, workload, M, dt, reps=20):
    """Decode kernel on the output projection of the model the workload is shaped after: dense
    4-bit codes (DENSE4, the reference packer's default for the tied embedding,
    src/cobaltkernel/pack_cobalt.py:561-563), vocabulary x hidden, one launch."""
    N = SHAPES[workload][0][2]
    K = VOCAB[workload]
    pm = F.synth_packed(K, N, F.DENSE4, seed=3, device=dev).to_tiled()
    copies = [pm]
    while len(copies) * pm.stream_bytes() < 2 * INFINITY_CACHE:
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


# ------------------------------------------------------------------ prefill
def prefill_parity(torch, ops, pm, x, nblocks=3, rows_per_block=64):
    """rel. Frobenius error of sampled output rows (blocks of weight rows at the start, middle and
    end of the matrix, every token) against a float64 matmul with the bit-exact dequantised
    weights, float32 output."""
    y = ops.gemm(pm, x, out_dtype=torch.float32)
    num = den = 0.0
    for b in range(nblocks):
        r0 = (pm.K - rows_per_block) * b // max(1, nblocks - 1)
        W = ops.dequant(pm, torch.float32, row0=r0, nrows=rows_per_block).double()
        ref = x.double() @ W.T
        num += float((y[:, r0:r0 + rows_per_block].double() - ref).pow(2).sum())
        den += float(ref.pow(2).sum())
        del W, ref
    del y
    return (num / den) ** 0.5


def prefill_gemm(torch, F, ops, dev, shapes, names, layout, bits, group, keep, M, dt, reps=20, warm=10, parity=True):
    """Prefill kernel on matrices `names` of a layer set (each distinct shape timed once, weighted
    by how often it occurs)."""
    by_name = {n: (K, N) for n, K, N in shapes}
    rows, timed = [], {}
    tot_flop = tot_ms = 0.0
    worst = 0.0
    bpw = None
    for name in names:
        K, N = by_name[name]
        if (K, N) not in timed:
            pm = F.synth_packed(K, N, layout, bits, group, keep, seed=7, device=dev).to_tiled()
            x = torch.randn(M, N, device=dev, generator=torch.Generator(device=dev).manual_seed(N)).to(dt)
            ws = ops.workspace_for(pm, M)                             # the caller's scratch, allocated once
            for _ in range(warm):                                     # the first launches run at a lower clock
                y = ops.gemm(pm, x, workspace=ws)
            torch.cuda.synchronize()
            st = torch.cuda.current_stream()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            y = ops.gemm(pm, x, workspace=ws)                         # untimed: the timed calls are enqueued while it runs
            e0.record(st)
            for _ in range(reps):
                y = ops.gemm(pm, x, workspace=ws)
            e1.record(st)
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / reps
            err = prefill_parity(torch, ops, pm, x) if parity else None
            dense_ms = library_dense_gemm_ms(torch, dev, M, K, N, dt, x) if parity else None
            if err is not None:
                worst = max(worst, err)
                assert err < 1e-3, f"prefill {name} {K}x{N} M={M}: rel. Frobenius error {err} against the dequantised weights"
            timed[(K, N)] = ms
            row = {"matrix": f"{name} {K}x{N}", "ms": round(ms, 4), "tflops": round(2.0 * M * K * N / ms / 1e9, 1)}
            if err is not None:
                row["rel_fro_vs_dequant_f64"] = float(f"{err:.3g}")
            if dense_ms is not None:
                row["library_dense_gemm_tflops"] = round(2.0 * M * K * N / dense_ms / 1e9, 1)
            rows.append(row)
            bpw = pm.bpw()
            del pm, x, y, ws
        tot_flop += 2.0 * M * K * N
        tot_ms += timed[(K, N)]
    ach = tot_flop / tot_ms / 1e9
    out = {"matrices": "+".join(names), "M": M, "dtype": str(dt)[6:], "layout": F.LAYOUT_NAME[layout], "bits": bits,
           "keep_per_32": keep, "group": group, "bpw": round(bpw, 4), "ms": round(tot_ms, 4), "tflops": round(ach, 1),
           "note": "time includes the activation pre-scaling kernel (and the reduction kernel of a split column range)",
           "per_matrix": rows,
           "roofline": {"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": round(ach / MFMA_PEAK_TFLOPS, 4), "traffic": None, "kernel": "cbk::gemm_big_kernel"}}
    if parity:
        out["parity"] = {"worst_rel_fro": float(f"{worst:.3g}"), "tolerance": 1e-3,
                         "how": "192 sampled weight rows x all tokens of every timed matrix, float32 output against "
                                "x.double() @ dequant(W).double().T"}
    return out


def library_dense_gemm_ms(torch, dev, M, K, N, dt, x, reps=10, warm=5):
    """The vendor library's dense GEMM (torch.matmul) on an unpacked matrix of the same shape and
    activation type: what the GPU does with 16-bit weights that need no decoding (five times the
    weight bytes).  A figure to read the packed kernel's against, not part of the path."""
    w = torch.randn(K, N, device=dev, generator=torch.Generator(device=dev).manual_seed(K)).mul_(0.02).to(dt)
    for _ in range(warm):
        y = x @ w.t()
    torch.cuda.synchronize()
    st = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    y = x @ w.t()                                                 # untimed, as for the packed kernel
    e0.record(st)
    for _ in range(reps):
        y = x @ w.t()
    e1.record(st)
    torch.cuda.synchronize()
    del w, y
    return e0.elapsed_time(e1) / reps



def decode_parity(torch, ops, pm, x, y):
    """rel. Frobenius error of decode outputs y [M, K] (float32) against x.double() @ W.double().T with W
    the library's bit-exact dequantisation of the same packed bytes (float64 on the GPU)."""
    W = ops.dequant(pm, torch.float32).double()
    ref = x.double() @ W.T
    err = float((y.double() - ref).norm() / ref.norm())
    del W, ref
    return err


def decode_rows_sweep(torch, F, L, dev, workload, layout, bits, group, keep, Ms, steps, warmup, use_graph=True,
                      launch="phase", parity=False, ops=None):
    """The decode step of one workload at several activation row counts on the same resident layer
    sets (built once)."""
    shapes = SHAPES[workload]
    dt = torch_dtype(torch, WORKLOAD_DTYPE[workload])
    sets, _ = make_sets(torch, F, dev, shapes, layout, bits, group, keep, 2 * INFINITY_CACHE)
    out = {}
    for M in Ms:
        res, xs, y_first = decode_layer_sets(torch, F, L, dev, shapes, sets, M, dt, launch, steps, warmup, use_graph)
        row = {"workload": f"{workload} decode layer set, 7 GEMVs, M={M}, {WORKLOAD_DTYPE[workload]} activations, "
                           f"{F.LAYOUT_NAME[layout]} {bits}-bit keep {keep}/32 group {group}, {sets[0][0].bpw():.4f} bpw",
               "M": M, "ms_per_step": round(res["ms_per_step"], 5), "gbs": round(res["gbs"], 1),
               "frac_of_hbm_peak": round(res["gbs"] / HBM_PEAK_GBS, 4), "layer_set_bytes": res["step_bytes"],
               "distinct_layer_sets": res["distinct_layer_sets"], "steps": steps, "hip_graph": use_graph}
        if parity:
            worst = max(decode_parity(torch, ops, pm, xs[N], y_first[name]) for pm, (name, _, N) in zip(sets[0], shapes))
            assert worst < 1e-3, f"{workload} M={M}: decode outputs off the dequantised weights by {worst}"
            row["parity"] = {"worst_rel_fro": float(f"{worst:.3g}"), "tolerance": 1e-3,
                             "how": "every matrix of the first layer set, float32 output against x.double() @ "
                                    "dequant(W).double().T (bit-exact dequantiser of the same bytes)"}
        out[M] = row
        del xs, y_first
    del sets
    torch.cuda.empty_cache()
    return out


def config0_single_layer(torch, F, ops, L, dev, cpu=True):
    """The reference's own CPU-runnable case: W 4096x4096 ~ N(0, 0.02) with 1 % of the columns
    scaled by 10, calibration activations 128x4096 ~ N(0, 1) for the Wanda score and the OBS
    update, column-balanced mask at sparsity 0.5, 4-bit RTN in groups of 128, packed as BLK1632_4;
    x is 1x4096 fp16.  Compressed and packed on the GPU by this package, decoded at M=1."""
    import numpy as np
    from cobalt_amd.linear import CobaltLinear
    g = torch.Generator().manual_seed(0)
    K = N = 4096
    W = torch.randn(K, N, generator=g) * 0.02
    W[:, torch.randperm(N, generator=g)[:41]] *= 10
    X = torch.randn(128, N, generator=g)
    x = torch.randn(1, N, generator=g).half()
    lin = torch.nn.Linear(N, K, bias=False)
    lin.weight.data.copy_(W)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    m = CobaltLinear.from_linear(lin.to(dev), X_cal=X.to(dev), sparsity=0.5, bits=4, group=128)
    torch.cuda.synchronize()
    t_compress = time.perf_counter() - t0
    pm_rm = m.packed()
    pm = pm_rm.to_tiled()
    xd = x.to(dev)
    y32 = ops.gemv(pm, xd, out_dtype=torch.float32)
    err = decode_parity(torch, ops, pm, xd, y32)
    assert err < 1e-3, f"config 0: decode off the dequantised weights by {err}"
    dense = xd.float() @ W.to(dev).T
    vs_dense = float((y32 - dense).norm() / dense.norm())
    copies = [pm] + [pm.clone() for _ in range(-(-2 * INFINITY_CACHE // pm.stream_bytes()) - 1)]
    st = torch.cuda.current_stream()
    y = None
    for c in copies:
        y = ops.gemv(c, xd)
    torch.cuda.synchronize()
    g_ = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream(dev)
    stream.wait_stream(st)
    with torch.cuda.stream(stream):
        ys = torch.empty(1, K, dtype=torch.float16, device=dev)
        P = ctypes.c_void_p
        xdt = F.dtype_code(torch.float16)
        args = [((F.CbkDesc * 1)(c.desc()), (P * 1)(xd.data_ptr()), (ctypes.c_int64 * 1)(N), (P * 1)(ys.data_ptr()),
                 (ctypes.c_int64 * 1)(K)) for c in copies]

        def rotation():
            for d, xp, ldx, yp, ldy in args:
                rc = L.cbk_gemv_batch(1, d, xp, ldx, xdt, 1, yp, ldy, xdt, None, None, 0, stream.cuda_stream)
                if rc:
                    raise RuntimeError(L.cbk_strerror(rc).decode())
        rotation()
        stream.synchronize()
        with torch.cuda.graph(g_, stream=stream):
            rotation()
        for _ in range(3):
            g_.replay()
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        g_.replay()                                               # untimed, in front of the start event (see GraphTimer.measure)
        e0.record(stream)
        for _ in range(3):
            g_.replay()
        e1.record(stream)
        stream.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (3 * len(copies))
    nbytes = algorithmic_bytes(pm, 1)
    out = {"workload": "single linear layer 4096x4096, CoBALT-compressed on the GPU (column-balanced mask, sparsity 0.5, "
                       "OBS, 4-bit RTN, group 128) -> BLK1632_4, x 1x4096 fp16",
           "bpw": round(pm.bpw(), 4), "compress_and_pack_s": round(t_compress, 3), "decode_us": round(us, 2),
           "distinct_copies": len(copies), "bytes": nbytes, "gbs": round(nbytes / us / 1e3, 1),
           "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
           "rel_fro_vs_dequant_f64": float(f"{err:.3g}"), "rel_fro_vs_uncompressed_layer": float(f"{vs_dense:.3g}")}
    if cpu:
        from oracle import cbk_ref_c as C
        from oracle import torch_ref as T
        cpm = pm_rm.to("cpu")
        stride = cpm.data_bytes // K
        data = cpm.array("data")[: K * stride].reshape(K, stride)
        scale, zero = cpm.array("scale").reshape(K, -1), cpm.array("zero").reshape(K, -1)
        cs = cpm.array("col_scale").reshape(1, N)
        pk = dict(data=cpm.array("data").numpy(), scale=scale.numpy(), zero=zero.numpy())
        yo = C.forward(pk, K, N, cpm.layout, x.float().numpy(), col_scale=cs.numpy())
        out["gpu_vs_oracle_rel_fro"] = float(np.linalg.norm(y32.cpu().numpy() - yo) / np.linalg.norm(yo))
        assert out["gpu_vs_oracle_rel_fro"] < 1e-3
        ta = []
        for i in range(6):
            t0 = time.perf_counter()
            Wh = T.dequant(data, scale, zero, cs, K, N, cpm.layout, 4, 128, 16)
            T.forward(Wh, x)
            ta.append(time.perf_counter() - t0)
        out["cpu_dequant_matmul_ms"] = round(sorted(ta[1:])[2] * 1e3, 2)
        out["cpu_note"] = "torch float32 dequantise-then-matmul of the same packed bytes on the host cores, median of 5 after a warm-up"
    del copies, g_
    torch.cuda.empty_cache()
    return out


def config2_block(torch, F, ops, L, dev, steps, warmup, use_graph=True):
    """Mistral-7B shapes at sparsity 0.7 (10 survivors per 32 columns), 3-bit codes, group 128:
    decode at M=1 and the MLP prefill at M=2048, fp16 activations, each with its parity figure."""
    dec = decode_rows_sweep(torch, F, L, dev, "mistral7b", F.BLKC, 3, 128, 10, [1], steps, warmup, use_graph, parity=True, ops=ops)[1]
    pf = prefill_gemm(torch, F, ops, dev, SHAPES["mistral7b"], ["gate", "up", "down"], F.BLKC, 3, 128, 10, 2048, torch.float16,
                      reps=10, warm=5)
    pf["workload"] = "mistral7b MLP (gate, up, down), M=2048, f16 activations"
    return {"workload": "mistral7b shapes, sparsity 0.6875 (10 of 32 kept), 3-bit codes across word boundaries, group 128, "
                        "f16 activations", "decode_m1": dec, "prefill_m2048": pf}


# ------------------------------------------------------------------ ceilings and CPU baseline
def measured_ceilings(torch, dev):
    """What this GPU reaches on back-to-back dense f16 MFMAs and on a plain streaming read of
    1 GiB (libcbk_bench.so, built by `python -m cobalt_amd.build`): ceilings to read the kernels'
    figures against, beside the published peaks.  None if the helper library is not built."""
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


def copy_calibration(torch, dev):
    """A 1 GiB device-to-device copy: the known reading the HBM traffic counters are scaled by."""
    src = torch.empty(2**30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return platform.processor() or "unknown"


def cpu_baseline(torch, pms, shapes, xs, ys, M, budget_s=18.0, prefill_budget_s=14.0, prefill_m=256, prefill_to=2048):
    """The reference's CPU forward restated in torch (oracle/torch_ref.py): per distinct shape of
    the layer set, (i) dequantise-then-matmul per call (the module's low-memory path,
    benchmarks/benchmark_suite.py:1201-1209) and (ii) matmul with the dequantised weights cached
    (:1210-1217), float32, all the host cores this process may use; on the packed bytes the GPU
    used.  Decode leg at M rows: one warm-up, then the median of 5 runs (fewer only if the time
    budget runs out, and the JSON says how many).  Prefill leg at `prefill_m` rows per distinct
    shape, with the figure for `prefill_to` rows extrapolated (dequantisation once, matmul time
    in proportion to the rows) and flagged as such.  The C oracle checks the GPU outputs of the
    same layer set first."""
    import numpy as np
    from oracle import cbk_ref_c as C
    from oracle import torch_ref as T
    usable = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    # the GPU boxes share their host: a process is given 16 cores whatever os.cpu_count() shows
    cores = max(1, min(usable, int(os.environ.get("OMP_NUM_THREADS", usable) or usable)))
    torch.set_num_threads(cores)
    C.set_threads(min(16, cores))
    worst = 0.0
    for pm, (name, K, N) in zip(pms, shapes):                       # parity of the GPU outputs (checker, untimed)
        pk = dict(data=pm.array("data").numpy(), scale=pm.array("scale").numpy().reshape(K, -1),
                  zero=pm.array("zero").numpy().reshape(K, -1))
        cs = pm.array("col_scale").numpy().reshape(pm.cs_rows, N) if pm.cs_rows else None
        y = C.forward(pk, K, N, pm.layout, xs[N].float().cpu().numpy(), col_scale=cs, bits=pm.bits, group=pm.group,
                      keep_per_block=pm.keep or None)
        got = ys[name].float().cpu().numpy()
        worst = max(worst, float(np.linalg.norm(got - y) / np.linalg.norm(y)))
    rows, prows, seen = [], [], set()
    tot_bytes = tot_a = tot_b = 0.0
    order = sorted(range(len(shapes)), key=lambda i: shapes[i][1] * shapes[i][2])       # small shapes first
    distinct = []
    for i in order:
        if (shapes[i][1], shapes[i][2]) not in seen:
            seen.add((shapes[i][1], shapes[i][2]))
            distinct.append(i)

    def arrays(pm, K, N):
        stride = pm.data_bytes // K
        return (pm.array("data")[: K * stride].reshape(K, stride), pm.array("scale").reshape(K, -1), pm.array("zero").reshape(K, -1),
                pm.array("col_scale").reshape(pm.cs_rows, N) if pm.cs_rows else None)

    med = lambda v: sorted(v)[len(v) // 2]
    t_stop = time.time() + budget_s
    for i in distinct:
        name, K, N = shapes[i]
        if rows and time.time() > t_stop:
            break
        pm = pms[i]
        data, scale, zero, cs = arrays(pm, K, N)
        x = xs[N].cpu()
        deq = lambda: T.dequant(data, scale, zero, cs, K, N, pm.layout, pm.bits, pm.group, pm.keep or 16)
        W = deq()
        T.forward(W, x)                                               # warm-up of both parts
        ta, tb = [], []
        for _ in range(5):
            t0 = time.perf_counter()
            W = deq()
            y = T.forward(W, x)
            ta.append(time.perf_counter() - t0)
            if time.time() > t_stop and len(ta) >= 3:
                break
        for _ in range(5):
            t0 = time.perf_counter()
            y = T.forward(W, x)
            tb.append(time.perf_counter() - t0)
        a, b = med(ta), med(tb)
        nbytes = algorithmic_bytes(pm, M)
        mult = sum(1 for _, k, n in shapes if (k, n) == (K, N))
        tot_bytes += nbytes * mult
        tot_a += a * mult
        tot_b += b * mult
        rows.append({"matrix": f"{name} {K}x{N}", "dequant_matmul_ms": round(a * 1e3, 2), "matmul_cached_ms": round(b * 1e3, 3),
                     "runs": [len(ta), len(tb)]})
        del W, y
    # prefill leg
    t_stop = time.time() + prefill_budget_s
    pf_flop = pf_s = 0.0
    for i in distinct:
        name, K, N = shapes[i]
        if prows and time.time() > t_stop:
            break
        pm = pms[i]
        data, scale, zero, cs = arrays(pm, K, N)
        x = torch.randn(prefill_m, N, generator=torch.Generator().manual_seed(N)).to(xs[N].dtype)
        W = T.dequant(data, scale, zero, cs, K, N, pm.layout, pm.bits, pm.group, pm.keep or 16)
        T.forward(W, x)
        td, tm = [], []
        for _ in range(5):
            t0 = time.perf_counter()
            W = T.dequant(data, scale, zero, cs, K, N, pm.layout, pm.bits, pm.group, pm.keep or 16)
            t1 = time.perf_counter()
            y = T.forward(W, x)
            t2 = time.perf_counter()
            td.append(t1 - t0)
            tm.append(t2 - t1)
            if time.time() > t_stop and len(td) >= 3:
                break
        d_, m_ = med(td), med(tm)
        ext = d_ + m_ * prefill_to / prefill_m
        mult = sum(1 for _, k, n in shapes if (k, n) == (K, N))
        pf_flop += 2.0 * prefill_to * K * N * mult
        pf_s += ext * mult
        prows.append({"matrix": f"{name} {K}x{N}", "M": prefill_m, "dequant_ms": round(d_ * 1e3, 2), "matmul_ms": round(m_ * 1e3, 2),
                      "runs": len(td), f"extrapolated_ms_at_M{prefill_to}": round(ext * 1e3, 1), "extrapolated": True})
        del W, y
    done = "+".join(r["matrix"].split()[0] for r in rows)
    return dict(value=round(tot_bytes / tot_a / 1e9, 4), unit="GB/s", cores=cores, kind="port",
                sample=f"torch {torch.__version__} float32 dequantise-then-matmul per call at M={M} over the distinct shapes "
                       f"{done} of the first layer set (same packed bytes as the GPU run), median of 5 runs each (see `runs`) "
                       f"after one warm-up, {cores} threads on {cpu_model()} ({os.cpu_count()} logical CPUs visible); `value` is the "
                       f"algorithmic bytes of those matrices per second of the per-call path; `matmul_cached_gbs` is the "
                       f"same bytes over the matmul with cached float32 weights (median of 5); `prefill` is the same path "
                       f"at M={prefill_m}, its M={prefill_to} figures extrapolated, not measured",
                matmul_cached_gbs=round(tot_bytes / tot_b / 1e9, 3), per_matrix=rows,
                ms_per_layer_set_dequant_matmul=round(tot_a * 1e3, 1), ms_per_layer_set_matmul_cached=round(tot_b * 1e3, 2),
                prefill={"M_measured": prefill_m, "M_extrapolated_to": prefill_to, "per_matrix": prows,
                         "extrapolated_tflops": round(pf_flop / pf_s / 1e12, 3) if pf_s else None,
                         "shapes_done": "+".join(r["matrix"].split()[0] for r in prows),
                         "note": "dequantise once + matmul time scaled by rows; an extrapolation, flagged per row"},
                gpu_vs_oracle_rel_fro=worst, checker="C oracle (oracle/cbk_ref.c) on every matrix of the first layer set")


# ------------------------------------------------------------------ the nine-cell grid
def grid(torch, F, ops, L, dev, a, prefill_reps=5, prefill_warm=3):
    """Gemma-3-27B shapes x 62 layers, sparsity 0.3 / 0.5 / 0.7 as 23 / 16 / 10 survivors per 32
    columns, 2 / 3 / 4-bit codes, group 64: decode step at M=1 and prefill at M=4096, bf16."""
    shapes = SHAPES["gemma27b"]
    dt = torch.bfloat16
    params = sum(K * N for _, K, N in shapes)
    cells = []
    for keep in (23, 16, 10):
        for bits in (2, 3, 4):
            sets, _ = make_sets(torch, F, dev, shapes, F.BLKC, bits, 64, keep, 2 * INFINITY_CACHE)
            res, _, _ = decode_layer_sets(torch, F, L, dev, shapes, sets, 1, dt, "phase", a.steps, a.warmup, not a.no_graph)
            bpw = sets[0][0].bpw()
            del sets
            torch.cuda.empty_cache()
            pf = prefill_gemm(torch, F, ops, dev, shapes, [n for n, _, _ in shapes], F.BLKC, bits, 64, keep, a.grid_prefill_m, dt,
                              reps=prefill_reps, warm=prefill_warm, parity=False)
            cell = {"sparsity": round(1 - keep / 32, 4), "keep_per_32": keep, "bits": bits, "group": 64, "bpw": round(bpw, 4),
                    "layer_set_bytes": res["step_bytes"],
                    "decode_ms_per_layer": round(res["ms_per_step"], 5), "decode_gbs": round(res["gbs"], 1),
                    "decode_frac_of_hbm_peak": round(res["gbs"] / HBM_PEAK_GBS, 4),
                    "decode_linear_ms_per_token_62_layers": round(res["ms_per_step"] * GEMMA_LAYERS, 3),
                    "prefill_ms_per_layer": pf["ms"], "prefill_tflops": pf["tflops"],
                    "prefill_frac_of_mfma_peak": round(pf["tflops"] / MFMA_PEAK_TFLOPS, 4),
                    "prefill_linear_us_per_token_62_layers": round(pf["ms"] * GEMMA_LAYERS * 1e3 / a.grid_prefill_m, 3)}
            cells.append(cell)
            print(json.dumps(cell), file=sys.stderr, flush=True)
    return {"metric": "decode GEMV HBM GB/s (% of 8 TB/s) at M=1; prefill GEMM TFLOP/s at M=4096", "mode": "grid",
            "config": {"workload": f"gemma27b 62-layer linear stack ({params} parameters per layer), bf16 activations, group 64, "
                                   f"sparsity 0.3/0.5/0.7 realised as 23/16/10 survivors per 32 columns, 2/3/4-bit codes; "
                                   f"decode M=1 (phase-batched launches from HIP graphs, distinct layer sets beyond 2x the "
                                   f"Infinity Cache in rotation, x62 for the stack), prefill M={a.grid_prefill_m} (all seven "
                                   f"matrices of a layer, x62)",
                       "steps": a.steps, "warmup": a.warmup},
            "n_gpus": 1, "data": "synthetic", "cells": cells}


# ------------------------------------------------------------------ main
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=640)
    ap.add_argument("--warmup", type=int, default=320)
    ap.add_argument("--workload", default="gemma27b", choices=list(SHAPES))
    ap.add_argument("--m", type=int, default=1)
    ap.add_argument("--dtype", default=None, choices=["f16", "bf16"], help="activation type (default: the workload's)")
    ap.add_argument("--bits", type=int, default=4)
    ap.add_argument("--keep", type=int, default=16)
    ap.add_argument("--group", type=int, default=128)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-core baseline")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill GEMM measurement")
    ap.add_argument("--no-lm-head", action="store_true", help="skip the output-projection GEMV measurement")
    ap.add_argument("--no-secondary", action="store_true", help="skip the other workload's decode step and the per-matrix rows")
    ap.add_argument("--prefill-workload", default="gemma27b", choices=list(SHAPES))
    ap.add_argument("--prefill-m", type=int, default=2048)
    ap.add_argument("--prefill-dtype", default="bf16", choices=["f16", "bf16"])
    ap.add_argument("--launch", default="phase", choices=["matrix", "phase", "layer"],
                    help="GEMVs per launch: one matrix, one dependency phase (qkv | o | gate,up | down), or the layer set")
    ap.add_argument("--no-graph", action="store_true", help="launch from the host instead of replaying HIP graphs")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 1 GiB device-to-device copy (reference reading for the HBM traffic counters)")
    ap.add_argument("--grid", action="store_true", help="the nine-cell sweep of the 62-layer Gemma stack instead of the headline")
    ap.add_argument("--grid-prefill-m", type=int, default=4096)
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the legs of the other benchmark configurations (single layer, M=4/8, 3-bit Mistral, the grid)")
    ap.add_argument("--only", default=None, choices=["per-matrix", "row-kernels"],
                    help="run one secondary leg alone (profiling runs): the per-matrix rows or the row-kernel layouts")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    from cobalt_amd import _lib, format as F, ops
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = _lib.lib()
    if a.grid:
        print(json.dumps(grid(torch, F, ops, L, dev, a)))
        return
    layout = layout_of(F, a.bits, a.keep, a.group)
    dname = a.dtype or WORKLOAD_DTYPE[a.workload]
    dt = torch_dtype(torch, dname)
    shapes = SHAPES[a.workload]
    M = a.m
    if a.only:                                                      # one leg alone, for profiler runs
        gate = [sh for sh in shapes if sh[0] == "gate"]
        if a.only == "per-matrix":
            rows = per_matrix(torch, F, L, dev, shapes, layout, a.bits, a.group, a.keep, M, dt, use_graph=not a.no_graph)
        else:
            rows = [dict(layout=F.LAYOUT_NAME[lay], **per_matrix(torch, F, L, dev, gate, lay, b, 128, None, M, dt, tiled=False,
                                                                 use_graph=not a.no_graph)[0])
                    for lay, b in ((F.SPARSE4X, 4), (F.DENSE8, 8))]
        if a.copy_calibration:
            copy_calibration(torch, dev)
        print(json.dumps({"leg": a.only, "workload": a.workload, "M": M, "rows": rows}))
        return

    sets, first_rowmajor = make_sets(torch, F, dev, shapes, layout, a.bits, a.group, a.keep, 2 * INFINITY_CACHE,
                                     keep_first_rowmajor=not a.no_cpu)
    bpw = sets[0][0].bpw()
    res, xs, y_first = decode_layer_sets(torch, F, L, dev, shapes, sets, M, dt, a.launch, a.steps, a.warmup, not a.no_graph)
    if a.copy_calibration:
        copy_calibration(torch, dev)
    del sets
    torch.cuda.empty_cache()

    ms_per_step, step_bytes, launches = res["ms_per_step"], res["step_bytes"], res["launches"]
    value = res["gbs"]
    # average launch of the decode kernel over the timed region (HIP events on the launch stream);
    # it contains the gap between consecutive launches, so it is an upper bound of the kernel time
    us_per_launch = ms_per_step * 1e3 / launches
    bytes_per_launch = step_bytes / launches
    achieved = bytes_per_launch / (us_per_launch * 1e-6) / 1e9
    traffic = MEASURED_TRAFFIC.get((a.workload, a.launch, M)) if (a.bits, a.keep, a.group) == (4, 16, 128) else None
    out = {
        "metric": "decode GEMV HBM GB/s (% of 8 TB/s) at M=1; prefill GEMM TFLOP/s at M=2048",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8 (int8 MFMA on integer codes and 3-digit block-fixed-point activations, f32 scales)",
        "data": "synthetic",
        "config": {"workload": f"{a.workload} decode layer set, 7 GEMVs, M={M}, {dname} activations, sparsity "
                               f"{1 - a.keep / 32:.4g}, {a.bits}-bit, group {a.group}, layout {F.LAYOUT_NAME[layout]}, "
                               f"{bpw:.4f} bpw",
                   "layer_set_bytes": step_bytes, "distinct_layer_sets": res["distinct_layer_sets"],
                   "launches_per_step": launches, "launch_grouping": a.launch,
                   "hip_graph": not a.no_graph, "graph_replays_timed": res["graph_replays_timed"],
                   "steps_per_full_graph": res["steps_per_full_graph"],
                   "steps_in_remainder_graph": res["steps_in_remainder_graph"],
                   "untimed_lead_replays": res["untimed_lead_replays"],
                   "warmup_steps_run": res["warmup_steps_run"], "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": ("stored figure of the rocprofv3 counter runs summarised under profiles/, "
                                        "not read in this run") if traffic else None,
                     "kernel": "cbk::gemv_mfma_kernel", "avg_launch_us": round(us_per_launch, 3),
                     "launches_timed": a.steps * launches, "bytes_per_launch": int(bytes_per_launch)},
    }
    if not a.no_secondary:
        out["per_matrix"] = per_matrix(torch, F, L, dev, shapes, layout, a.bits, a.group, a.keep, M, dt, use_graph=not a.no_graph)
        # the layouts off the main kernel, on the workload's gate matrix: SPARSE4X (rows of different
        # lengths: the 16-row matrix-core stream kernel) at one and at eight activation rows, DENSE8
        # (integer-dot row kernel)
        gate = [sh for sh in shapes if sh[0] == "gate"]
        out["row_kernel_layouts"] = [
            dict(layout=F.LAYOUT_NAME[lay], M=m_, **per_matrix(torch, F, L, dev, gate, lay, b, 128, None, m_, dt, tiled=False,
                                                               use_graph=not a.no_graph)[0])
            for lay, b, m_ in ((F.SPARSE4X, 4, M), (F.SPARSE4X, 4, 8), (F.DENSE8, 8, M))]
        other = "mistral7b" if a.workload == "gemma27b" else "gemma27b"
        oshapes, odt = SHAPES[other], torch_dtype(torch, WORKLOAD_DTYPE[other])
        osets, _ = make_sets(torch, F, dev, oshapes, layout, a.bits, a.group, a.keep, 2 * INFINITY_CACHE)
        ores, _, _ = decode_layer_sets(torch, F, L, dev, oshapes, osets, M, odt, a.launch, a.steps, a.warmup, not a.no_graph)
        out[f"decode_{other}"] = {"workload": f"{other} decode layer set, M={M}, {WORKLOAD_DTYPE[other]} activations, same layout",
                                  "ms_per_step": round(ores["ms_per_step"], 5), "gbs": round(ores["gbs"], 1),
                                  "frac_of_hbm_peak": round(ores["gbs"] / HBM_PEAK_GBS, 4),
                                  "layer_set_bytes": ores["step_bytes"], "distinct_layer_sets": ores["distinct_layer_sets"]}
        del osets
        torch.cuda.empty_cache()
    if not a.no_prefill:
        pdt = torch_dtype(torch, a.prefill_dtype)
        out["prefill_gemm"] = prefill_gemm(torch, F, ops, dev, SHAPES[a.prefill_workload], ["gate", "up", "down"], layout,
                                           a.bits, a.group, a.keep, a.prefill_m, pdt)
        out["prefill_gemm"]["workload"] = f"{a.prefill_workload} MLP (gate, up, down), M={a.prefill_m}, {a.prefill_dtype} activations"
        # the same kernel's 64-token tile at a batched-decoding row count, on the decode workload's shapes
        mid = prefill_gemm(torch, F, ops, dev, shapes, ["gate", "up", "down"], layout, a.bits, a.group, a.keep, 64, dt,
                           parity=False)
        out["gemm_m64"] = {"workload": f"{a.workload} MLP (gate, up, down), M=64, {dname} activations",
                           "tflops": mid["tflops"], "per_matrix": mid["per_matrix"]}
    if not a.no_lm_head:
        out["lm_head_gemv"] = lm_head_gemv(torch, F, ops, dev, a.workload, M, dt)
    if not a.no_configs:
        # the other configurations the benchmark names, each a block of its own
        g = not a.no_graph
        out["config0_single_layer"] = config0_single_layer(torch, F, ops, L, dev, cpu=not a.no_cpu)
        rows = {wl: decode_rows_sweep(torch, F, L, dev, wl, layout, a.bits, a.group, a.keep, [4, 8], a.steps, a.warmup, g,
                                      a.launch, parity=True, ops=ops) for wl in ("mistral7b", "gemma27b")}
        out["config1_mistral7b_m4"], out["config1_mistral7b_m8"] = rows["mistral7b"][4], rows["mistral7b"][8]
        out["config3_gemma27b_m4"], out["config3_gemma27b_m8"] = rows["gemma27b"][4], rows["gemma27b"][8]
        out["config2_mistral7b_b3_keep10"] = config2_block(torch, F, ops, L, dev, a.steps, a.warmup, g)
        cells = grid(torch, F, ops, L, dev, a, prefill_reps=3, prefill_warm=2)
        out["config4_grid"] = {"workload": cells["config"]["workload"], "cells": cells["cells"]}
    ceil = measured_ceilings(torch, dev)
    if ceil:
        out["measured_ceilings"] = ceil
        out["roofline"]["frac_of_measured_read"] = round(achieved / ceil["hbm_read_gbs"], 4)
        if "prefill_gemm" in out:
            out["prefill_gemm"]["roofline"]["frac_of_measured_mfma"] = round(
                out["prefill_gemm"]["tflops"] / ceil["mfma_f16_dense_tflops"], 4)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(torch, first_rowmajor, shapes, xs, y_first, M)
        assert out["cpu_baseline"]["gpu_vs_oracle_rel_fro"] < 1e-3, "GPU outputs disagree with the oracle"
    print(json.dumps(out))


if __name__ == "__main__":
    main()
