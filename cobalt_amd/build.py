"""Builds libcbk_hip.so (the C-ABI HIP library) in-tree with hipcc for gfx950."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libcbk_hip.so")
SOURCES = ["cbk_api.hip", "cbk_dequant.hip", "cbk_gemv_generic.hip", "cbk_gemv.hip", "cbk_gemm.hip", "cbk_gemm_big.hip",
           "cbk_gemm_big_b2.hip", "cbk_gemm_big_b3.hip", "cbk_gemm_big_b4.hip", "cbk_gemm_big_b6.hip"] + [
           f"cbk_gemm_big_b{b}_t{t}.hip" for b in (2, 3, 4) for t in (1, 2, 4)] + ["cbk_act.hip", "cbk_pack.hip"]
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-shared", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-inline-asm"]


def build_lib(verbose=True, extra=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for s in SOURCES:
        o = os.path.join(CSRC, s.replace(".hip", ".o"))
        cmd = [hipcc] + [f for f in FLAGS if f != "-shared"] + list(extra) + ["-c", os.path.join(CSRC, s), "-o", o]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(o)
    for s, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {s}:\n{out}")
        if verbose and out.strip():
            print(out)
    cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


BENCH_LIB = os.path.join(HERE, "libcbk_bench.so")


def build_bench_lib(verbose=True):
    """libcbk_bench.so: the measured-ceiling probes bench.py reports beside the published peaks."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + [os.path.join(CSRC, "cbk_bench.hip"), "-o", BENCH_LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed on cbk_bench.hip:\n" + out.stdout)
    return BENCH_LIB


if __name__ == "__main__":
    build_lib()
    build_bench_lib()
    print("built", LIB, BENCH_LIB)
