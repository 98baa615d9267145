"""Builds the C restatement of the oracle (oracle/cbk_ref.c) into oracle/libcbk_ref.so with gcc.

Test infrastructure: the shared object is loaded by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py only.  The reference itself is Python plus CUDA sources that
need nvcc and an NVIDIA GPU, so there is no oracle/_ref build of it here."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "cbk_ref.c")
LIB = os.path.join(HERE, "libcbk_ref.so")


def build_oracle_c(verbose=False):
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-Wall", "-Wextra", "-o", LIB, SRC, "-lm"]
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build_oracle_c(verbose=True))
