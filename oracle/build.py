"""Build recipe for the CPU oracle (test infrastructure, never the product).

`python oracle/build.py` compiles oracle/lbann_cpu_oracle.cpp into
oracle/liblbann_cpu_oracle.so with g++ and OpenMP.  The flags follow the
reference's plain CMake Release build (no -march, no fast-math), and
-ffp-contract=off keeps fused multiply-adds out so the fp32 rounding pattern
is the one an x86-64 baseline build of the reference produces.

The reference's own sources for this path cannot be compiled here (they need
Hydrogen, DiHydrogen, cereal, protobuf-generated headers and MPI, none of
which exist in the image), so there is no oracle/_ref build.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "lbann_cpu_oracle.cpp")
LIB = os.path.join(HERE, "liblbann_cpu_oracle.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(LIB) and os.path.getmtime(LIB) >= os.path.getmtime(SRC):
        return LIB
    cmd = ["g++", "-std=c++17", "-O3", "-fopenmp", "-ffp-contract=off", "-fPIC",
           "-shared", "-Wall", "-Wextra", "-o", LIB, SRC]
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(force=True))
    sys.exit(0)
