"""Build the CPU oracle (test infrastructure) into oracle/_build/libsessd_oracle.so.

The reference itself cannot be compiled here: its hot path is CUDA inside classes deriving from
TensorRT's IPluginV2DynamicExt, and neither nvcc nor the TensorRT headers exist in this image, so
there is no oracle/_ref build.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "_build", "libsessd_oracle.so")
SRC = os.path.join(HERE, "sessd_oracle.cpp")
# IEEE division, no FMA contraction: voxel coordinates and the summation order depend on it.
FLAGS = ["-O2", "-fno-fast-math", "-ffp-contract=off", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-fopenmp"]


def build(force=True):
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    cmd = ["g++"] + FLAGS + ["-o", OUT, SRC]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
