"""Build the CPU oracle (oracle/kernels.cpp) into oracle/_build/liboracle.so.

Test infrastructure only: nothing in the product loads this library.
x86-64-v3 (AVX2 + FMA) is the code-generation baseline so the library built
in one container also runs on the GPU host.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "liboracle.so")


def build(force: bool = True) -> str:
    src = os.path.join(HERE, "kernels.cpp")
    if not force and os.path.exists(LIB) and os.path.getmtime(LIB) >= os.path.getmtime(src):
        return LIB
    os.makedirs(OUT_DIR, exist_ok=True)
    cmd = ["g++", "-O3", "-fopenmp", "-march=x86-64-v3", "-fno-fast-math",
           "-shared", "-fPIC", "-o", LIB, src]
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
