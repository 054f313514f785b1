"""Builds the CPU checker (oracle/ft_oracle.cpp) into oracle/_build/libft_oracle.so.

Test infrastructure only. The reference itself is Rust (no cargo/rustc in this image, registry
crates not vendored), so there is no `oracle/_ref` build: the checker is this restatement, pinned
by the reference's fixtures in tests/golden/.
"""
from __future__ import annotations

import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_build")
LIB_PATH = os.path.join(OUT_DIR, "libft_oracle.so")

# -ffp-contract=off: Rust never fuses a*b+c. -O3 vectorises the independent-lane loops; without
# -ffast-math no floating-point reduction is reassociated, so sequential sums stay sequential.
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-fno-fast-math", "-fopenmp"]


def build_oracle() -> str:
    gxx = shutil.which("g++")
    if gxx is None:
        raise RuntimeError("g++ not found: cannot build the CPU checker")
    os.makedirs(OUT_DIR, exist_ok=True)
    tmp = LIB_PATH + ".tmp"
    cmd = [gxx, *FLAGS, os.path.join(HERE, "ft_oracle.cpp"), "-o", tmp, "-lm"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + proc.stdout)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_oracle())
