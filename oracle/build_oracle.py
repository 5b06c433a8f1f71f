"""Builds the C brute-force checker (oracle/libgs2d_bruteforce.so) with gcc.

The reference is pure Python (no C/C++ sources), so there is no `oracle/_ref` build."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "gs2d_bruteforce.c")
OUT = os.path.join(HERE, "libgs2d_bruteforce.so")


def build(force: bool = True) -> str:
    if force or not os.path.exists(OUT) or os.path.getmtime(OUT) < os.path.getmtime(SRC):
        subprocess.check_call(["gcc", "-O2", "-shared", "-fPIC", "-o", OUT, SRC, "-lm"])
    return OUT


if __name__ == "__main__":
    print(build())
