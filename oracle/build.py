#!/usr/bin/env python3
"""Compile the C restatement (block_walk.c) into oracle/_build/libomni_oracle.so."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "libomni_oracle.so")


def build() -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    cmd = ["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-Wall",
           os.path.join(HERE, "block_walk.c"), "-o", LIB, "-lm"]
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print("built", build())
    sys.exit(0)
