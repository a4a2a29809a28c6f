#!/usr/bin/env python3
"""Writes tests/golden/c1_causal_seed0.npz: expected output and logsumexp of the first
benchmark configuration (causal, B=1 H=8 S=512 D=64 fp16, seed 0), computed by the fp32
dense oracle of this repository on the CPU.  The inputs are not stored: they are
regenerated from the seed by baseline_configs.make_workload.  Run from the repo root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "omni-attention_amd")]

from baseline_configs import make_workload  # noqa: E402
from oracle.dense_oracle import attention_dense_fp32, prefix_mask  # noqa: E402


def main():
    w = make_workload("c1_causal", seed=0)
    S = w.q.shape[2]
    o, lse = attention_dense_fp32(w.q, w.k, w.v, prefix_mask(w.prefix_len, S).unsqueeze(1))
    path = os.path.join(HERE, "c1_causal_seed0.npz")
    np.savez_compressed(path, o=o.numpy(), lse=lse.numpy(),
                        q_checksum=np.float64(w.q.double().sum().item()))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
