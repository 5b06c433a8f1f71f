"""Writes tests/golden/koleo_golden.npz: fp64 oracle loss, nearest-neighbour index and gradient of
the KoLeo diversity loss for small seeded cases.  Inputs are regenerated from the seeds, so only
results are stored.  Made by this repository's own oracle (the reference holds no vectors for this
function); a regression pin for the oracle and a fixed target for the HIP path.

    python tests/golden/make_golden_koleo.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import koleo_oracle as K  # noqa: E402

# name: (B, N, D, seed, offset added to the N(0,1) features)
CASES = {
    "gs_feature_like": (2, 96, 9, 5101, 0.0),
    "latent_like": (1, 24, 512, 5102, 0.0),
    "one_orthant": (1, 70, 5, 5103, 1.0),
    "ragged": (3, 33, 17, 5104, 0.0),
}


def inputs(case):
    B, N, D, seed, off = CASES[case]
    x = torch.randn(B, N, D, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * (0.2 if off else 1.0)
    return (x + off).to(torch.float32).to(torch.float64)      # exactly representable in fp32


def compute(case):
    x = inputs(case)
    val, idx, gap = K.nearest_neighbours(x)
    return x, {"loss": K.koleo_diversity_loss(x), "nearest": val, "index": idx, "gap": gap,
               "grad": K.koleo_backward(x, grad_loss=1.0)}


if __name__ == "__main__":
    blob = {}
    for case in CASES:
        _, res = compute(case)
        for k, v in res.items():
            blob[f"{case}/{k}"] = v.numpy()
    path = os.path.join(HERE, "koleo_golden.npz")
    np.savez_compressed(path, **blob)
    print(path, os.path.getsize(path), "bytes")
