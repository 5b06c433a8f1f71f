"""Writes tests/golden/gs2d_golden.npz: fp64 oracle outputs and gradients for small seeded
cases.  Inputs are regenerated from the seeds by oracle.gs2d_oracle.make_inputs, so only
results are stored.  Made by this repository's own oracle (the reference holds no vectors
for this path); it is a regression pin for the oracle and a fixed target for the HIP path.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import gs2d_oracle as O  # noqa: E402

# name: kwargs of make_inputs
CASES = {
    "c1_like": dict(B=2, N=96, H=24, W=40, C=3, smin=0.02, smax=0.3, colors="uniform", seed=4101),
    "c0_like": dict(B=1, N=37, H=16, W=16, C=3, smin=0.25, smax=0.75, colors="uniform", seed=4100),
    "c4_like": dict(B=1, N=128, H=12, W=20, C=16, smin=0.02, smax=0.15, colors="normal", seed=4104),
    "one_channel": dict(B=1, N=50, H=9, W=31, C=1, smin=0.05, smax=0.4, colors="uniform", seed=4105),
}


def compute(case):
    d = O.make_inputs(dtype=torch.float64, **CASES[case])
    out, g = O.render_autograd(d["positions"], d["colors"], d["scales"], d["rotations"], d["alphas"],
                               d["x_grid"], d["y_grid"], d["grad_out"])
    res = {"out": out}
    res.update({"g_" + k: v for k, v in g.items()})
    return d, res


if __name__ == "__main__":
    blob = {}
    for case in CASES:
        _, res = compute(case)
        for k, v in res.items():
            blob[f"{case}/{k}"] = v.numpy()
    path = os.path.join(HERE, "gs2d_golden.npz")
    np.savez_compressed(path, **blob)
    print(path, os.path.getsize(path), "bytes")
