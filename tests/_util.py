"""Shared helpers of the parity tests: package loading, device transfer, error metrics."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

pkg = entry.load_package()

# Tolerances stated by the task for this path: max-abs error against the fp32 host reference attention.
TOL_FP16 = 2e-3
TOL_FP8 = 5e-2
# The reference's own gate (src/fmha-pipeline/fmha_forward.cu:638-639): error percentages.
ERRPCT_FP16 = 1e-4
ERRPCT_FP8 = 1e-3


def to_dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to("cuda:0")


def subset_pairs(B, H, seed=7):
    """First, last and two seeded-random (batch, head) problems."""
    rng = np.random.default_rng(seed)
    pairs = {(0, 0), (B - 1, H - 1)}
    while len(pairs) < min(4, B * H):
        pairs.add((int(rng.integers(B)), int(rng.integers(H))))
    return sorted(pairs)


def max_abs(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float32) - np.asarray(b, np.float32))))
