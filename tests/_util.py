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


def climbing_keys(k, ramp=8.0, spike=40.0):
    """K [B,Skv,H,D] with key n scaled by 1 + (ramp-1) n/(Skv-1), and one key three quarters along scaled by `spike`
    on top: the scores grow along the key axis, so the running softmax reference point has to move again and again
    (online_softmax.h:123-165), by more than the fp16 range (and, for the rows the spike key favours, more than the
    fp32 range of exp2) in one step."""
    skv = k.shape[1]
    w = 1.0 + (ramp - 1.0) * np.arange(skv, dtype=np.float32) / max(skv - 1, 1)
    w[(3 * skv) // 4 + 3 if skv > 4 else skv - 1] *= spike
    return k * w[None, :, None, None]
