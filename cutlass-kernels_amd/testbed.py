"""Seeded synthetic inputs, after the reference driver's ``testFmhaForward``
(src/fmha-pipeline/fmha_forward.cu:479-500): Q, K, V iid N(0,1) with seeds 3080+{1,2,3}; or the integer-valued
uniform [-8, 8] fill the reference uses to make GEMM-I exact (include/utils/random.hpp:13-32,
src/fmha/fmha_forward.cu:671-674).  The reference draws from curand on the device; that stream is not
reproducible, so these use numpy's Philox with the same seeds.
"""
from __future__ import annotations

import numpy as np

SEED = 3080  # fmha_forward.cu:479


def _rng(seed):
    return np.random.Generator(np.random.Philox(seed))


def gaussian(shape, seed, dtype=np.float32):
    return _rng(seed).standard_normal(shape, dtype=np.float32).astype(dtype)


def uniform_int(shape, seed, lo=-8, hi=8, dtype=np.float32):
    return _rng(seed).integers(lo, hi + 1, shape).astype(dtype)


def uniform(shape, seed, lo=-1.0, hi=1.0, dtype=np.float32):
    """U(lo,hi), the cute-gemm fill (src/cute-gemm-tma-gma/gemm.cu:482-485)."""
    return (_rng(seed).random(shape, dtype=np.float32) * (hi - lo) + lo).astype(dtype)


def qkv(batch, seqlen, heads, head_dim, kind="gaussian", seqlen_kv=None, seed=SEED):
    """(Q, K, V) float32 in [B,S,H,D]; seeds seed+1, seed+2, seed+3 as the reference driver."""
    skv = seqlen if seqlen_kv is None else seqlen_kv
    f = gaussian if kind == "gaussian" else uniform_int
    return (f((batch, seqlen, heads, head_dim), seed + 1), f((batch, skv, heads, head_dim), seed + 2),
            f((batch, skv, heads, head_dim), seed + 3))


def fmha_flops(batch, heads, seqlen_q, seqlen_kv, head_dim) -> float:
    """4*B*H*Sq*Skv*D (fmha_forward.cu:572-573)."""
    return 4.0 * batch * heads * seqlen_q * seqlen_kv * head_dim
