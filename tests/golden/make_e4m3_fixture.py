"""Writes tests/golden/e4m3_fixture.npz: the OCP e4m3fn codec as torch.float8_e4m3fn implements it, independent of the
oracle's own codec (oracle.e4m3_decode / e4m3_encode), which tests/test_oracle.py checks against this file.

  decode  float32[256]   value of every code (NaN for 0x7F / 0xFF)
  x       float32[n]     probe values: every midpoint between neighbouring representable magnitudes, its two float32
                         neighbours, the representable values themselves, both signs, and 4096 N(0,1)*2^k samples
  codes   uint8[n]       torch's round-to-nearest-even encoding of clamp(x, -448, 448) -- torch itself maps overflow to
                         NaN; the kernels and the reference (cutlass::float_e4m3_t, satfinite) saturate

Run from the repository root:  python tests/golden/make_e4m3_fixture.py
"""
import os

import numpy as np
import torch

here = os.path.dirname(os.path.abspath(__file__))
decode = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
mags = np.sort(decode[:0x7F].astype(np.float64))                      # 0 .. 448, ascending
mids = ((mags[:-1] + mags[1:]) / 2).astype(np.float32)                # exactly representable in float32
probes = np.concatenate([mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
                         mags.astype(np.float32), np.array([448.0, 449.0, 463.9, 464.0, 1e9], np.float32)])
rng = np.random.default_rng(20240607)
rand = np.concatenate([rng.standard_normal(512).astype(np.float32) * np.float32(2.0 ** k) for k in range(-10, 6, 2)])
x = np.concatenate([probes, -probes, rand]).astype(np.float32)
codes = torch.from_numpy(np.clip(x, -448.0, 448.0)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
np.savez_compressed(os.path.join(here, "e4m3_fixture.npz"), decode=decode, x=x, codes=codes)
print("wrote e4m3_fixture.npz:", x.size, "probe values")
