"""GPU parity on a seeded draw of problem sizes: batch, head count, query length, key length and head dim vary together,
so the automatic choice lands on most of the kernels (compiler-scheduled and hand-scheduled, 4 and 8 waves, with and
without leftover key tiles, one and several work items per workgroup) without the test naming any of them.  Every
problem is checked against the CPU oracle on every 211th query row of every (batch, head), to the same gates as the
other parity tests: max-abs error against the fp32 host reference attention, plus the reference's error percentage
(include/utils/random.hpp:54-90, thresholds src/fmha-pipeline/fmha_forward.cu:638-639)."""
import collections

import numpy as np
import pytest

import oracle
from _util import ERRPCT_FP8, ERRPCT_FP16, TOL_FP8, TOL_FP16, climbing_keys, max_abs, pkg, to_dev

pytestmark = pytest.mark.gpu

N_PROBLEMS = 40


def _draw(rng, it):
    dt = "f8" if it % 5 == 4 else "f16"
    D = int(rng.choice([64, 128, 256], p=[0.3, 0.4, 0.3])) if dt == "f16" else int(rng.choice([64, 128, 256], p=[0.3, 0.5, 0.2]))
    # key lengths: any multiple of the 64-key tile for fp16; e4m3 on both sides of the hand-scheduled kernel's minimum
    Skv = 64 * int(rng.integers(2, 72)) if dt == "f16" else 128 * int(rng.integers(4, 40)) if it % 3 else 256 * int(rng.integers(16, 20))
    # query lengths: whole 128-row tiles two times out of three, else any multiple of 32 rows (a partly filled last tile)
    Sq = 128 * int(rng.integers(1, 17)) if rng.integers(0, 3) else 32 * int(rng.integers(1, 65))
    B, H = int(rng.integers(1, 9)), int(rng.integers(1, 65))
    while (B * H * Sq * Skv > 1.2e10 or B * H * max(Sq, Skv) * D > 5e7) and B * H > 1:   # seconds per problem, host side
        B, H = (B, H // 2) if H > 1 else (B // 2, H)
    return dt, B, Sq, Skv, H, D, bool(rng.integers(0, 5) == 0)


def _quant(x):
    c, s = oracle.quantize_e4m3_per_tensor(x)
    return c, float(s), oracle.e4m3_decode(c) * s


def test_seeded_draw_of_problem_sizes():
    import torch
    f = pkg.fmha
    rng = np.random.default_rng(20240521)
    kernels = collections.Counter()
    for it in range(N_PROBLEMS):
        dt, B, Sq, Skv, H, D, climb = _draw(rng, it)
        q, k, v = pkg.testbed.qkv(B, Sq, H, D, seqlen_kv=Skv, seed=1000 + it)
        if climb:
            k, v = climbing_keys(k, ramp=6.0 if dt == "f16" else 4.0, spike=1.0), v / 4
        if dt == "f16":
            q16, k16, v16 = (x.astype(np.float16) for x in (q, k, v))
            name = f.fmha_forward_kernel(f.CFK_FP16, B, H, Sq, Skv, D)
            print(f"problem {it}: fp16 B={B} Sq={Sq} Skv={Skv} H={H} D={D} climb={climb} {name}", flush=True)
            o = pkg.fmha_forward(to_dev(q16), to_dev(k16), to_dev(v16))
            qf, kf, vf = (x.astype(np.float32) for x in (q16, k16, v16))
            tol, pct_limit = TOL_FP16, ERRPCT_FP16
        else:
            (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = _quant(q), _quant(k), _quant(v)
            name = f.fmha_forward_kernel(f.CFK_FP8_E4M3, B, H, Sq, Skv, D)
            print(f"problem {it}: e4m3 B={B} Sq={Sq} Skv={Skv} H={H} D={D} climb={climb} {name}", flush=True)
            o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=qs, k_descale=ks, v_descale=vs)
            tol, pct_limit = TOL_FP8, ERRPCT_FP8
        torch.cuda.synchronize()
        got = o.float().cpu().numpy()
        ref = np.full(got.shape, np.nan, np.float32)
        oracle.attention_f32(qf, kf, vf, bh_pairs=[(b, h) for b in range(B) for h in range(H)],
                             row_start=int(rng.integers(0, min(211, Sq))), row_step=211, out=ref)
        sel = ~np.isnan(ref)
        assert sel.sum() >= B * H * D
        assert np.all(np.isfinite(got)), (it, name)
        err = max_abs(got[sel], ref[sel])
        ok, pct = oracle.verify_tensor(got[sel], ref[sel], pct_limit)
        print(f"    checked {sel.sum()} elements: max-abs {err:.3e}, error% {pct:.2e}", flush=True)
        # (e4m3 weights on climbing keys: a handful of keys carry each row, so the 6 % rounding of a weight does not average
        # out and the percentage criterion, calibrated on N(0,1) scores, does not apply; max-abs does)
        assert err <= tol and (ok or (dt == "f8" and climb)), (it, name, err, pct)
        kernels[name] += 1
    print({n: c for n, c in kernels.items()})
    # the draw is only worth its time while it spreads over the kernels
    assert len(kernels) >= 10, kernels
    assert sum("16p" in n or "8p" in n for n in kernels) >= 4, kernels   # hand-scheduled builds among them
