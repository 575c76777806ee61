"""Seeded random shapes through the C-ABI against the CPU oracle: batch, heads, query and key lengths and head dim drawn
at random within what the tiles allow (query length a multiple of 128, key length of 64; the library picks tile, MFMA
shape and pipeline form by itself), for fp16, e4m3 and the hybrid mode.  The fixed-shape tests pin the cases the
reference's own driver runs; this one walks the combinations in between (odd key-tile counts against every tile
choice, rectangular problems, ragged grids).  Gates as in the fixed-shape tests: max-abs error against the fp32 host
reference attention (src/fmha-pipeline/fmha_forward.cu:599-683) within 2e-3 (fp16 P) / 5e-2 (e4m3 P)."""
import numpy as np
import pytest

import oracle
from _util import TOL_FP16, TOL_FP8, max_abs, pkg, to_dev

pytestmark = pytest.mark.gpu


def _shapes(seed, n):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        D = int(rng.choice([64, 128, 256]))
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 6))
        Sq = 128 * int(rng.integers(1, 7))
        Skv = 64 * int(rng.integers(1, 13))
        if rng.integers(0, 4) == 0:  # every fourth or so: a key length from which the e4m3 kernel walks the keys in two passes
            Skv, B, H, Sq = 64 * int(rng.integers(56, 72)), 1, int(rng.integers(1, 3)), 128 * int(rng.integers(1, 3))
        out.append((B, Sq, H, D, Skv))
    return out


def _quant(x):
    codes, scale = oracle.quantize_e4m3_per_tensor(x)
    return codes, float(scale), oracle.e4m3_decode(codes) * scale


@pytest.mark.parametrize("mode,seed", [("fp16", 11), ("fp8", 12), ("hybrid", 13)])
def test_random_shapes_match_the_oracle(mode, seed):
    import torch
    f = pkg.fmha
    for B, Sq, H, D, Skv in _shapes(seed, 10):
        q, k, v = pkg.testbed.qkv(B, Sq, H, D, seqlen_kv=Skv, seed=seed)
        if mode == "fp16":
            q16, k16, v16 = (x.astype(np.float16) for x in (q, k, v))
            plan = f.fmha_forward_plan(f.CFK_FP16, B, H, Sq, Skv, D)
            o = pkg.fmha_forward(to_dev(q16), to_dev(k16), to_dev(v16))
            qf, kf, vf = (x.astype(np.float32) for x in (q16, k16, v16))
            tol = TOL_FP16
        else:
            (qc, qs, qf), (kc, ks, kf) = _quant(q), _quant(k)
            if mode == "fp8":
                vc, vs, vf = _quant(v)
                plan = f.fmha_forward_plan(f.CFK_FP8_E4M3, B, H, Sq, Skv, D)
                o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=qs, k_descale=ks, v_descale=vs)
                tol = TOL_FP8
            else:
                v16 = v.astype(np.float16)
                vf = v16.astype(np.float32)
                plan = f.fmha_forward_plan(f.CFK_FP8_E4M3, B, H, Sq, Skv, D, v_dtype=f.CFK_FP16)
                o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(v16), q_descale=qs, k_descale=ks)
                tol = TOL_FP16
        torch.cuda.synchronize()
        got = o.float().cpu().numpy()
        ref = oracle.attention_f32(qf, kf, vf)["O"]
        err = max_abs(got, ref)
        print(f"{mode} B={B} S={Sq}/{Skv} H={H} D={D} tile {plan[0]}x{plan[1]}: max-abs {err:.3e}")
        assert not np.isnan(got).any(), (mode, B, Sq, H, D, Skv)
        assert err <= tol, (mode, B, Sq, H, D, Skv, err)
