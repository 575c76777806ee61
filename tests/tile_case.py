"""Helper of test_tiles.py (not a test module): runs FMHA forward cases in THIS process -- whose environment carries
the tile wish CFK_FMHA_TILE, read once per process by the library -- and prints one JSON line per case with the
tile the library planned and the errors against the CPU oracle.

usage: tile_case.py mode:B,S,H,D[,Skv] ...      mode = f16 | f16nt | f8 | hyb, with the suffix `climb` for keys whose
scores climb along the key axis (tests/_util.py: climbing_keys); f16nt = fp16 without the row taps (the hand-scheduled
build serves calls with taps through its max-tracking loop: only a call without them runs the scheduled loop)
"""
import json
import sys

import numpy as np

import oracle
from _util import climbing_keys, max_abs, pkg, to_dev


def run_case(spec):
    import torch
    mode, dims = spec.split(":")
    vals = [int(x) for x in dims.split(",")]
    B, S, H, D = vals[:4]
    Skv = vals[4] if len(vals) > 4 else S
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=Skv)
    if mode.endswith("climb"):
        mode = mode[:-5]
        # (e4m3 P has two binades above the reference point where fp16 P has eight: a gentler climb already takes every slow path)
        k, v = (climbing_keys(k, ramp=4.0, spike=8.0) if mode == "f8" else climbing_keys(k)), v / 4
    f = pkg.fmha
    mfma = 32
    no_taps = mode == "f16nt"
    if no_taps: mode = "f16"
    if mode == "f16":
        q16, k16, v16 = (x.astype(np.float16) for x in (q, k, v))
        plan = f.fmha_forward_plan(f.CFK_FP16, B, H, S, Skv, D)
        mfma = f.fmha_forward_mfma(f.CFK_FP16, B, H, S, Skv, D)
        rm = torch.full((B, H, S), -1.0, dtype=torch.float32, device="cuda:0")
        rs = torch.full((B, H, S), -1.0, dtype=torch.float32, device="cuda:0")
        if no_taps: o = pkg.fmha_forward(to_dev(q16), to_dev(k16), to_dev(v16))
        else: o = pkg.fmha_forward(to_dev(q16), to_dev(k16), to_dev(v16), row_max=rm, row_sum=rs)
        qf, kf, vf = (x.astype(np.float32) for x in (q16, k16, v16))
    else:
        (qc, qs), (kc, ks) = oracle.quantize_e4m3_per_tensor(q), oracle.quantize_e4m3_per_tensor(k)
        qf, kf = oracle.e4m3_decode(qc) * qs, oracle.e4m3_decode(kc) * ks
        if mode == "f8":
            vc, vs = oracle.quantize_e4m3_per_tensor(v)
            vf = oracle.e4m3_decode(vc) * vs
            plan = f.fmha_forward_plan(f.CFK_FP8_E4M3, B, H, S, Skv, D)
            o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=float(qs), k_descale=float(ks),
                                 v_descale=float(vs))
        else:
            v16 = v.astype(np.float16)
            vf = v16.astype(np.float32)
            plan = f.fmha_forward_plan(f.CFK_FP8_E4M3, B, H, S, Skv, D, v_dtype=f.CFK_FP16)
            o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(v16), q_descale=float(qs), k_descale=float(ks))
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    # full check of the first and last (batch, head), every 29th row of the others
    pairs = sorted({(0, 0), (B - 1, H - 1)})
    ref = oracle.attention_f32(qf, kf, vf, bh_pairs=pairs)["O"]
    oracle.attention_f32(qf, kf, vf, bh_pairs=[(b, h) for b in range(B) for h in range(H)], row_start=5, row_step=29,
                         out=ref)
    sel = ~np.isnan(ref)
    _, pct = oracle.verify_tensor(got[sel], ref[sel])
    taps = None
    if mode == "f16" and not no_taps:
        # the row-max / row-sum taps of the first and last (batch, head): log2-domain max, sum not reciprocal
        st = oracle.attention_f32(qf, kf, vf, bh_pairs=pairs, want_stats=True)
        m_ref, inv_ref = st["row_max"], st["inv_sum"]
        ok = ~np.isnan(m_ref)
        mi = rm.cpu().numpy() / oracle.LOG2E
        taps = [float(np.abs(mi[ok] - m_ref[ok]).max() / max(1.0, np.abs(m_ref[ok]).max())),
                float(np.abs(1.0 / rs.cpu().numpy()[ok] / inv_ref[ok] - 1.0).max())]
    return dict(taps=taps, case=spec, block_m=plan[0], block_n=plan[1], mfma=mfma, lds_bytes=plan[2], checked=int(sel.sum()),
                max_abs=max_abs(got[sel], ref[sel]), err_pct=pct, nan=bool(np.isnan(got).any()))


if __name__ == "__main__":
    for spec in sys.argv[1:]:
        print("TILECASE " + json.dumps(run_case(spec)), flush=True)
