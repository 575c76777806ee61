#!/usr/bin/env python3
"""Times FMHA forward on a seeded draw of problem sizes, one JSON line per problem (kernel chosen, ms, TFLOP/s), and
compares two such runs.  Companion of run_problem_sizes.sh: that one sweeps one dimension at a time at whole tiles, this
one mixes batch, heads, query length (whole 128-row tiles two times out of three, else any multiple of 32), key length
(any multiple of 64 for fp16, of 128 -- one time in three of 256, from 4096 -- for e4m3) and head dim, to find shapes
where the automatic choice (fmha_fwd_kernel.h: first_fit, hand_loop_pays) takes a hand-scheduled build and loses.  The
reference has no counterpart (its tile is a compile-time choice, src/fmha-pipeline/compile_run_all_config.sh:3-6).

  run_problem_draw.py --seed 80 --problems 120 > auto.jsonl
  CFK_FMHA_HANDLOOP=0 run_problem_draw.py --seed 80 --problems 120 > compiler.jsonl
  run_problem_draw.py --compare auto.jsonl compiler.jsonl
"""
import argparse
import json
import os
import statistics
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def draw(rng, it):
    import numpy as np  # noqa: F401
    f8 = it % 5 == 4
    D = int(rng.choice([64, 128, 256], p=[0.3, 0.4, 0.3])) if not f8 else int(rng.choice([64, 128, 256], p=[0.3, 0.5, 0.2]))
    Skv = 64 * int(rng.integers(2, 72)) if not f8 else 128 * int(rng.integers(4, 40)) if it % 3 else 256 * int(rng.integers(16, 20))
    Sq = 128 * int(rng.integers(1, 17)) if rng.integers(0, 3) else 32 * int(rng.integers(1, 65))
    B, H = int(rng.integers(1, 9)), int(rng.integers(1, 65))
    while (B * H * Sq * Skv > 1.2e10 or B * H * max(Sq, Skv) * D > 5e7) and B * H > 1:
        B, H = (B, H // 2) if H > 1 else (B // 2, H)
    rng.integers(0, 5)
    return f8, B, Sq, Skv, H, (128 if f8 else D)   # (e4m3: head dim 128, the one with a hand-scheduled build)


def run(seed, problems, launches):
    import numpy as np
    import torch
    sys.path.insert(0, ROOT)
    import __graft_entry__ as entry
    pkg = entry.load_package()
    f = pkg.fmha
    rng = np.random.default_rng(seed)
    for it in range(problems):
        f8, B, Sq, Skv, H, D = draw(rng, it)
        g = torch.Generator(device="cuda:0").manual_seed(1)

        def tensor(shape):
            x = torch.randn(shape, generator=g, device="cuda:0")
            return x.to(torch.float8_e4m3fn).view(torch.uint8) if f8 else x.half()
        q, k, v = tensor((B, Sq, H, D)), tensor((B, Skv, H, D)), tensor((B, Skv, H, D))
        o = torch.empty((B, Sq, H, D), dtype=torch.float16, device="cuda:0")
        kw = dict(q_descale=1.0, k_descale=1.0, v_descale=1.0) if f8 else {}
        name = f.fmha_forward_kernel(f.CFK_FP8_E4M3 if f8 else f.CFK_FP16, B, H, Sq, Skv, D)
        call = pkg.fmha_forward(q, k, v, o=o, prepare=True, **kw)
        for _ in range(30):
            call()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / launches
        print(json.dumps(dict(it=it, dtype="e4m3" if f8 else "fp16", B=B, Sq=Sq, Skv=Skv, H=H, D=D, kernel=name, ms=ms,
                              tflops=4.0 * B * H * Sq * Skv * D / ms / 1e9)), flush=True)


def compare(path_a, path_b):
    a = [json.loads(line) for line in open(path_a) if line.startswith("{")]
    b = [json.loads(line) for line in open(path_b) if line.startswith("{")]
    assert len(a) == len(b) and all(x["it"] == y["it"] for x, y in zip(a, b))
    same = [x["tflops"] / y["tflops"] for x, y in zip(a, b) if x["kernel"] == y["kernel"]]
    diff = sorted(((x["tflops"] / y["tflops"], x, y) for x, y in zip(a, b) if x["kernel"] != y["kernel"]), key=lambda r: r[0])
    print("%d problems; geometric mean of first / second: %.3f" % (len(a), statistics.geometric_mean([x["tflops"] / y["tflops"] for x, y in zip(a, b)])))
    if same:
        print("same kernel in both (%d): ratio %.3f .. %.3f (run-to-run noise)" % (len(same), min(same), max(same)))
    if diff:
        print("different kernels (%d): geometric mean %.3f" % (len(diff), statistics.geometric_mean([r[0] for r in diff])))
        for r, x, y in diff:
            print("  %.2f %s B=%d Sq=%d Skv=%d H=%d D=%d  %s %.0f | %s %.0f" % (r, x["dtype"], x["B"], x["Sq"], x["Skv"], x["H"], x["D"],
                                                                                 x["kernel"], x["tflops"], y["kernel"], y["tflops"]))


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--seed", type=int, default=80)
    ap.add_argument("--problems", type=int, default=120)
    ap.add_argument("--launches", type=int, default=100)
    ap.add_argument("--compare", nargs=2, metavar=("FIRST", "SECOND"))
    args = ap.parse_args()
    if args.compare:
        compare(*args.compare)
    else:
        run(args.seed, args.problems, args.launches)
