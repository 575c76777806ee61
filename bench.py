#!/usr/bin/env python3
"""FMHA-forward benchmark on one MI355X: prints ONE JSON line.

Headline workload (benchmark configuration 2): fp16, B=8 H=16 S=2048 D=128, non-causal, Q/K/V iid N(0,1) synthetic, fp32
softmax/accumulate, fp16 output.  A "step" is one forward call over the whole batch through the C-ABI
(``cfk_fmha_forward``), inputs resident in HBM.  FLOP = 4*B*H*Sq*Skv*D per step
(src/fmha-pipeline/fmha_forward.cu:572-573); timing protocol = the reference's: warm-up launches, then the mean of
K back-to-back launches between events (fmha_forward.cu:578-593).

Also reported in the same line: ``roofline`` (MFMA-bound; achieved TFLOP/s over the measured mean launch duration
against the published dense peak), ``cpu_baseline`` (the CPU oracle -- a restatement of the reference's host
reference attention -- timed on this host's cores on a bounded sample of the same workload), and ``secondary``
(the other single-GPU workloads: fp8 e4m3 config 4, the long-sequence config 3, the GEMM example).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f16": 2500.0, "f8": 5000.0, "f32": 157.3}   # MI355X published dense MFMA peaks
# HBM bytes per launch, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch, two runs) and scaled by what
# the same counters read for a plain device copy of known size in the same session.  Every figure names the profile it
# was read from and the kernel it was read for: tests/test_bench_contract.py parses the figures out of those files and
# checks that the kernel is the one the library picks for the workload, so a stale figure fails in the CPU suite.
COPY_CALIBRATION = dict(profile="profiles/fmha_fwd_f16_B8_H16_S2048_D128.md", kernel="__amd_rocclr_copyBuffer",
                        known_kib=262144, fetch_kib=131090, write_kib=262144)
TRAFFIC_SOURCE = {
    "cfg2": dict(profile="profiles/fmha_fwd_f16_B8_H16_S2048_D128.md", kernel="fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>",
                 fetch_kib=107998, write_kib=65536),
    "cfg3": dict(profile="profiles/fmha_fwd_f16_B2_H8_S8192_D256.md", kernel="fmha_fwd_kernel16p<256,32,4,1,0,0,0,0,2,0,1,1>",
                 fetch_kib=172627, write_kib=65536),
    "cfg4": dict(profile="profiles/fmha_fwd_fp8_B4_H16_S4096_D128.md", kernel="fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>",
                 fetch_kib=53713, write_kib=65536),
    "cfg5": dict(profile="profiles/gemm_M8192_N8192_K8192.md", kernel="gemm_kernel16<0,4>", fetch_kib=787716, write_kib=131072),
}


def measured_traffic(workload):
    """(HBM bytes per launch, where the figure comes from) or (None, None) for a workload that has no counter run."""
    t = TRAFFIC_SOURCE.get(workload)
    if t is None:
        return None, None
    c = COPY_CALIBRATION
    kib = t["fetch_kib"] * c["known_kib"] / c["fetch_kib"] + t["write_kib"] * c["known_kib"] / c["write_kib"]
    return int(round(kib * 1024)), {"profile": t["profile"], "kernel": t["kernel"], "FETCH_SIZE_KiB": t["fetch_kib"],
                                    "WRITE_SIZE_KiB": t["write_kib"],
                                    "fetch_scale": round(c["known_kib"] / c["fetch_kib"], 4),
                                    "write_scale": round(c["known_kib"] / c["write_kib"], 4)}


WORKLOADS = {
    "cfg1": dict(kind="fmha", dtype="f16", B=1, H=8, S=512, D=64, scale=0.125),
    "cfg2": dict(kind="fmha", dtype="f16", B=8, H=16, S=2048, D=128, scale=None),
    "cfg3": dict(kind="fmha", dtype="f16", B=2, H=8, S=8192, D=256, scale=None),
    "cfg4": dict(kind="fmha", dtype="f8", B=4, H=16, S=4096, D=128, scale=None),
    "cfg5": dict(kind="gemm", dtype="f16", M=8192, N=8192, K=8192),
    # the data-dependent side of the e4m3 kernel: keys whose scores climb along the key axis send every workgroup through
    # its second (max-tracking) pass; `one_pass` runs the same data under cfk_set_option(CFK_OPT_PREDICTABLE_LATENCY, 1)
    "cfg4_climb": dict(kind="fmha", dtype="f8", B=4, H=16, S=4096, D=128, scale=None, climb=True),
    "cfg4_climb_one_pass": dict(kind="fmha", dtype="f8", B=4, H=16, S=4096, D=128, scale=None, climb=True, one_pass=True),
    "cfg4_one_pass": dict(kind="fmha", dtype="f8", B=4, H=16, S=4096, D=128, scale=None, one_pass=True),
    # cfk_set_option(CFK_OPT_FAST_E4M3_WEIGHTS, 1): e4m3 weights written as codes, without an exponential (an option: a
    # fifth of the weights are then one e4m3 step off the correctly rounded one)
    "cfg4_fast_weights": dict(kind="fmha", dtype="f8", B=4, H=16, S=4096, D=128, scale=None, fast_weights=True),
    "d64_f8_fast_weights": dict(kind="fmha", dtype="f8", B=4, H=32, S=4096, D=64, scale=None, fast_weights=True),
    # one sequence, 256 work items of 128 rows: what the 4-wave shapes of the hand-scheduled loops are for
    "b1_f16": dict(kind="fmha", dtype="f16", B=1, H=16, S=2048, D=128, scale=None),
    "b1_f8": dict(kind="fmha", dtype="f8", B=1, H=8, S=4096, D=128, scale=None),
    "d64_f16": dict(kind="fmha", dtype="f16", B=4, H=32, S=4096, D=64, scale=None),   # the reference sweep's head size 64
    "d64_f8": dict(kind="fmha", dtype="f8", B=4, H=32, S=4096, D=64, scale=None),
    "gemm_f32": dict(kind="gemm", dtype="f32", M=8192, N=8192, K=8192, max_steps=50),  # the CuTe example's type 1
}
NAMES = {
    "cfg1": "fmha_fwd fp16 B=1 H=8 S=512 D=64 non-causal",
    "cfg2": "fmha_fwd fp16 B=8 H=16 S=2048 D=128 non-causal",
    "cfg3": "fmha_fwd fp16 B=2 H=8 S=8192 D=256 non-causal",
    "cfg4": "fmha_fwd fp8-e4m3 B=4 H=16 S=4096 D=128 non-causal, per-tensor amax scales, V [B,S,H,D]",
    "cfg5": "gemm fp16 M=N=K=8192 TN fp32-accumulate",
    "b1_f16": "fmha_fwd fp16 B=1 H=16 S=2048 D=128 non-causal (one sequence: 256 work items of 128 rows)",
    "b1_f8": "fmha_fwd fp8-e4m3 B=1 H=8 S=4096 D=128 non-causal (one sequence: 256 work items of 128 rows)",
    "cfg4_climb": "fmha_fwd fp8-e4m3 B=4 H=16 S=4096 D=128, keys scaled 1..4 along the key axis and one key x8 (scores climb: "
                  "every workgroup takes the second, max-tracking pass)",
    "cfg4_climb_one_pass": "... the same data with cfk_set_option(CFK_OPT_PREDICTABLE_LATENCY, 1): max-tracking pass only",
    "cfg4_one_pass": "fmha_fwd fp8-e4m3 B=4 H=16 S=4096 D=128 N(0,1) data with cfk_set_option(CFK_OPT_PREDICTABLE_LATENCY, 1)",
    "cfg4_fast_weights": "fmha_fwd fp8-e4m3 B=4 H=16 S=4096 D=128 N(0,1) data with cfk_set_option(CFK_OPT_FAST_E4M3_WEIGHTS, 1): e4m3 weights "
                         "written as codes without an exponential (not the default: a fifth of them one e4m3 step off)",
    "d64_f8_fast_weights": "fmha_fwd fp8-e4m3 B=4 H=32 S=4096 D=64 with cfk_set_option(CFK_OPT_FAST_E4M3_WEIGHTS, 1)",
    "d64_f16": "fmha_fwd fp16 B=4 H=32 S=4096 D=64 non-causal (the reference sweep's problem at head size 64)",
    "d64_f8": "fmha_fwd fp8-e4m3 B=4 H=32 S=4096 D=64 non-causal, per-tensor amax scales, V [B,S,H,D]",
    "gemm_f32": "gemm fp32 M=N=K=8192 TN (fp32 MFMA: gfx950 has no tf32)",
}


def _time_launches(fn, steps, warmup):
    """Mean launch duration in ms: `warmup` untimed calls, then exactly `steps` back-to-back calls between two
    events recorded on the stream the kernels are launched on (torch's current stream)."""
    import torch
    # Untimed clock-settle burst: the GPU's clock governor needs sustained load for some tens of milliseconds
    # before it leaves its idle state; without it a short timed region measures the ramp, not the kernel.
    t_end = time.perf_counter() + 0.4
    while time.perf_counter() < t_end:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(stop) / steps, wall_ms / steps


def _make_fmha(pkg, w, seed=3080):
    import torch
    dev = torch.device("cuda:0")
    B, H, S, D = w["B"], w["H"], w["S"], w["D"]
    gens = [torch.Generator(device=dev).manual_seed(seed + i) for i in (1, 2, 3)]
    q, k, v = (torch.randn((B, S, H, D), generator=g, device=dev, dtype=torch.float32) for g in gens)
    if w.get("climb"):   # (tests/_util.py: climbing_keys with the e4m3 test's parameters)
        ramp = 1.0 + 3.0 * torch.arange(S, device=dev, dtype=torch.float32) / (S - 1)
        ramp[(3 * S) // 4 + 3] *= 8.0
        k = k * ramp[None, :, None, None]
    kw = dict(softmax_scale=w["scale"])
    if w["dtype"] == "f16":
        q, k, v = q.half(), k.half(), v.half()
    else:
        def quant(x):
            s = float(x.abs().max()) / 448.0
            return (x / s).clamp(-448, 448).to(torch.float8_e4m3fn), s
        (q, qs), (k, ks), (v, vs) = quant(q), quant(k), quant(v)
        kw.update(q_descale=qs, k_descale=ks, v_descale=vs)
    o = torch.empty((B, S, H, D), dtype=torch.float16, device=dev)
    flop = pkg.testbed.fmha_flops(B, H, S, S, D)
    # the parameter block is filled in once; a step is then one cfk_fmha_forward call, as in the reference's launch loop
    # (src/fmha-pipeline/fmha_forward.cu:578-592)
    return pkg.fmha_forward(q, k, v, o=o, prepare=True, **kw), flop, (q, k, v, o, kw)


def _make_gemm(pkg, w, seed=3080):
    import torch
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(seed)
    dt = torch.float16 if w["dtype"] == "f16" else torch.float32
    a = (torch.rand((w["M"], w["K"]), generator=g, device=dev) * 2 - 1).to(dt)
    b = (torch.rand((w["N"], w["K"]), generator=g, device=dev) * 2 - 1).to(dt)
    c = torch.empty((w["M"], w["N"]), dtype=dt, device=dev)
    return (lambda: pkg.gemm(a, b, out=c)), 2.0 * w["M"] * w["N"] * w["K"], (a, b, c)


def run_workload(pkg, name, steps, warmup):
    w = WORKLOADS[name]
    fn, flop, keep = (_make_fmha if w["kind"] == "fmha" else _make_gemm)(pkg, w)
    # configuration 1 is a 9-microsecond kernel: the reference's protocol (mean over back-to-back launches) needs
    # many more of them for a stable mean
    n = steps * 20 if name == "cfg1" else steps * 4 if name.startswith("b1_") else min(steps, w.get("max_steps", steps))
    if w.get("one_pass"):
        pkg.fmha.set_option(pkg.fmha.CFK_OPT_PREDICTABLE_LATENCY, 1)
    if w.get("fast_weights"):
        pkg.fmha.set_option(pkg.fmha.CFK_OPT_FAST_E4M3_WEIGHTS, 1)
    try:
        kernel = None
        if w["kind"] == "fmha":   # the instantiation the library launches for this call (cfk_fmha_forward_kernel)
            f = pkg.fmha
            kernel = f.fmha_forward_kernel(f.CFK_FP8_E4M3 if w["dtype"] == "f8" else f.CFK_FP16, w["B"], w["H"], w["S"], w["S"], w["D"])
        ms, wall_ms = _time_launches(fn, n, warmup)
    finally:
        if w.get("one_pass"):
            pkg.fmha.set_option(pkg.fmha.CFK_OPT_PREDICTABLE_LATENCY, 0)
        if w.get("fast_weights"):
            pkg.fmha.set_option(pkg.fmha.CFK_OPT_FAST_E4M3_WEIGHTS, 0)
    tflops = flop / (ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS[w["dtype"]]
    return dict(workload=NAMES[name], ms_per_step=ms, wall_ms_per_step=wall_ms, tflops=tflops, flop_per_step=flop,
                dtype=w["dtype"], frac_of_peak=tflops / peak, peak_tflops=peak, kernel=kernel), keep


def cpu_baseline(pkg, w, budget_s=12.0):
    """Time the CPU oracle (restatement of TestAttention::compute, include/utils/fmha_cutlass.hpp:154-317) on whole
    (batch, head) problems of the headline workload until ~budget_s of CPU work is done."""
    import numpy as np
    import oracle
    B, H, S, D = 1, 2, w["S"], w["D"]
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    q, k, v = (x.astype(np.float16).astype(np.float32) for x in (q, k, v))
    oracle.attention_f32(q, k, v, bh_pairs=[(0, 0)], row_start=0, row_step=64)  # warm-up (threads, pages)
    heads = 0
    t0 = time.perf_counter()
    while True:
        oracle.attention_f32(q, k, v, bh_pairs=[(0, heads % H)])
        heads += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s:
            break
    flop = 4.0 * heads * S * S * D
    return dict(value=flop / dt / 1e12, unit="TFLOP/s", cores=oracle.num_threads(), kind="port",
                sample=f"{heads} whole (batch, head) problems of S={S} D={D} (fp32 host reference attention, "
                       f"OpenMP), {dt:.1f} s of CPU time")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)   # the reference's FLOP runs use --iterations=1000
    ap.add_argument("--warmup", type=int, default=10)    # reference: 10 warm-up launches
    ap.add_argument("--workload", default="cfg2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-secondary", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one plain 256 MiB device copy (a kernel of known traffic, for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is single-GPU (one MI355X); --gpus must be 1. "
                 "(batch, head) problems are independent: shard them over GPUs without communication.")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import __graft_entry__ as entry
    pkg = entry.load_package()
    pkg.lib()  # fail loudly if the HIP library is missing

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    main_res, keep = run_workload(pkg, args.workload, args.steps, args.warmup)
    del keep
    torch.cuda.empty_cache()
    secondary = []
    if not args.no_secondary:
        for name in sorted(WORKLOADS):
            if name == args.workload:
                continue
            try:
                r, keep = run_workload(pkg, name, args.steps, args.warmup)
                del keep
                torch.cuda.empty_cache()
                secondary.append({k: r[k] for k in ("workload", "kernel", "ms_per_step", "tflops", "dtype", "frac_of_peak")})
            except pkg.CfkError as e:
                secondary.append({"workload": NAMES[name], "error": str(e)})
    w = WORKLOADS[args.workload]
    traffic, traffic_source = measured_traffic(args.workload)
    out = {
        "metric": "fmha_fwd_tflops",
        "value": main_res["tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w["dtype"],
        "data": "synthetic",
        "config": {"workload": main_res["workload"], "kernel": main_res["kernel"], "flop_per_step": main_res["flop_per_step"],
                   "layout": "[B,S,H,D]", "seeds": [3081, 3082, 3083],
                   "protocol": "reference protocol (warm-up launches, then the mean of back-to-back launches between two "
                               "events on the launch stream, src/fmha-pipeline/fmha_forward.cu:578-593) preceded by an "
                               "untimed 0.4 s burst of launches that lets the clock governor settle; not in the reference"},
        "roofline": {"bound": "mfma", "achieved": main_res["tflops"], "peak": main_res["peak_tflops"],
                     "unit": "TFLOP/s", "frac": main_res["frac_of_peak"],
                     "traffic": traffic, "traffic_source": traffic_source},
        "secondary": secondary,
    }
    if not args.no_cpu_baseline and w["kind"] == "fmha":
        out["cpu_baseline"] = cpu_baseline(pkg, w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
