"""The C++ bench/test driver (cutlass-kernels_amd/driver/fmha_forward): command line of the reference driver
(src/fmha-pipeline/fmha_forward.cu:687-794), its check lines, and an independent check of what it dumps."""
import os
import subprocess

import numpy as np
import pytest

import oracle
from _util import ERRPCT_FP16, ERRPCT_FP8, ROOT, TOL_FP16, TOL_FP8, max_abs

DRIVER = os.path.join(ROOT, "cutlass-kernels_amd", "driver", "fmha_forward")


def _run(*args, check=True):
    r = subprocess.run([DRIVER, *args], capture_output=True, text=True, timeout=600)
    if check:
        assert r.returncode == 0, r.stdout + r.stderr
    return r


def test_driver_is_built():
    assert os.path.exists(DRIVER), "build it: python -c 'import __graft_entry__ as g; g.build()'"


def test_usage_and_flag_errors_without_gpu():
    out = _run("--help").stdout
    for flag in ("--prec-type", "--batch-size", "--dim-size", "--head-size", "--seq-length", "--iterations",
                 "--num-cuda-streams", "--reference-check", "--print-values"):
        assert flag in out
    r = _run("--head-size=96", check=False)
    assert r.returncode != 0 and "Unsupported head dim: 96" in r.stdout
    r = _run("--prec-type=3", check=False)
    assert r.returncode != 0 and "Unsupported type: 3" in r.stdout
    r = _run("--batch-size=2", "--num-cuda-streams=4", check=False)
    assert r.returncode != 0 and "max no. of cuda streams" in r.stdout


def test_driver_e4m3_encoder_matches_codec():
    lines = _run("--selftest-e4m3").stdout.split()
    bits = np.array([int(x, 16) for x in lines[0::2]], dtype=np.uint32)
    codes = np.array([int(x, 16) for x in lines[1::2]], dtype=np.uint8)
    assert bits.size == 4096
    assert np.array_equal(codes, oracle.e4m3_encode(bits.view(np.float32)))


def _load_dump(d):
    meta = dict(l.split() for l in open(os.path.join(d, "meta.txt")).read().strip().splitlines())
    B, S, H, D, prec = (int(meta[k]) for k in ("B", "S", "H", "D", "prec"))
    shape = (B, S, H, D)
    if prec == 1:
        q, k, v = (np.fromfile(os.path.join(d, f + ".bin"), dtype=np.float16).reshape(shape).astype(np.float32)
                   for f in "qkv")
    else:
        q, k = (oracle.e4m3_decode(np.fromfile(os.path.join(d, f + ".bin"), dtype=np.uint8).reshape(shape)) *
                np.float32(meta[f + "_descale"]) for f in "qk")
        if int(meta["v_fp8"]):
            v = oracle.e4m3_decode(np.fromfile(os.path.join(d, "v.bin"), dtype=np.uint8).reshape(shape)) * \
                np.float32(meta["v_descale"])
        else:
            v = np.fromfile(os.path.join(d, "v.bin"), dtype=np.float16).reshape(shape).astype(np.float32)
    o = np.fromfile(os.path.join(d, "o.bin"), dtype=np.float16).reshape(shape).astype(np.float32)
    return q, k, v, o, prec


@pytest.mark.gpu
@pytest.mark.parametrize("prec,head,extra", [(1, 64, []), (1, 128, ["--num-cuda-streams=2"]), (1, 256, []),
                                             (2, 128, []), (2, 128, ["--fp8-scales=amax"]), (2, 64, []), (2, 256, []), (2, 128, ["--gemm2-fp8=false"]),
                                             (2, 128, ["--v-layout=bdhs"]), (2, 64, ["--v-layout=bdhs", "--fp8-scales=amax"]),
                                             # sequence lengths that leave the last 128-row query tile partly filled
                                             (1, 128, ["seq=1088"]), (1, 256, ["seq=608"]), (2, 128, ["seq=4160"])])
def test_driver_reference_check_and_dump(tmp_path, prec, head, extra):
    # fp8 needs the reference's own sequence length for its percentage criterion; fp16 passes at any length
    seq = 4096 if prec == 2 else 512   # (e4m3 P: the two-pass path starts at 3072 keys)
    seq = next((int(e[4:]) for e in extra if e.startswith("seq=")), seq)
    extra = [e for e in extra if not e.startswith("seq=")]
    out = _run(f"--prec-type={prec}", "--batch-size=2", f"--dim-size={2 * head}", f"--head-size={head}",
               f"--seq-length={seq}", "--iterations=3", "--reference-check=true", "--verify-all=true",
               f"--dump-dir={tmp_path}", *extra).stdout
    assert "CUTE_FMHA:" in out and "Gflop/s" in out
    assert "gemm-check-2: Passed" in out and "max-check: Passed" in out and "sum-check: Passed" in out
    assert "gemm-check-1: Passed" in out
    assert f"K = {head}" in out and "QBLK = " in out
    # independent check of the dumped tensors against the CPU oracle
    q, k, v, o, p = _load_dump(str(tmp_path))
    ref = oracle.attention_f32(q, k, v)["O"]
    assert max_abs(o, ref) <= (TOL_FP16 if p == 1 else TOL_FP8)
    assert oracle.verify_tensor(o, ref, ERRPCT_FP16 if p == 1 else ERRPCT_FP8)[0]


def test_driver_rejects_bdhs_for_fp16_v():
    r = _run("--prec-type=1", "--v-layout=bdhs", check=False)
    assert r.returncode != 0 and "bdhs" in r.stdout
    r = _run("--prec-type=2", "--v-layout=hdbs", check=False)
    assert r.returncode != 0 and "Unsupported V layout" in r.stdout


@pytest.mark.gpu
def test_sweep_script_verify_all_on_a_reduced_problem():
    # run_all_config.sh (the counterpart of compile_run_all_config.sh) in its verify-all mode: every precision mode x
    # head size x tile shape that exists, each with gemm-check-1 / max-check / sum-check / gemm-check-2
    script = os.path.join(ROOT, "cutlass-kernels_amd", "driver", "run_all_config.sh")
    # (the reference's own sequence length, 4096: its error-percentage gate is calibrated there, and the e4m3 kernel walks
    # the keys in two passes from that length on -- the path its FLOP runs time)
    env = dict(os.environ, BATCH="1", SEQ="4096", DIM="512")
    r = subprocess.run(["bash", script, "verify-all"], env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-4000:] + r.stderr[-2000:]
    blocks = r.stdout.split("CONFIG ")[1:]
    assert len(blocks) == 38, len(blocks)
    seen = set()
    for blk in blocks:
        head_line = blk.splitlines()[0]
        mode, head, tile = (x.split("=")[1] for x in head_line.replace(",", "").split())
        shape, _, mfma = tile.partition("/")          # <query rows>x<keys>[/16|/16h|/32h]: MFMA shape, hand-scheduled loop
        bm, bn = shape.split("x")
        hand = mfma.endswith("h")
        mfma = mfma.rstrip("h") or ("16" if bm == "32" else "32")            # (the 32-row build runs on 16x16x32 MFMAs)
        assert f"QBLK = {bm}" in blk and f"KBLK = {bn}" in blk, blk          # the wished tile is the one that ran
        assert f"MFMA = {mfma}x{mfma}" in blk, blk
        assert ("kernel16p<" in blk or "kernel8p<" in blk) == hand, blk      # ... and the wished kind of kernel
        for line in ("gemm-check-1: Passed", "max-check: Passed", "sum-check: Passed", "gemm-check-2: Passed"):
            assert line in blk, (head_line, blk)
        assert "Failed" not in blk
        seen.add((mode, head, tile))
    assert len(seen) == 38
    assert {m for m, _, _ in seen} == {"fp16", "fp8", "fp8-bdhs", "hybrid"}


GEMM_DRIVER = os.path.join(ROOT, "cutlass-kernels_amd", "driver", "gemm")


def test_gemm_driver_rejects_other_types():
    # type 2 (tf32) is commented out in the reference as well (src/cute-gemm-tma-gma/gemm.cu:679-681)
    r = subprocess.run([GEMM_DRIVER, "2"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "invalid type value" in r.stdout
    r = subprocess.run([GEMM_DRIVER, "--help"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and "--alpha" in r.stdout


@pytest.mark.gpu
def test_gemm_driver_runs_and_checks():
    r = subprocess.run([GEMM_DRIVER, "3", "1024", "768", "512", "2", "check"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "CUTE_GEMM:" in r.stdout and "GFlop/s" in r.stdout and "L = 2" in r.stdout
    assert r.stdout.count("Passed") == 2 and "Failed" not in r.stdout


@pytest.mark.gpu
def test_gemm_driver_float_type():
    # type 1 of the CuTe example: float operands (gemm.cu:677-678)
    r = subprocess.run([GEMM_DRIVER, "1", "512", "256", "256", "1", "check"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "CUTE_GEMM:" in r.stdout and r.stdout.count("Passed") == 2 and "Failed" not in r.stdout


@pytest.mark.gpu
def test_gemm_driver_cutlass_example_options():
    # the CUTLASS-API example's command line and report (src/cutlass-gemm/gemm.cu:198-236, 390-413)
    r = subprocess.run([GEMM_DRIVER, "--m=1024", "--n=512", "--k=1024", "--alpha=2", "--beta=0.5", "--iterations=5"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "Disposition: Passed" in r.stdout and "Problem Size: 1024x512x1024" in r.stdout
    assert "Avg runtime:" in r.stdout and "GFLOPS:" in r.stdout
