#!/usr/bin/env python3
"""Register / scratch / LDS usage of every kernel of the library, read from the compiler
(hipcc -Rpass-analysis=kernel-resource-usage, the flags of the Makefile; no GPU needed).

    python3 resource_usage.py            # markdown table on stdout (the committed copy: profiles/kernel_resource_usage.md)

tests/test_resource_usage.py runs the same and holds the kernels the automatic choice can pick to their allowances:
a spill that creeps into a main loop shows there, in the container, before it shows as WRITE_SIZE on the GPU.
"""
import concurrent.futures
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["fmha_fwd_f16.hip", "fmha_fwd_f16_d256.hip", "fmha_fwd_fp8.hip", "fmha_fwd_hybrid.hip", "gemm.hip"]
FLAGS = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-fno-gpu-rdc", "--offload-device-only", "-Rpass-analysis=kernel-resource-usage",
         "-c", "-o", "/dev/null"]
EXTRA = {"fmha_fwd_f16_d256.hip": ["-mllvm", "-amdgpu-sched-strategy=iterative-ilp"]}   # as in the Makefile
FIELDS = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch", "VGPRs Spill": "vgpr_spill",
          "SGPRs Spill": "sgpr_spill", "Occupancy [waves/SIMD]": "occupancy", "LDS Size [bytes/block]": "lds_static"}


def demangle(names):
    out = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True, check=True).stdout
    return out.splitlines()


def short_name(d):
    """cfk::fmha_fwd_kernel16<cfk::FmhaCfg<128, 64, 8, 2, false, ...>>(cfk::FmhaArgs) -> fmha_fwd_kernel16<128,64,8,2,0,0,0,0,2,0,1>"""
    m = re.match(r"_ZN3cfk12_GLOBAL__N_1\d+([a-z_0-9]+?)I(.*?)EEv", d)   # (the system's c++filt does not know _Float16 parameters)
    if m: return m.group(1) + "<" + m.group(2).replace("Lb0E", "0,").replace("Lb1E", "1,").replace("Li4E", "4").rstrip(",") + ">"
    d = re.sub(r"^void ", "", d).replace("(anonymous namespace)::", "")
    d = re.sub(r"\(.*\)$", "", d)
    direct = "DirectCfg<" in d     # the build with e4m3 weights written as codes: shown as <...>/direct
    d = d.replace("cfk::", "").replace("DirectCfg<", "").replace("FmhaCfg<", "").replace("KsCfg<", "").replace(">>", ">").replace(">>", ">")
    d = d.replace("false", "0").replace("true", "1").replace(" ", "")
    return re.sub(r">+$", ">", d) + ("/direct" if direct else "")


def compile_one(src):
    cmd = ["/opt/rocm/bin/hipcc"] + FLAGS + EXTRA.get(src, []) + [src]
    r = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(src + ":\n" + r.stderr[-3000:])
    kernels, cur = [], None
    for line in r.stderr.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            cur = {"source": src, "mangled": m.group(1)}
            kernels.append(cur)
            continue
        m = re.search(r"remark: (?:\S+: )? *([A-Za-z]+(?: [A-Za-z]+)*(?: \[[^\]]+\])?): +(\d+) \[-Rpass", line)
        if m and cur is not None and m.group(1) in FIELDS:
            cur[FIELDS[m.group(1)]] = int(m.group(2))
    return kernels


def collect():
    with concurrent.futures.ThreadPoolExecutor(max_workers=5) as ex:
        lists = list(ex.map(compile_one, SOURCES))
    kernels = [k for l in lists for k in l]
    for k, d in zip(kernels, demangle([k["mangled"] for k in kernels])):
        k["name"] = short_name(d)
    return kernels


def table(kernels):
    rows = ["| kernel (FmhaCfg: head dim, keys/tile, waves, waves/SIMD, e4m3 QK, e4m3 PV, V^T, score tap, tiles/barrier, K prefetch, 16x16x32, hand loop) | source | VGPRs | AGPRs | spilled VGPRs | scratch B/lane | waves/SIMD |",
            "|---|---|---|---|---|---|---|"]
    for k in sorted(kernels, key=lambda k: (k["source"], k["name"])):
        rows.append("| `%s` | %s | %d | %d | %d | %d | %d |" % (k["name"], k["source"], k["vgprs"], k["agprs"], k["vgpr_spill"], k["scratch"], k["occupancy"]))
    return "\n".join(rows)


if __name__ == "__main__":
    print(table(collect()))
