"""Compile-time register gate: every kernel of the library is compiled with -Rpass-analysis=kernel-resource-usage
(cutlass-kernels_amd/csrc/resource_usage.py: the Makefile's flags, no GPU) and held to an allowance of spilled
registers.  A spill that creeps into a main loop costs tens of per cent and is otherwise only found on the GPU, as
extra bytes in WRITE_SIZE.  The kernels the automatic choice can pick are listed by name; the table of all kernels is
committed as profiles/kernel_resource_usage.md."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# name -> (spilled VGPRs allowed, why).  FmhaCfg arguments: head dim, keys per tile, waves, waves per SIMD, e4m3 Q/K, e4m3
# P/V, V pre-transposed, score tap, tiles per barrier, K fragment prefetch, 16x16x32 build, hand-scheduled loop.
AUTO_PICKED = {
    # fp16, head dim 128, big problems: the hand-scheduled persistent build.  Its main loop is hand-allocated (no spills
    # possible); the allowance is one 64-bit address that the max-tracking fall-back keeps, stored and reloaded once per item
    "fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>": (2, "outside the loop"),
    # ... its one-pass alternatives (key length not a multiple of 256, cfk_set_option(CFK_OPT_PREDICTABLE_LATENCY)): the
    # spills sit in the code of the last key tiles, behind the loop (seen as one dword per lane in WRITE_SIZE)
    "fmha_fwd_kernel16<128,64,8,2,0,0,0,0,2,0,1,0>": (112, "behind the loop"),
    "fmha_fwd_kernel16<128,64,8,2,0,0,0,0,1,0,1,0>": (19, "behind the loop"),
    "fmha_fwd_kernel<128,64,8,2,0,0,0,0,1,4,0,0>": (0, ""),
    "fmha_fwd_kernel<128,64,8,2,0,0,0,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<128,64,4,2,0,0,0,0,1,0,0,0>": (0, ""),
    # fp16, small grids (the waves split the keys)
    "fmha_fwd_kernel_ks<64,8>": (0, ""),
    "fmha_fwd_kernel_ks<128,8>": (0, ""),
    # ... and its 4-wave shapes (128 query rows, one wave per SIMD) for up to 256 items of 128 rows
    "fmha_fwd_kernel16p<128,64,4,1,0,0,0,0,2,0,1,1>": (0, ""),
    "fmha_fwd_kernel16p<64,64,4,1,0,0,0,0,2,0,1,1>": (0, ""),
    # fp16 head dim 64: big problems run the hand-scheduled persistent build
    "fmha_fwd_kernel16p<64,64,8,2,0,0,0,0,2,0,1,1>": (0, ""),
    "fmha_fwd_kernel16<64,64,4,3,0,0,0,0,1,0,1,0>": (14, "the slow path of the row-sum test"),
    "fmha_fwd_kernel<64,64,4,3,0,0,0,0,1,0,0,0>": (0, ""),
    # fp16 head dim 256: big problems run the hand-scheduled persistent build (one wave per SIMD, O in accumulation registers)
    "fmha_fwd_kernel16p<256,32,4,1,0,0,0,0,2,0,1,1>": (0, ""),
    "fmha_fwd_kernel<256,32,4,1,0,0,0,0,1,4,0,0>": (0, ""),
    "fmha_fwd_kernel<256,32,4,1,0,0,0,0,1,0,0,0>": (0, ""),
    # e4m3: big problems at head dim 128 from 4096 keys run the hand-scheduled persistent build
    "fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>": (0, ""),
    "fmha_fwd_kernel8p<128,64,4,2,1,1,0,0,2,0,0,1>": (0, ""),   # (its 4-wave shape, up to 256 items of 128 rows)
    "fmha_fwd_kernel<64,64,4,3,1,1,0,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<128,64,8,2,1,1,0,0,2,0,0,0>": (12, "between the two passes"),
    "fmha_fwd_kernel<128,64,4,2,1,1,0,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<256,64,4,1,1,1,0,0,2,0,0,0>": (5, "between the two passes"),
    "fmha_fwd_kernel<256,64,4,1,1,1,0,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<64,64,4,2,1,1,1,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<128,64,4,2,1,1,1,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<256,64,4,1,1,1,1,0,1,0,0,0>": (0, ""),
    # hybrid
    "fmha_fwd_kernel<64,64,4,3,1,0,0,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<128,64,8,2,1,0,0,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<128,64,4,2,1,0,0,0,1,0,0,0>": (0, ""),
    "fmha_fwd_kernel<256,32,4,1,1,0,0,0,1,0,0,0>": (0, ""),
    # GEMM
    "gemm_kernel16<0,4>": (0, ""),
    "gemm_kernel16<1,4>": (0, ""),
    "gemm_kernel_f32<128>": (0, ""),
}


def _ru():
    spec = importlib.util.spec_from_file_location("resource_usage", os.path.join(ROOT, "cutlass-kernels_amd", "csrc", "resource_usage.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


@pytest.fixture(scope="module")
def kernels():
    return {k["name"]: k for k in _ru().collect()}


def test_auto_picked_kernels_stay_within_their_spill_allowance(kernels):
    for name, (allowed, _) in AUTO_PICKED.items():
        assert name in kernels, (name, sorted(kernels))
        k = kernels[name]
        assert k["vgpr_spill"] <= allowed, (name, k)
        # (a spilled scalar register is a lane of a vector register, not memory: a few of them in the 4-wave hand-scheduled
        # builds, whose item set-up juggles twice the copy addresses, and in the e4m3 hand-scheduled build, which keeps two
        # work items' pointers across its loop for the tiles behind it; none anywhere else)
        juggles = name.startswith(("fmha_fwd_kernel8p<", "fmha_fwd_kernel16p<128,64,4,", "fmha_fwd_kernel16p<64,64,4,"))
        assert k["sgpr_spill"] <= (4 if juggles else 0), (name, k)
    # the headline kernel: two waves per SIMD within the 256 registers of the unified file
    k = kernels["fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>"]
    assert k["occupancy"] == 2 and k["vgprs"] + k["agprs"] <= 256 and k["scratch"] <= 16
    k = kernels["fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>"]
    assert k["occupancy"] == 2 and k["vgprs"] + k["agprs"] <= 256 and k["scratch"] == 0


def test_no_kernel_spills_more_than_the_table_says(kernels):
    # every kernel, picked automatically or only through CFK_FMHA_TILE: the committed table is the ceiling
    table = open(os.path.join(ROOT, "profiles", "kernel_resource_usage.md")).read()
    listed = {}
    for line in table.splitlines():
        cells = [c.strip() for c in line.split("|")]
        if len(cells) > 6 and cells[1].startswith("`"):
            listed[cells[1].strip("`")] = int(cells[5])
    assert set(listed) == set(kernels), set(listed) ^ set(kernels)
    for name, k in kernels.items():
        assert k["vgpr_spill"] <= listed[name], (name, k["vgpr_spill"], listed[name])
