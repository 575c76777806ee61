"""Every tile shape the library builds, forced through CFK_FMHA_TILE -- the run-time counterpart of the reference's
compile-time -DQBLKSIZE / -DKBLKSIZE sweep (src/fmha-pipeline/compile_run_all_config.sh:3-6) -- checked against the CPU
oracle.  The wish is read once per process, so each tile runs in a fresh interpreter (tests/tile_case.py)."""
import json
import os
import subprocess
import sys

import pytest

from _util import ERRPCT_FP16, ERRPCT_FP8, ROOT, TOL_FP16, TOL_FP8, pkg

# tile wish -> cases (mode:B,S,H,D) that have an instantiation of exactly that tile
CASES = {
    "128x64": ["f16:1,512,2,64", "f16:1,512,2,128", "f16climb:1,256,2,128,384", "f8:1,2048,2,64", "f8:1,2048,2,128", "f8:1,2048,1,256",
               "f8climb:1,256,2,64,4096", "f8climb:1,256,2,128,4096", "f8climb:1,128,1,256,4096", "f8:1,4096,1,64", "f8:1,4096,1,128", "f8:1,4096,1,256",
               "hyb:1,512,2,64", "hyb:1,512,2,128", "f16:1,256,2,256", "f16climb:1,256,1,256,192",
               # ... 3072 keys, where the pass without a row max per tile starts
               "f8:1,3072,2,64", "f8:1,3072,1,128", "f8:1,3072,1,256", "f8climb:1,256,2,64,3072", "f8climb:1,256,2,128,3072", "f8climb:1,128,1,256,3072",
               # ... a last query tile filled to a whole number of waves (32 rows each)
               "f16:2,160,2,64,192", "f16:2,288,3,128,192", "f16:2,160,2,256,128", "f16climb:2,160,2,128,384", "f8:2,160,2,64,2048",
               "f8:2,288,2,128,2048", "f8:2,96,1,256,2048", "f8climb:2,160,2,128,4096", "hyb:2,160,2,64,512", "hyb:2,96,2,128,512"],
    "256x64": ["f16:2,288,2,128,320", "f8:2,320,2,128,2048", "hyb:2,416,2,128,512",
               "f16:1,512,2,64", "f16:1,512,2,128", "f16:1,768,2,128", "f16:1,512,2,128,320", "f8:1,2048,2,128", "hyb:1,512,2,128",
               "f8climb:1,256,2,128,4096", "f8:1,4096,1,128"],
    "128x128": ["f16:2,224,2,64,256", "f8:2,160,2,64,2048", "hyb:2,160,2,64,512", "f16:1,512,2,64", "f16:1,512,2,128", "f16:1,384,2,128", "f8:1,2048,2,64", "f8:1,2048,2,128",
                "f8:1,2048,1,256", "hyb:1,512,2,64", "f8climb:1,256,2,64,4096", "f8climb:1,256,2,128,4096", "f8climb:1,128,1,256,4096", "f8:1,4096,1,64", "f8:1,4096,1,128"],
    "256x128": ["f8:1,3072,1,128", "f8climb:1,256,2,128,3072", "f16:2,416,2,128,384", "f8:2,1184,2,128,2048", "f16:1,512,2,64", "f16:1,512,2,128", "f16:1,768,2,128,384", "f8:1,2048,2,128", "hyb:1,512,2,128", "f8climb:1,256,2,128,4096", "f8:1,4096,1,128"],
    "128x32": ["f16:1,256,2,256", "hyb:1,256,2,256", "f16:2,96,2,256,256", "hyb:2,224,2,256,256"],
    # the fp16 builds on 16x16x32 MFMAs
    "128x64/16": ["f16:1,512,2,64", "f16:1,512,2,128", "f16:2,384,3,128,192", "f16:1,256,2,64,64", "f16climb:1,256,2,64,512",
                  "f16climb:1,384,2,128", "f16climb:1,128,1,128,64"],
    "256x64/16": ["f16:1,512,2,128", "f16:1,768,2,128", "f16:1,512,2,128,320", "f16:2,256,1,128,64", "f16climb:1,512,2,128,448"],
    "128x128/16": ["f16:1,512,2,128", "f16:2,384,3,128,128", "f16:1,256,2,128,640", "f16climb:1,384,2,128"],
    "256x128/16": ["f16:1,512,2,128", "f16:1,768,2,128,384", "f16:2,256,1,128,128", "f16climb:1,512,2,128,768"],
    # ... with the hand-scheduled main loop and persistent workgroups (key length at least 512): the
    # scheduled loop (no taps), its fall-back for scores that leave the fp16 range of the weights (climbing keys), the
    # max-tracking loop that serves the taps; 2x16 heads x 2048 rows = 256 items (one per workgroup), 3x16x2048 = 384
    # (half of the workgroups take a second item), 5x16x1024 = 320 with climbing keys (fall-back, then a next item)
    "256x128/16h": ["f16nt:1,512,2,128", "f16nt:1,256,3,128,768", "f16nt:2,2048,16,128", "f16nt:3,2048,16,128", "f16nt:1,512,2,128,1024",
                    "f16ntclimb:1,512,2,128,768", "f16ntclimb:5,1024,16,128", "f16:1,512,2,128", "f16:3,2048,16,128", "f16climb:1,512,2,128,768",
                    # ... its head-dim-64 shape (row sum on the matrix pipe)
                    "f16nt:1,512,2,64", "f16nt:1,256,3,64,768", "f16nt:3,2048,16,64", "f16ntclimb:1,512,2,64,768", "f16ntclimb:5,1024,16,64",
                    "f16:1,512,2,64", "f16climb:1,512,2,64,1024",
                    # ... key lengths with one to three tiles behind the last group of four (taken outside the generated loop)
                    "f16nt:1,512,2,128,576", "f16nt:2,2048,16,128,2240", "f16nt:1,256,3,128,640", "f16ntclimb:1,512,2,128,704",
                    "f16nt:1,512,2,64,640", "f16nt:3,2048,16,64,2112", "f16ntclimb:1,512,2,64,576", "f16ntclimb:1,512,2,64,640",
                    "f16ntclimb:1,512,2,128,576", "f16ntclimb:1,512,2,64,704",    # (the spike key inside the loop's tiles, and behind them)
                    # ... a last query tile filled to a whole number of waves: 2x16 heads x 2016 rows, 3x16x2016 (second items)
                    "f16nt:2,416,3,128,768", "f16nt:2,2016,16,128,2048", "f16nt:3,2016,16,64,2112", "f16ntclimb:2,288,2,128,768",
                    "f16ntclimb:2,352,2,64,640", "f16:2,416,2,128,768",
                    "f16ntclimb:2,352,2,64,2112", "f16nt:3,2016,16,128,2240", "f16ntclimb:2,288,2,128,2176"],   # (... with leftover key tiles as well)
    # ... and its head-dim-256 shape (4 waves, one per SIMD, 32-key tiles; key length a multiple of 128, at least 256):
    # 3x6 heads x 2048 rows = 288 items of 128 rows (32 workgroups take a second one), climbing keys, taps
    "128x64/16h": ["f16nt:1,256,2,256", "f16nt:1,128,3,256,640", "f16nt:3,2048,6,256,512", "f16ntclimb:1,256,2,256,512",
                   "f16ntclimb:3,1024,12,256,256", "f16:1,256,2,256,384", "f16climb:1,256,2,256,512",
                   "f16nt:2,160,2,256,512", "f16nt:3,2016,6,256,512", "f16ntclimb:2,224,3,256,512", "f16:2,96,2,256,384"],   # (partly filled last tile)
    # ... and the head-dim-128 loop for 128 query rows (4 waves, one per SIMD, O in accumulation registers): 1x20 heads x
    # 2048 rows = 320 items (64 workgroups take a second one), climbing keys, taps
    "128x128/16h": ["f16nt:1,256,2,128,512", "f16nt:1,128,3,128,768", "f16nt:1,2048,20,128", "f16nt:2,384,3,128,1024", "f16ntclimb:1,256,2,128,768",
                    "f16ntclimb:5,1024,8,128", "f16:1,256,2,128,512", "f16climb:1,256,2,128,768",
                    # ... and the head-dim-64 loop likewise
                    "f16nt:1,256,2,64,512", "f16nt:1,128,3,64,768", "f16nt:1,2048,20,64", "f16ntclimb:1,256,2,64,768", "f16ntclimb:5,1024,8,64",
                    "f16:1,256,2,64,512", "f16climb:1,256,2,64,1024",
                    "f16nt:1,256,2,128,1088", "f16nt:1,2048,20,128,1216", "f16nt:1,256,2,64,1216", "f16ntclimb:1,256,2,64,1088", "f16ntclimb:1,128,2,128,576",
                    "f16nt:2,160,3,128,1088", "f16nt:1,2016,20,64,1216", "f16ntclimb:2,224,2,128,768", "f16:2,96,2,64,512"],   # (partly filled last tile)
    # the e4m3 build with the hand-scheduled loop and persistent workgroups (by the automatic choice from 3072 keys): the
    # scheduled loop, 4352 keys (an odd number of loop turns), 2x10 heads x 4096 rows = 320 items (a quarter of the
    # workgroups take a second one), climbing keys (the vote, the max-tracking loop, then a next item: 5x13x1024 rows = 260)
    # 32 query rows per workgroup, the eight waves split the keys (the automatic choice for small grids): key lengths with
    # fewer tiles than waves, with tiles left over, query lengths that no other tile divides, taps, climbing keys
    "32x64": ["f16:1,512,8,64", "f16:1,512,2,128", "f16:2,96,3,64,64", "f16:1,160,2,128,192", "f16:1,128,2,64,1216", "f16nt:1,256,2,128,640",
              "f16climb:1,256,2,64,512", "f16climb:1,128,2,128,1024", "f16:3,2048,4,128,2048"],
    "256x128/32h": ["f8climb:2,288,2,128,3264", "f8:2,1184,3,128,3136",   # (leftover key tiles and a partly filled last query tile together)
                    "f8:1,512,2,128,4160", "f8:2,512,3,128,4288", "f8climb:1,256,2,128,4224", "f8:3,4096,10,128,3136",   # (one to three tiles behind the last group of four)
                    "f8:1,512,2,128,512", "f8:2,512,2,128,1280", "f8:1,512,2,128,3072", "f8climb:1,256,2,128,768",   # (key lengths below 3072:
                    "f8:2,1184,2,128,4096", "f8:2,4064,10,128,4096", "f8climb:2,288,2,128,4096",   # (partly filled last query tile)
                    "f8:1,256,2,128,4096", "f8:1,512,1,128,4352", "f8:2,4096,10,128", "f8climb:1,256,2,128,4096", "f8climb:5,1024,13,128,4096"],
    # ... and its 4-wave shape (128 query rows, two copies per wave and tile): 1x9 heads x 4096 rows = 288 items
    "128x128/32h": ["f8climb:2,224,2,128,3264", "f8:2,1184,3,128,3136",   # (likewise)
                    "f8:1,256,2,128,4160", "f8:2,384,3,128,3264", "f8climb:1,128,2,128,4288", "f8:1,4096,9,128,3136",     # (likewise)
                    "f8:1,256,2,128,512", "f8:1,384,3,128,3072", "f8climb:1,128,2,128,1024",   #  by wish only)
                    "f8:2,1184,2,128,4096", "f8:1,4064,9,128,4096", "f8climb:2,224,2,128,4096",    # (partly filled last query tile)
                    "f8:1,128,2,128,4096", "f8:1,256,1,128,4352", "f8:1,4096,9,128", "f8climb:1,128,2,128,4096", "f8climb:5,512,13,128,4096"],
}


def test_tile_wish_is_honoured_by_the_plan_without_gpu():
    # the plan query needs no GPU; a wish no instantiation serves is ignored
    f = pkg.fmha
    code = ("import sys; sys.path.insert(0, %r); import __graft_entry__ as e; p = e.load_package(); f = p.fmha; "
            "print(f.fmha_forward_plan(f.CFK_FP16, 2, 4, 1536, 512, 128)[:2], f.fmha_forward_plan(f.CFK_FP16, 2, 4, 1536, 512, 256)[:2], "
            "f.fmha_forward_plan(f.CFK_FP8_E4M3, 2, 4, 1536, 512, 128)[:2], f.fmha_forward_plan(f.CFK_FP16, 2, 16, 384, 384, 128)[:2], "
            "f.fmha_forward_plan(f.CFK_FP16, 2, 4, 512, 512, 128)[:2])" % ROOT)
    def plans(wish):
        env = dict(os.environ)
        env.pop("CFK_FMHA_TILE", None)
        if wish:
            env["CFK_FMHA_TILE"] = wish
        return subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, check=True).stdout.strip()
    # medium problems: 128-row tiles; small ones (the last: 128 workgroups of 32 rows fit on the chip at once): fp16 at head
    # dims 64 and 128 takes 32-row workgroups whose waves split the keys
    assert plans(None) == "(128, 64) (128, 32) (128, 64) (128, 64) (32, 64)"
    # no such tile at head dim 256; 384 query rows: the second 256-row tile is half filled (whole waves of 32 rows)
    assert plans("256x128") == "(256, 128) (128, 32) (256, 128) (256, 128) (256, 128)"
    assert plans("large") == "(256, 64) (128, 32) (256, 64) (256, 64) (256, 64)"
    assert plans("128x128") == "(128, 128) (128, 32) (128, 128) (128, 128) (128, 128)"
    assert plans("32x64") == "(32, 64) (128, 32) (128, 64) (32, 64) (32, 64)"              # fp16 at head dims 64 / 128 only
    # the MFMA shape suffix: served for fp16 at head dims 64/128 only (e4m3 and head dim 256 ignore the wish)
    mfma_code = ("import sys; sys.path.insert(0, %r); import __graft_entry__ as e; p = e.load_package(); f = p.fmha; "
                 "print(f.fmha_forward_mfma(f.CFK_FP16, 2, 4, 1536, 512, 128), f.fmha_forward_mfma(f.CFK_FP16, 2, 4, 1536, 512, 64), "
                 "f.fmha_forward_mfma(f.CFK_FP16, 2, 4, 1536, 512, 256), f.fmha_forward_mfma(f.CFK_FP8_E4M3, 2, 4, 1536, 512, 128), "
                 "f.fmha_forward_plan(f.CFK_FP16, 2, 4, 1536, 512, 128)[:2])" % ROOT)
    def shapes(wish):
        env = dict(os.environ, CFK_FMHA_TILE=wish)
        return subprocess.run([sys.executable, "-c", mfma_code], env=env, capture_output=True, text=True, check=True).stdout.strip()
    assert shapes("128x64/16") == "16 16 32 32 (128, 64)"
    assert shapes("256x64/16") == "16 32 32 32 (256, 64)"      # no 256-row 16x16x32 build at head dim 64
    assert shapes("256x64/32") == "32 32 32 32 (256, 64)"
    assert shapes("128x64") == "32 32 32 32 (128, 64)"
    assert shapes("256x128") == "32 32 32 32 (256, 128)"
    assert shapes("256x128/16") == "16 32 32 32 (256, 128)"   # two key tiles per barrier on 16x16x32: head dim 128 only
    assert shapes("256x128/16h") == "16 16 32 32 (256, 128)"  # ... with the hand-scheduled loop: head dims 128 and 64
    # the hand-scheduled build needs 160 KB of LDS; a wish for the compiler-scheduled one (no `h`) is kept apart from it
    lds_code = ("import sys; sys.path.insert(0, %r); import __graft_entry__ as e; p = e.load_package(); f = p.fmha; "
                "print(f.fmha_forward_plan(f.CFK_FP16, 2, 4, 1536, 512, 128)[2], f.fmha_forward_plan(f.CFK_FP16, 2, 4, 1536, 384, 128)[:3])" % ROOT)
    def lds(wish):
        env = dict(os.environ, CFK_FMHA_TILE=wish)
        return subprocess.run([sys.executable, "-c", lds_code], env=env, capture_output=True, text=True, check=True).stdout.strip()
    assert lds("256x128/16h") == "163840 (128, 64, 65536)"    # key length 384: fewer than eight tiles, the wish is ignored
    assert lds("256x128/16") == "131072 (256, 128, 131072)"
    assert f.fmha_forward_plan(f.CFK_FP16, 8, 16, 2048, 2048, 128)[:2] == (256, 128)  # big problem: automatic choice
    assert f.fmha_forward_plan(f.CFK_FP16, 8, 16, 2048, 2112, 128)[:2] == (256, 128)  # ... also with a tile left over behind the last four
    assert f.fmha_forward_kernel(f.CFK_FP16, 8, 16, 2048, 2112, 128) == "fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>"
    # (... from 2048 keys on and while the tiles left over are few: 31 tiles, three of them left over, stay compiler-scheduled)
    assert "kernel16p<" not in f.fmha_forward_kernel(f.CFK_FP16, 8, 16, 2048, 1984, 128)
    # ... on 16x16x32 MFMAs for fp16; problems with fewer work items than half the CUs (head dims 64, 128) and e4m3 stay on 32x32
    assert f.fmha_forward_mfma(f.CFK_FP16, 8, 16, 2048, 2048, 128) == 16
    assert f.fmha_forward_mfma(f.CFK_FP16, 4, 32, 4096, 4096, 64) == 16
    assert f.fmha_forward_plan(f.CFK_FP16, 4, 32, 4096, 4096, 64)[:2] == (256, 128)      # hand-scheduled
    assert f.fmha_forward_kernel(f.CFK_FP16, 4, 32, 4096, 4096, 64) == "fmha_fwd_kernel16p<64,64,8,2,0,0,0,0,2,0,1,1>"
    assert f.fmha_forward_plan(f.CFK_FP16, 4, 32, 4096, 4032, 64)[:2] == (256, 128)      # ... also with tiles left over
    assert f.fmha_forward_mfma(f.CFK_FP16, 2, 4, 1536, 512, 128) == 32
    assert f.fmha_forward_kernel(f.CFK_FP16, 1, 8, 512, 512, 64) == "fmha_fwd_kernel_ks<64,8>"      # benchmark configuration 1
    assert f.fmha_forward_kernel(f.CFK_FP16, 2, 4, 512, 512, 128) == "fmha_fwd_kernel_ks<128,8>"
    assert f.fmha_forward_plan(f.CFK_FP16, 1, 2, 96, 192, 64)[:2] == (32, 64)                       # query rows a multiple of 32
    assert f.fmha_forward_mfma(f.CFK_FP16, 2, 8, 8192, 8192, 256) == 16                             # hand-scheduled, 16x16x32
    assert f.fmha_forward_kernel(f.CFK_FP16, 2, 8, 8192, 8192, 256) == "fmha_fwd_kernel16p<256,32,4,1,0,0,0,0,2,0,1,1>"
    assert f.fmha_forward_kernel(f.CFK_FP16, 2, 8, 8192, 8160, 256) == "fmha_fwd_kernel<256,32,4,1,0,0,0,0,1,0,0,0>"   # key length % 128 != 0
    assert f.fmha_forward_mfma(f.CFK_FP16, 2, 4, 1536, 1024, 256) == 16                             # ... from 1024 keys on
    assert f.fmha_forward_mfma(f.CFK_FP16, 2, 4, 1536, 512, 256) == 32                              # below: 32x32
    assert f.fmha_forward_mfma(f.CFK_FP8_E4M3, 4, 16, 4096, 4096, 128) == 32
    assert f.fmha_forward_plan(f.CFK_FP8_E4M3, 4, 16, 4096, 4096, 128)[:2] == (256, 128)


@pytest.mark.gpu
@pytest.mark.parametrize("wish", sorted(CASES))
def test_forced_tiles_match_the_oracle(wish):
    env = dict(os.environ, CFK_FMHA_TILE=wish, PYTHONPATH=os.path.join(ROOT, "tests") + os.pathsep + ROOT)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "tile_case.py"), *CASES[wish]], env=env,
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr
    rows = [json.loads(l.split(" ", 1)[1]) for l in r.stdout.splitlines() if l.startswith("TILECASE ")]
    assert len(rows) == len(CASES[wish])
    shape, _, mfma = wish.partition("/")
    mfma = mfma.rstrip("h")
    bm, bn = (int(x) for x in shape.split("x"))
    for row in rows:
        print(row)
        assert (row["block_m"], row["block_n"]) == (bm, bn), row     # the wished tile really ran
        if row["case"].startswith("f16"):
            assert row["mfma"] == (16 if bm == 32 else int(mfma or 32)), row   # ... on the wished MFMA shape (the 32-row build: 16x16x32)
            # row-max tap (relative to the largest row max): exact fp32 products, so only summation order separates
            # it from the oracle; row-sum tap (relative): the kernel adds the weights as rounded to fp16 (2^-11 each,
            # unbiased), the oracle the fp32 values
            # (with climbing keys one or two weights carry a row's sum: no averaging, up to 2^-11 = 4.9e-4)
            if row["taps"] is not None:
                assert row["taps"][0] <= 2e-5 and row["taps"][1] <= (5e-4 if "climb" in row["case"] else 3e-4), row
        fp8 = row["case"].startswith("f8")
        assert not row["nan"] and row["max_abs"] <= (TOL_FP8 if fp8 else TOL_FP16), row
        # (e4m3 P with climbing keys: a handful of keys carry each row, so the 6 % rounding of a weight does not average out
        # and the percentage criterion, calibrated on N(0,1) scores, does not apply; max-abs does)
        # (... nor over fewer than 2048 keys, where the rounding of a row's few large weights shows in every e4m3 kernel)
        dims = [int(x) for x in row["case"].split(":")[1].split(",")]
        if not (fp8 and ("climb" in row["case"] or dims[-1 if len(dims) > 4 else 1] < 2048)):
            assert row["err_pct"] <= (ERRPCT_FP8 if fp8 else ERRPCT_FP16), row
