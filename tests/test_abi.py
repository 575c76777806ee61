"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares, validates
arguments the way the reference driver's error paths do, and the plan query works without a GPU."""
import ctypes
import os
import re

import pytest

from _util import ROOT, pkg


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "cfk_fmha.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cfk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert {"cfk_fmha_forward", "cfk_fmha_forward_plan", "cfk_gemm", "cfk_gemm_f16", "cfk_init", "cfk_last_error",
            "cfk_version"} <= set(names)
    lib = ctypes.CDLL(pkg.lib_path())
    for n in names:
        assert getattr(lib, n) is not None, n


def test_params_struct_matches_header_layout():
    # 8 int32, 4 pointers, 4 floats, 3 pointers on LP64
    assert ctypes.sizeof(pkg.fmha.FmhaFwdParams) == 8 * 4 + 4 * 8 + 4 * 4 + 3 * 8
    assert pkg.fmha.FmhaFwdParams.q.offset == 32 and pkg.fmha.FmhaFwdParams.softmax_scale.offset == 64
    assert pkg.fmha.FmhaFwdParams.dbg_s.offset == 80 and pkg.fmha.FmhaFwdParams.dbg_row_max.offset == 88


def test_version_and_plan_without_gpu():
    assert "gfx950" in pkg.version()
    bm, bn, lds, threads = pkg.fmha_forward_plan(pkg.CFK_FP16, 8, 16, 2048, 2048, 128)
    assert 2048 % bm == 0 and 2048 % bn == 0 and 0 < lds <= 160 * 1024 and threads % 64 == 0
    for d in (64, 128, 256):
        pkg.fmha_forward_plan(pkg.CFK_FP16, 1, 1, 512, 512, d)
        pkg.fmha_forward_plan(pkg.CFK_FP8_E4M3, 1, 1, 512, 512, d)


def test_error_paths_mirror_reference_driver():
    # unsupported head dim (fmha_forward.cu:758-760) and precision (:788-790) -> error codes, never exit()
    with pytest.raises(pkg.CfkError) as e:
        pkg.fmha_forward_plan(pkg.CFK_FP16, 1, 1, 512, 512, 96)
    assert e.value.code == -2 and "Unsupported head dim: 96" in str(e.value)
    with pytest.raises(pkg.CfkError) as e:
        pkg.fmha_forward_plan(3, 1, 1, 512, 512, 64)
    assert e.value.code == -1 and "Unsupported type: 3" in str(e.value)
    with pytest.raises(pkg.CfkError) as e:
        pkg.fmha_forward_plan(pkg.CFK_FP16, 1, 1, 500, 512, 64)  # no masks: tiles must divide S
    assert e.value.code == -2
    with pytest.raises(pkg.CfkError) as e:
        pkg.fmha_forward_plan(pkg.CFK_FP16, 0, 1, 512, 512, 64)
    assert e.value.code == -1
    pkg.fmha_forward_plan(pkg.CFK_FP8_E4M3, 1, 1, 512, 512, 64, v_dtype=pkg.CFK_FP16)      # hybrid mode
    with pytest.raises(pkg.CfkError):
        pkg.fmha_forward_plan(pkg.CFK_FP16, 1, 1, 512, 512, 64, v_dtype=pkg.CFK_FP8_E4M3)  # not a reference mode
    with pytest.raises(pkg.CfkError):
        pkg.fmha_forward_plan(pkg.CFK_FP16, 1, 1, 512, 512, 64, v_layout=1)
    pkg.fmha_forward_plan(pkg.CFK_FP8_E4M3, 1, 1, 512, 512, 128, v_layout=1)
    # one batch entry is addressed with 32-bit byte offsets: S * H * D * 2 bytes must stay below 2 GiB
    with pytest.raises(pkg.CfkError) as e:
        pkg.fmha_forward_plan(pkg.CFK_FP16, 1, 64, 131072, 131072, 128)
    assert e.value.code == -2 and "2 GiB" in str(e.value)
    pkg.fmha_forward_plan(pkg.CFK_FP16, 64, 16, 65536, 65536, 128)   # large batch is fine: entries are 64-bit apart
    # null params / null pointers
    lib = pkg.lib()
    assert lib.cfk_fmha_forward(None, None) == -1
    p = pkg.fmha.make_params(pkg.CFK_FP16, 1, 1, 512, 512, 64)
    assert lib.cfk_fmha_forward(ctypes.byref(p), None) == -1 and "non-NULL" in pkg.last_error()
    p = pkg.fmha.make_params(pkg.CFK_FP16, 1, 1, 512, 512, 64, softmax_scale=-1.0)
    assert lib.cfk_fmha_forward_plan(ctypes.byref(p), None, None, None, None) == -1
    assert lib.cfk_gemm_f16(100, 256, 64, None, None, None, 0, None) == -1
    assert lib.cfk_gemm_f16(100, 256, 64, 1, 1, 1, 0, None) == -2
    # cfk_gemm: argument checks come before any GPU work
    assert lib.cfk_gemm(None, None) == -1
    g = pkg.fmha.GemmParams()
    assert ctypes.sizeof(g) == 8 * 4 + 4 * 8   # six int32, two floats, four pointers
    g.dtype, g.layout, g.m, g.n, g.k, g.batch, g.a, g.b, g.d = pkg.CFK_FP32, 0, 256, 256, 64, 1, 1, 1, 1
    g.dtype = 2                                 # e4m3 is not a GEMM type
    assert lib.cfk_gemm(ctypes.byref(g), None) == -1
    g.dtype, g.layout = pkg.CFK_FP32, 1         # fp32 has the TN layout only
    assert lib.cfk_gemm(ctypes.byref(g), None) == -2
    g.layout, g.k = 0, 100
    assert lib.cfk_gemm(ctypes.byref(g), None) == -2
    g.k, g.batch = 64, 0
    assert lib.cfk_gemm(ctypes.byref(g), None) == -1
    # the kernel addresses a 256-row operand tile with 32-bit byte offsets: 256 * K * element size < 4 GiB
    g.batch, g.k = 1, 1 << 22                   # fp32: 256 * 4 Mi * 4 B = 4 GiB
    assert lib.cfk_gemm(ctypes.byref(g), None) == -2 and "K too large" in pkg.last_error()
    g.dtype, g.k = pkg.CFK_FP16, 1 << 23        # fp16: 256 * 8 Mi * 2 B = 4 GiB
    assert lib.cfk_gemm(ctypes.byref(g), None) == -2 and "K too large" in pkg.last_error()
    g.k, g.layout, g.n = 64, 1, 1 << 25         # NN: 64 * N * 2 B = 4 GiB
    assert lib.cfk_gemm(ctypes.byref(g), None) == -2 and "N too large" in pkg.last_error()


def test_plan_query_from_many_host_threads():
    # the plan query touches no GPU and keeps its error message per thread
    import threading
    errors = []

    def worker(i):
        try:
            for _ in range(200):
                d = (64, 128, 256)[i % 3]
                bm, bn, lds, thr = pkg.fmha_forward_plan(pkg.CFK_FP16 if i % 2 else pkg.CFK_FP8_E4M3, 2, 4, 1024, 1024, d)
                assert 1024 % bm == 0 and 1024 % bn == 0
                try:
                    pkg.fmha_forward_plan(pkg.CFK_FP16, 1, 1, 512, 512, 96 + i)
                except pkg.CfkError as e:
                    assert f"Unsupported head dim: {96 + i}" in str(e)   # this thread's own message
                else:
                    raise AssertionError("head dim must be rejected")
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_python_binding_refuses_cpu_tensors():
    import torch
    x = torch.zeros((1, 128, 1, 64), dtype=torch.float16)
    with pytest.raises(ValueError):
        pkg.fmha_forward(x, x, x)


def test_predictable_latency_option_changes_the_choice_of_kernel_without_gpu():
    # big fp16 problems at head dim 128 run the two-pass build with the hand-scheduled loop (160 KB of LDS); with the option
    # set the choice falls on the one-pass build (128 KB); unknown options are refused
    f = pkg.fmha
    assert f.fmha_forward_plan(f.CFK_FP16, 8, 16, 2048, 2048, 128)[:3] == (256, 128, 163840)
    # ... and so do big e4m3 problems from 3072 keys (below, e4m3 weights always follow the running max: one pass)
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 16, 4096, 4096, 128) == "fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>"
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 16, 4096, 2048, 128) == "fmha_fwd_kernel<128,64,8,2,1,1,0,0,2,0,0,0>"
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 16, 4096, 4096, 128, v_layout=f.CFK_V_BDHS) == "fmha_fwd_kernel<128,64,4,2,1,1,1,0,1,0,0,0>"
    f.set_option(f.CFK_OPT_PREDICTABLE_LATENCY, 1)
    try:
        assert f.fmha_forward_plan(f.CFK_FP16, 8, 16, 2048, 2048, 128)[:3] == (256, 128, 131072)
        assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 16, 4096, 4096, 128) == "fmha_fwd_kernel<128,64,8,2,1,1,0,0,2,0,0,0>"
    finally:
        f.set_option(f.CFK_OPT_PREDICTABLE_LATENCY, 0)
    # where the hand-scheduled persistent builds start (one workgroup per CU): fp16 from more 256-row items than half the
    # CUs (head dim 256, 128-row items on either side: always); e4m3 likewise, while the last round keeps four
    # fifths of the CUs busy
    assert f.fmha_forward_kernel(f.CFK_FP16, 1, 16, 2048, 2048, 128) == "fmha_fwd_kernel16p<128,64,4,1,0,0,0,0,2,0,1,1>"   # 128 items: the 4-wave shape
    assert f.fmha_forward_kernel(f.CFK_FP16, 1, 6, 2048, 2048, 64) == "fmha_fwd_kernel16p<64,64,4,1,0,0,0,0,2,0,1,1>"     # (up to 256 items of 128 rows,
    assert "kernel16p<" not in f.fmha_forward_kernel(f.CFK_FP16, 1, 64, 512, 512, 128)                                    #  from 1024 keys)
    assert f.fmha_forward_kernel(f.CFK_FP16, 1, 2, 2048, 2048, 128) == "fmha_fwd_kernel_ks<128,8>"                        # small grids: the key-split build
    assert "kernel16p<128" in f.fmha_forward_kernel(f.CFK_FP16, 1, 20, 2048, 2048, 128)         # 160
    assert "kernel16p<128" in f.fmha_forward_kernel(f.CFK_FP16, 1, 40, 2048, 2048, 128)         # 320
    assert "kernel16p<64" in f.fmha_forward_kernel(f.CFK_FP16, 1, 24, 2048, 2048, 64)
    assert "kernel16p<256" in f.fmha_forward_kernel(f.CFK_FP16, 1, 3, 8192, 8192, 256)          # 192 items of 128 rows
    assert "kernel16p<256" in f.fmha_forward_kernel(f.CFK_FP16, 1, 1, 8192, 8192, 256)          # (at head dim 256 from 1024 keys)
    assert "kernel16p<256" in f.fmha_forward_kernel(f.CFK_FP16, 1, 2, 1024, 1024, 256)
    assert "kernel16p<" not in f.fmha_forward_kernel(f.CFK_FP16, 16, 64, 512, 512, 256)
    assert "kernel16p<128" in f.fmha_forward_kernel(f.CFK_FP16, 1, 64, 2048, 2048 + 64, 128)    # (a key length with a tile left over)
    # (... while idle rows, leftover tiles and a thinly filled last round of items do not add up: 320 items in two rounds
    # and a leftover tile on top stay compiler-scheduled)
    assert "kernel16p<" not in f.fmha_forward_kernel(f.CFK_FP16, 1, 40, 2048, 2048 + 64, 128)
    assert "kernel16p<" not in f.fmha_forward_kernel(f.CFK_FP16, 8, 17, 896, 3520, 64)
    # big problems with short keys: the compiler-scheduled 256-row builds need key length to pay (fp16 below 1152 keys and
    # e4m3 below 2048 take 128-row tiles)
    assert f.fmha_forward_kernel(f.CFK_FP16, 8, 27, 1536, 896, 128) == "fmha_fwd_kernel16<128,64,4,2,0,0,0,0,1,0,1,0>"
    assert f.fmha_forward_kernel(f.CFK_FP16, 8, 32, 2048, 1216, 128) == "fmha_fwd_kernel16<128,64,8,2,0,0,0,0,1,0,1,0>"
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 8, 32, 2048, 1024, 128) == "fmha_fwd_kernel<128,64,4,2,1,1,0,0,1,0,0,0>"
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 8, 32, 2048, 2048, 128) == "fmha_fwd_kernel<128,64,8,2,1,1,0,0,2,0,0,0>"
    # the compiler-scheduled 256-row builds for e4m3 Q and K (one 8-wave workgroup per CU) while their rounds of 256 items fill
    hyb = lambda h: f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, h, 4096, 4096, 128, v_dtype=f.CFK_FP16).split(",")[2]
    assert [hyb(h) for h in (8, 10, 16, 20, 24, 32, 36, 48)] == ["4", "8", "8", "4", "4", "8", "4", "8"]
    e4 = lambda h: f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, h, 2048, 2048, 128).split(",")[2]
    assert [e4(h) for h in (16, 20, 32, 40, 64, 72)] == ["4", "8", "8", "4", "8", "4"]
    # query lengths that leave the last 256-row tile partly filled: the 8-wave shape while at most a quarter of the rows idle
    assert f.fmha_forward_kernel(f.CFK_FP16, 8, 16, 2016, 2048, 128) == "fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>"
    assert f.fmha_forward_kernel(f.CFK_FP16, 8, 16, 384, 2048, 128) == "fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>"
    assert f.fmha_forward_kernel(f.CFK_FP16, 8, 128, 128, 2048, 128) == "fmha_fwd_kernel<128,64,4,2,0,0,0,0,1,0,0,0>"     # (half would)
    assert f.fmha_forward_kernel(f.CFK_FP16, 8, 16, 320, 2048, 128) == "fmha_fwd_kernel<128,64,4,2,0,0,0,0,1,0,0,0>"
    assert f.fmha_forward_kernel(f.CFK_FP16, 4, 16, 160, 2048, 128) == "fmha_fwd_kernel16p<128,64,4,1,0,0,0,0,2,0,1,1>"    # (128-row tiles: no smaller one to prefer)
    assert "kernel16p<" not in f.fmha_forward_kernel(f.CFK_FP16, 1, 8, 8192, 8192 + 32, 256)    # (head dim 256: whole 128s only)
    assert "kernel8p<" not in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 16, 4096, 4096 + 64, 128)  # (e4m3 from 4096 keys: whole 256s only,
    assert "kernel8p<" in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 16, 4096, 3072 + 64, 128)      #  below that also with tiles left over)
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 8, 4096, 4096, 128) == "fmha_fwd_kernel8p<128,64,4,2,1,1,0,0,2,0,0,1>"   # 128 items: the 4-wave shape
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 9, 4096, 4096, 128) == "fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>"   # 288 items of 128 rows, 144 of 256
    assert "kernel8p<" in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 10, 4096, 4096, 128)         # 160
    assert "kernel8p<" in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 16, 4096, 4096, 128)         # 256: one round
    assert "kernel8p<" not in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 20, 4096, 4096, 128)     # 320: a quarter-full second round
    assert "kernel8p<" in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 28, 4096, 4096, 128)         # 448
    # ... by the same rules from 3072 keys on; below, where the first-tile reference point of the first pass costs accuracy
    # and the kernels run their max-tracking pass only, the hand-scheduled build runs by wish only
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 8, 3072, 3072, 128) == "fmha_fwd_kernel8p<128,64,4,2,1,1,0,0,2,0,0,1>"
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 16, 4096, 3072, 128) == "fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>"
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 16, 4064, 3072, 128) == "fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>"   # (a partly filled last query tile)
    assert "kernel8p<" not in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 20, 4096, 3072, 128)     # (320: a quarter-full second round)
    assert "kernel8p<" not in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 16, 4096, 2816, 128)
    # e4m3 weights without an exponential: the same choice of tile, the DirectCfg build of it; kernels without e4m3 P
    # have no such build
    f.set_option(f.CFK_OPT_FAST_E4M3_WEIGHTS, 1)
    try:
        assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 16, 4096, 4096, 128) == "fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>/direct"
        assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 32, 4096, 4096, 64) == "fmha_fwd_kernel<64,64,4,3,1,1,0,0,1,0,0,0>/direct"
        assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 1, 16, 4096, 3072, 128) == "fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>/direct"
        assert "kernel8p<" not in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 16, 4096, 2048, 128)
        assert f.fmha_forward_kernel(f.CFK_FP16, 8, 16, 2048, 2048, 128) == "fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>"
        assert "/direct" not in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 16, 4096, 4096, 128, v_dtype=f.CFK_FP16)
        assert "/direct" not in f.fmha_forward_kernel(f.CFK_FP8_E4M3, 2, 8, 4096, 4096, 256)
    finally:
        f.set_option(f.CFK_OPT_FAST_E4M3_WEIGHTS, 0)
    assert f.fmha_forward_kernel(f.CFK_FP8_E4M3, 4, 16, 4096, 4096, 128) == "fmha_fwd_kernel8p<128,64,8,2,1,1,0,0,2,0,0,1>"
    with pytest.raises(pkg.CfkError):
        f.set_option(99, 1)
