"""GPU parity of the fp8 e4m3 FMHA forward (through the C-ABI) against the CPU oracle run on the DEQUANTISED
operands, as the reference's own check does (src/fmha-pipeline/fmha_forward.cu:613-631).  Gates: max-abs error
<= 5e-2 everywhere; the reference's error-percentage criterion at its fp8 threshold (fmha_forward.cu:638-639) from
S >= 2048 on; below that, "no worse than the reference's device algorithm emulated on the same operands"."""
import numpy as np
import pytest

import oracle
from _util import ERRPCT_FP8, TOL_FP8, climbing_keys, max_abs, pkg, subset_pairs, to_dev

pytestmark = pytest.mark.gpu


def _quant(x, per_tensor=True):
    if per_tensor:
        codes, scale = oracle.quantize_e4m3_per_tensor(x)
    else:  # the reference's mode: values cast straight to e4m3, no scales (fmha_forward.cu:498-500)
        codes, scale = oracle.e4m3_encode(x), np.float32(1.0)
    return codes, float(scale), oracle.e4m3_decode(codes) * scale


def _run(q, k, v, per_tensor=True, **kw):
    import torch
    (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = (_quant(x, per_tensor) for x in (q, k, v))
    o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=qs, k_descale=ks, v_descale=vs, **kw)
    torch.cuda.synchronize()
    return o.float().cpu().numpy(), (qf, kf, vf)


def _reference_algorithm_error(qf, kf, vf, ref, D):
    """Error of the REFERENCE's device algorithm against the fp32 oracle on the same operands: tiled online softmax
    with P in (0, 1] cast straight to e4m3 (fmha_consumer.h:54, online_softmax.h:87-207), emulated in numpy.
    Returns (max-abs, error-%)."""
    B, _, H, _ = qf.shape
    emu = np.empty_like(ref)
    for b in range(B):
        for h in range(H):
            emu[b, :, h], _, _ = oracle.online_softmax_tiled(qf[b, :, h], kf[b, :, h], vf[b, :, h], 64,
                                                             oracle.LOG2E / np.sqrt(np.float32(D)), p_cast="e4m3")
    return max_abs(emu, ref), oracle.verify_tensor(emu, ref, ERRPCT_FP8)[1]


# the kernel may not be worse than the reference's own algorithm by more than this factor (plus a floor for
# shapes where both errors are tiny)
EMU_FACTOR, EMU_ABS_FLOOR, EMU_PCT_FLOOR = 1.25, 1e-3, 1e-3


def _check_full(B, S, H, D, per_tensor=True, seqlen_kv=None):
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=seqlen_kv)
    got, (qf, kf, vf) = _run(q, k, v, per_tensor)
    ref = oracle.attention_f32(qf, kf, vf)["O"]
    err = max_abs(got, ref)
    ok, pct = oracle.verify_tensor(got, ref, ERRPCT_FP8)
    print(f"fp8 B={B} S={S}/{seqlen_kv or S} H={H} D={D} per_tensor={per_tensor}: max-abs {err:.3e}, error% {pct:.2e}")
    assert err <= TOL_FP8, err
    if S >= 2048 and (seqlen_kv or S) >= 2048:
        # the reference's own gate at its fp8 threshold (fmha_forward.cu:638-639), calibrated for its problem size
        # (S = 4096, where the e4m3 rounding noise of P averages over thousands of keys)
        assert ok, pct
    else:
        # Short sequences: with few keys the e4m3 rounding of P does not average out and the reference's device
        # algorithm itself misses that gate.  The criterion that replaces it: the kernel is no worse than that
        # algorithm, emulated on the same operands, in both of the reference's error measures.
        emu_err, emu_pct = _reference_algorithm_error(qf, kf, vf, ref, D)
        print(f"    reference algorithm (P cast to e4m3, emulated): max-abs {emu_err:.3e}, error% {emu_pct:.2e}")
        assert err <= EMU_FACTOR * emu_err + EMU_ABS_FLOOR, (err, emu_err)
        assert pct <= EMU_FACTOR * emu_pct + EMU_PCT_FLOOR, (pct, emu_pct)
    return got, ref


@pytest.mark.parametrize("B,S,H,D", [(1, 256, 2, 128), (2, 512, 3, 128), (1, 1024, 4, 128), (1, 4096, 2, 128),
                                     (2, 512, 3, 64), (1, 4096, 2, 64), (2, 384, 2, 256), (1, 4096, 1, 256)])
def test_shapes_per_tensor_scales(B, S, H, D):
    _check_full(B, S, H, D)


@pytest.mark.parametrize("B,S,H,D,Skv", [(1, 128, 1, 64, 64), (1, 128, 1, 128, 64), (2, 256, 2, 128, 192), (1, 128, 2, 256, 64)])
def test_shortest_and_odd_key_tile_counts(B, S, H, D, Skv):
    _check_full(B, S, H, D, seqlen_kv=Skv)


@pytest.mark.parametrize("mode", ["fp8", "hybrid"])
@pytest.mark.parametrize("B,S,H,D,Skv", [(1, 256, 2, 128, 512), (1, 128, 2, 64, 384), (1, 128, 1, 256, 256), (1, 128, 1, 128, 64),
                                         (2, 2048, 32, 128, 2048)])
def test_scores_that_climb_along_the_keys_move_the_reference_point(mode, B, S, H, D, Skv):
    # the deferred rescale's slow path, many times per row (e4m3 P has two binades of head-room above the row max of
    # the moment, so here almost every tile takes it); from 3072 keys on the e4m3 kernel starts in its pass without a row
    # max per tile, finds non-finite rows and walks the keys again (the tests of the second pass below).  The last shape is large enough for the automatic
    # choice of the 256-row tile (two sub-tiles per barrier for e4m3 P).
    import torch
    from _util import TOL_FP16
    if B * H * (S // 256) >= 512:
        f = pkg.fmha
        plan = f.fmha_forward_plan(f.CFK_FP8_E4M3, B, H, S, Skv, D, v_dtype=f.CFK_FP8_E4M3 if mode == "fp8" else f.CFK_FP16)
        assert plan[:2] == ((256, 128) if mode == "fp8" else (256, 64)), plan
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=Skv)
    k, v = climbing_keys(k, ramp=4.0, spike=8.0), v / 4
    (qc, qs, qf), (kc, ks, kf) = _quant(q), _quant(k)
    if mode == "fp8":
        vc, vs, vf = _quant(v)
        o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=qs, k_descale=ks, v_descale=vs)
    else:
        v16 = v.astype(np.float16)
        vf = v16.astype(np.float32)
        o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(v16), q_descale=qs, k_descale=ks)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    pairs = sorted({(0, 0), (B - 1, H - 1)})
    ref = oracle.attention_f32(qf, kf, vf, bh_pairs=pairs)["O"]
    sel = ~np.isnan(ref)
    err = max_abs(got[sel], ref[sel])
    print(f"{mode} climbing B={B} S={S}/{Skv} H={H} D={D}: max-abs {err:.3e}")
    assert not np.isnan(got).any()
    assert err <= (TOL_FP8 if mode == "fp8" else TOL_FP16), err


def test_reference_mode_unit_scales():
    _check_full(1, 512, 2, 128, per_tensor=False)


def test_rectangular_q_kv():
    _check_full(1, 256, 2, 128, seqlen_kv=640)
    _check_full(1, 512, 2, 128, seqlen_kv=128)


def test_not_worse_than_the_reference_algorithm_with_e4m3_p():
    # One head in detail: the kernel against the fp32 oracle and against the numpy emulation of the reference's
    # algorithm (P in (0, 1] cast straight to e4m3).  The kernel keeps P 2^7 higher (small weights stay out of
    # e4m3's flush zone) and sums the rounded weights, so it differs from the emulation by about as much as either
    # differs from the fp32 result -- what is asserted is that its error is not the larger one.
    B, S, H, D = 1, 256, 1, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    got, (qf, kf, vf) = _run(q, k, v)
    ref = oracle.attention_f32(qf, kf, vf)["O"]
    emu, _, _ = oracle.online_softmax_tiled(qf[0, :, 0], kf[0, :, 0], vf[0, :, 0], 64, oracle.LOG2E / np.sqrt(D),
                                            p_cast="e4m3")
    e_ref, e_emu, emu_ref = max_abs(got[0, :, 0], ref[0, :, 0]), max_abs(got[0, :, 0], emu), max_abs(emu, ref[0, :, 0])
    print(f"kernel vs fp32 attention {e_ref:.3e}; kernel vs e4m3-P emulation {e_emu:.3e}; emulation vs fp32 {emu_ref:.3e}")
    assert e_ref <= TOL_FP8 and e_ref <= EMU_FACTOR * emu_ref + EMU_ABS_FLOOR


def test_exact_arithmetic_pins_the_v_layout_transform():
    # Exact-arithmetic mode (the reference's integer-input trick, include/utils/random.hpp:13-32, taken one step
    # further): integer scores with scale*log2e = 1 make every P a power of two, exactly representable in e4m3,
    # and integer V in [-8, 8] is exact too -- so the fp8 kernel has NO rounding left but the fp16 output, and any
    # wrong key <-> V-row association in the tr8 operand transform shows up at full size.
    rng = np.random.default_rng(11)
    for D in (64, 128, 256):
        B, S, H = 1, 512, 2
        q = np.zeros((B, S, H, D), np.float32)
        idx = rng.integers(0, D, (B, S, H, 4))
        np.put_along_axis(q, idx, 1.0, axis=-1)                       # up to four ones per query row
        k = rng.integers(-1, 2, (B, S, H, D)).astype(np.float32)      # scores are integers in [-4, 4]
        v = rng.integers(-8, 9, (B, S, H, D)).astype(np.float32)
        got, (qf, kf, vf) = _run(q, k, v, per_tensor=False, softmax_scale=float(np.log(2.0)))
        assert np.array_equal(qf, q) and np.array_equal(kf, k) and np.array_equal(vf, v)
        ref = oracle.attention_f32(qf, kf, vf, alpha0=np.log(2.0))["O"]
        np.testing.assert_allclose(got, ref, rtol=1.5e-3, atol=2e-4)


def test_taps_and_invariants():
    import torch
    B, S, H, D = 1, 512, 2, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    rm = torch.full((B, H, S), -1.0, dtype=torch.float32, device="cuda:0")
    rs = torch.full((B, H, S), -1.0, dtype=torch.float32, device="cuda:0")
    base, (qf, kf, vf) = _run(q, k, v, row_max=rm, row_sum=rs)
    r = oracle.attention_f32(qf, kf, vf, want_stats=True)
    # max-check / sum-check (fmha_forward.cu:655-676); scores are exact products of e4m3 values in fp32
    np.testing.assert_allclose(rm.cpu().numpy() / oracle.LOG2E, r["row_max"], rtol=1e-4, atol=1e-4)
    # the e4m3 kernel sums the weights AS ROUNDED to e4m3 (the ones the second GEMM applies; the reference sums them
    # in fp32 before the cast, online_softmax.h:173-206): rounding is unbiased, so the two sums agree to well under 1 %
    np.testing.assert_allclose(1.0 / rs.cpu().numpy(), r["inv_sum"], rtol=1e-2)
    # V = 1 -> O = 1 up to fp16 rounding: numerator and denominator add up the same rounded weights.  Also pins the
    # lane mapping of the row-sum MFMA (sums landing on another query's lane would break this)
    ones, _ = _run(q, k, np.ones_like(v))
    assert max_abs(ones, 1.0) <= 1e-3
    # a common permutation of the keys (pins the V-tile layout transform: wrong key order in V would show here
    # and in every other test)
    perm = np.random.default_rng(5).permutation(S)
    permd, _ = _run(q, k[:, perm], v[:, perm])
    assert max_abs(base, permd) <= 2e-2
    # one dominant key selects its V row exactly (e4m3 V values are exact in fp16)
    qd = np.zeros_like(q)
    qd[..., 0] = 300.0
    kd = np.zeros_like(k)
    kd[0, 77, :, 0] = 300.0
    sel, (_, _, vf2) = _run(qd, kd, v)
    np.testing.assert_allclose(sel[0, :, 0], np.broadcast_to(vf2[0, 77, 0], sel[0, :, 0].shape), rtol=2e-3, atol=1e-4)  # fp16 output rounding only


@pytest.mark.parametrize("B,S,H,D", [(1, 512, 2, 128), (2, 256, 3, 64), (1, 384, 2, 256), (2, 2048, 4, 128)])
def test_hybrid_mode_fp8_qk_fp16_pv(B, S, H, D):
    # the reference's --prec-type=2 without -DGEMM2FP8: Q,K e4m3, P and V fp16 (fmha_forward.cu:446-450).
    # GEMM-I on e4m3 products is exact in fp32, so the error is that of the fp16 path.
    import torch
    from _util import ERRPCT_FP16, TOL_FP16
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    (qc, qs, qf), (kc, ks, kf) = _quant(q), _quant(k)
    v16 = v.astype(np.float16)
    o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(v16), q_descale=qs, k_descale=ks)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    ref = oracle.attention_f32(qf, kf, v16.astype(np.float32))["O"]
    err = max_abs(got, ref)
    ok, pct = oracle.verify_tensor(got, ref, ERRPCT_FP16)
    print(f"hybrid B={B} S={S} H={H} D={D}: max-abs {err:.3e}, error% {pct:.2e}")
    assert err <= TOL_FP16 and ok


def test_hybrid_production_size_picks_the_256_row_tile():
    # a problem large enough for the automatic choice of the 256-row tile (batch*heads*(S/256) >= 512)
    import torch
    from _util import ERRPCT_FP16, TOL_FP16
    B, S, H, D = 4, 2048, 16, 128
    f = pkg.fmha
    assert f.fmha_forward_plan(f.CFK_FP8_E4M3, B, H, S, S, D, v_dtype=f.CFK_FP16)[0] == 256
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    (qc, qs, qf), (kc, ks, kf) = _quant(q), _quant(k)
    v16 = v.astype(np.float16)
    o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(v16), q_descale=qs, k_descale=ks)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    vf = v16.astype(np.float32)
    ref = oracle.attention_f32(qf, kf, vf, bh_pairs=subset_pairs(B, H))["O"]
    oracle.attention_f32(qf, kf, vf, bh_pairs=[(b, h) for b in range(B) for h in range(H)], row_start=11, row_step=61,
                         out=ref)
    sel = ~np.isnan(ref)
    err = max_abs(got[sel], ref[sel])
    ok, pct = oracle.verify_tensor(got[sel], ref[sel], ERRPCT_FP16)
    print(f"hybrid 256-row tile: checked {sel.sum()} elements, max-abs {err:.3e}, error% {pct:.2e}")
    assert err <= TOL_FP16 and ok and not np.any(np.isnan(got))


def test_hybrid_exact_arithmetic():
    rng = np.random.default_rng(12)
    for D in (64, 128, 256):
        B, S, H = 1, 384, 2
        q = np.zeros((B, S, H, D), np.float32)
        np.put_along_axis(q, rng.integers(0, D, (B, S, H, 4)), 1.0, axis=-1)
        k = rng.integers(-1, 2, (B, S, H, D)).astype(np.float32)
        v = rng.integers(-8, 9, (B, S, H, D)).astype(np.float32)
        import torch
        o = pkg.fmha_forward(to_dev(oracle.e4m3_encode(q)), to_dev(oracle.e4m3_encode(k)), to_dev(v.astype(np.float16)),
                             softmax_scale=float(np.log(2.0)))
        torch.cuda.synchronize()
        ref = oracle.attention_f32(q, k, v, alpha0=np.log(2.0))["O"]
        np.testing.assert_allclose(o.float().cpu().numpy(), ref, rtol=1.5e-3, atol=2e-4)


@pytest.mark.parametrize("B,S,H,D", [(2, 512, 3, 128), (1, 384, 2, 64), (1, 256, 2, 256), (1, 4096, 2, 128)])
def test_pretransposed_v_layout(B, S, H, D):
    # V handed over as [B,D,H,S], the reference's offline transpose (fmha_forward.cu:514-532): same result as the
    # [B,S,H,D] path up to the order of the fp32 accumulation
    import torch
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = (_quant(x) for x in (q, k, v))
    vt = oracle.transpose_v_bdhs(vc)
    assert vt.shape == (B, D, H, S)
    o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vt), q_descale=qs, k_descale=ks, v_descale=vs,
                         v_layout=pkg.fmha.CFK_V_BDHS)
    o2 = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=qs, k_descale=ks, v_descale=vs)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    ref = oracle.attention_f32(qf, kf, vf)["O"]
    err = max_abs(got, ref)
    print(f"fp8 [B,D,H,S] V B={B} S={S} H={H} D={D}: max-abs {err:.3e}; vs [B,S,H,D] path {max_abs(got, o2.float().cpu().numpy()):.3e}")
    assert err <= TOL_FP8
    assert max_abs(got, o2.float().cpu().numpy()) <= 2e-3   # same P, same V, different summation order
    if S >= 2048:
        assert oracle.verify_tensor(got, ref, ERRPCT_FP8)[0]
    else:
        emu_err, emu_pct = _reference_algorithm_error(qf, kf, vf, ref, D)
        assert err <= EMU_FACTOR * emu_err + EMU_ABS_FLOOR, (err, emu_err)
        assert oracle.verify_tensor(got, ref, ERRPCT_FP8)[1] <= EMU_FACTOR * emu_pct + EMU_PCT_FLOOR


def test_pretransposed_v_exact_arithmetic():
    rng = np.random.default_rng(13)
    import torch
    for D in (64, 128, 256):
        B, S, H = 1, 384, 2
        q = np.zeros((B, S, H, D), np.float32)
        np.put_along_axis(q, rng.integers(0, D, (B, S, H, 4)), 1.0, axis=-1)
        k = rng.integers(-1, 2, (B, S, H, D)).astype(np.float32)
        v = rng.integers(-8, 9, (B, S, H, D)).astype(np.float32)
        o = pkg.fmha_forward(to_dev(oracle.e4m3_encode(q)), to_dev(oracle.e4m3_encode(k)),
                             to_dev(oracle.transpose_v_bdhs(oracle.e4m3_encode(v))), softmax_scale=float(np.log(2.0)),
                             v_layout=pkg.fmha.CFK_V_BDHS)
        torch.cuda.synchronize()
        ref = oracle.attention_f32(q, k, v, alpha0=np.log(2.0))["O"]
        np.testing.assert_allclose(o.float().cpu().numpy(), ref, rtol=1.5e-3, atol=2e-4)


@pytest.mark.parametrize("mode", ["fp8", "fp8_bdhs", "hybrid"])
def test_score_tap(mode):
    import torch
    B, S, H, D = 1, 256, 2, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = (_quant(x) for x in (q, k, v))
    sc = torch.full((B, H, S, S), -1.0, dtype=torch.float32, device="cuda:0")
    if mode == "hybrid":
        vdev, kw, vf = to_dev(v.astype(np.float16)), {}, v.astype(np.float16).astype(np.float32)
    elif mode == "fp8_bdhs":
        vdev, kw = to_dev(oracle.transpose_v_bdhs(vc)), dict(v_descale=vs, v_layout=pkg.fmha.CFK_V_BDHS)
    else:
        vdev, kw = to_dev(vc), dict(v_descale=vs)
    o = pkg.fmha_forward(to_dev(qc), to_dev(kc), vdev, q_descale=qs, k_descale=ks, scores=sc, **kw)
    torch.cuda.synchronize()
    r = oracle.attention_f32(qf, kf, vf, want_scores=True)
    assert max_abs(o.float().cpu().numpy(), r["O"]) <= TOL_FP8
    # the oracle multiplies the dequantised floats (each rounded after its descale), the kernel scales the exact
    # product of the codes once: differences of a few 1e-4 on scores of magnitude ~1-5
    assert oracle.verify_tensor(sc.cpu().numpy(), r["S"])[0]
    np.testing.assert_allclose(sc.cpu().numpy(), r["S"], rtol=1e-3, atol=1e-3)


def test_unsupported_modes_report_errors():
    import torch
    x = torch.zeros((1, 128, 1, 64), dtype=torch.uint8, device="cuda:0")
    xt16 = torch.zeros((1, 64, 1, 128), dtype=torch.float16, device="cuda:0")
    with pytest.raises(pkg.CfkError) as e:
        pkg.fmha_forward(x, x, xt16, v_layout=pkg.fmha.CFK_V_BDHS)   # pre-transposed V is an e4m3-V layout
    assert e.value.code == -2


def test_config4_subset_check():
    # benchmark configuration 4: fp8 e4m3 B=4 H=16 S=4096 D=128, per-tensor amax scales, V in [B,S,H,D]
    B, S, H, D = 4, 4096, 16, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    got, (qf, kf, vf) = _run(q, k, v)
    pairs = subset_pairs(B, H)
    ref = oracle.attention_f32(qf, kf, vf, bh_pairs=pairs)["O"]
    oracle.attention_f32(qf, kf, vf, bh_pairs=[(b, h) for b in range(B) for h in range(H)], row_start=17,
                         row_step=61, out=ref)
    sel = ~np.isnan(ref)
    err = max_abs(got[sel], ref[sel])
    ok, pct = oracle.verify_tensor(got[sel], ref[sel], ERRPCT_FP8)
    # for information: error against the attention of the UNQUANTISED tensors
    full = oracle.attention_f32(q, k, v, bh_pairs=pairs[:1])["O"]
    s1 = ~np.isnan(full)
    print(f"fp8 cfg4: checked {sel.sum()} elements, max-abs {err:.3e}, error% {pct:.2e}; "
          f"vs unquantised fp32 attention {max_abs(got[s1], full[s1]):.3e}")
    assert err <= TOL_FP8 and ok
    assert not np.any(np.isnan(got))


# ---- the two-pass e4m3 kernel (from 3072 keys on): first pass without a row max per tile, second pass only where a
# weight left the range of e4m3.  Every instantiation that can take the second pass is driven through it here.
def _climb_case(B, S, H, D, Skv, v_layout=None, ramp=4.0, spike=8.0):
    import torch
    f = pkg.fmha
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=Skv)
    k, v = climbing_keys(k, ramp=ramp, spike=spike), v / 4
    (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = _quant(q), _quant(k), _quant(v)
    if v_layout == "bdhs":
        vdev = to_dev(np.ascontiguousarray(vc.transpose(0, 3, 2, 1)))  # [B,S,H,D] -> [B,D,H,S]
        o = pkg.fmha_forward(to_dev(qc), to_dev(kc), vdev, q_descale=qs, k_descale=ks, v_descale=vs, v_layout=f.CFK_V_BDHS)
    else:
        o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=qs, k_descale=ks, v_descale=vs)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    pairs = sorted({(0, 0), (B - 1, H - 1)})
    ref = oracle.attention_f32(qf, kf, vf, bh_pairs=pairs)["O"]
    sel = ~np.isnan(ref)
    err = max_abs(got[sel], ref[sel])
    print(f"e4m3 climbing B={B} S={S}/{Skv} H={H} D={D} v_layout={v_layout}: max-abs {err:.3e}")
    assert not np.isnan(got).any()
    assert err <= TOL_FP8, err


@pytest.mark.parametrize("B,S,H,D,Skv", [(1, 256, 2, 64, 4096), (1, 128, 3, 64, 4352), (1, 128, 2, 256, 4096), (1, 256, 1, 256, 4224)])
def test_second_pass_at_head_dims_64_and_256(B, S, H, D, Skv):
    # head dim 64 runs three waves per SIMD; head dim 256 has no row sum on the MFMA pipe: a non-finite O is all its
    # detection has
    _climb_case(B, S, H, D, Skv)


@pytest.mark.parametrize("B,S,H,D,Skv", [(1, 256, 2, 64, 4096), (1, 256, 2, 128, 4096), (1, 128, 1, 256, 4096), (1, 256, 2, 128, 4608)])
def test_second_pass_with_pretransposed_v(B, S, H, D, Skv):
    _climb_case(B, S, H, D, Skv, v_layout="bdhs")


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("where", ["one_row_mid", "one_row_last_tile"])
def test_second_pass_for_a_single_row(D, where):
    # N(0,1) operands, except that ONE query row is a large multiple of ONE key -- in the middle of the key sequence, or
    # in its last tile: that row's score there exceeds the first tile's max by far more than e4m3 P has room for, every
    # other row of the workgroup (and every other workgroup) is ordinary.  The workgroup that owns the row takes the
    # second pass; the result must be right for the row and for its neighbours.
    import torch
    B, S, H, Skv = 1, 256, 2, 4096
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=Skv)
    row, key = 77, (1000 if where == "one_row_mid" else Skv - 3)
    q[0, row, 1] = 6.0 * k[0, key, 1]
    (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = _quant(q), _quant(k), _quant(v)
    o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=qs, k_descale=ks, v_descale=vs)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    ref = oracle.attention_f32(qf, kf, vf)["O"]
    err = max_abs(got, ref)
    # the row itself: its softmax is one key
    assert max_abs(got[0, row, 1], vf[0, key, 1]) <= TOL_FP8
    print(f"e4m3 single climbing row D={D} {where}: max-abs {err:.3e}")
    assert not np.isnan(got).any() and err <= TOL_FP8, err


def test_both_sides_of_the_key_length_where_the_passes_change():
    # below 2048 keys: one pass whose reference point follows the running max (tau = 0); from 2048 on it moves only when it
    # must (deferred rescale); from 3072 on: two passes.  The same operands, cut on both sides of each boundary.
    B, S, H, D = 1, 256, 2, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=4096)
    for skv in (1984, 2048, 3008, 3072, 4096):
        got, (qf, kf, vf) = _run(q, k[:, :skv], v[:, :skv])
        ref = oracle.attention_f32(qf, kf, vf)["O"]
        err, (ok, pct) = max_abs(got, ref), oracle.verify_tensor(got, ref, ERRPCT_FP8)
        print(f"e4m3 S_kv={skv}: max-abs {err:.3e}, error% {pct:.2e}")
        assert err <= TOL_FP8 and pct <= 2 * ERRPCT_FP8 + EMU_PCT_FLOOR, (skv, err, pct)


def test_predictable_latency_option_takes_the_tracked_pass():
    # cfk_set_option(CFK_OPT_PREDICTABLE_LATENCY, 1): straight to the pass that tracks the row max -- the pass a call
    # with taps takes, so the two outputs are bit-identical; the default (two passes) agrees to rounding
    import torch
    f = pkg.fmha
    B, S, H, D = 1, 256, 2, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=4096)
    (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = _quant(q), _quant(k), _quant(v)
    args = (to_dev(qc), to_dev(kc), to_dev(vc))
    kw = dict(q_descale=qs, k_descale=ks, v_descale=vs)
    o_default = pkg.fmha_forward(*args, **kw).float().cpu().numpy()
    rm = torch.zeros((B, H, S), dtype=torch.float32, device="cuda:0")
    o_taps = pkg.fmha_forward(*args, row_max=rm, **kw).float().cpu().numpy()
    f.set_option(f.CFK_OPT_PREDICTABLE_LATENCY, 1)
    try:
        o_opt = pkg.fmha_forward(*args, **kw).float().cpu().numpy()
    finally:
        f.set_option(f.CFK_OPT_PREDICTABLE_LATENCY, 0)
    assert np.array_equal(o_opt, o_taps)
    ref = oracle.attention_f32(qf, kf, vf)["O"]
    assert max_abs(o_default, ref) <= TOL_FP8 and max_abs(o_opt, ref) <= TOL_FP8


# ---- cfk_set_option(CFK_OPT_FAST_E4M3_WEIGHTS, 1): the first pass writes the e4m3 codes of the weights without an
# exponential (the DirectCfg builds).  Same gate as everything else here; what is looser than with the default is
# the reference's own error percentage, which is why this is an option (the header says by how much).
@pytest.fixture
def fast_weights():
    f = pkg.fmha
    f.set_option(f.CFK_OPT_FAST_E4M3_WEIGHTS, 1)
    try:
        yield f
    finally:
        f.set_option(f.CFK_OPT_FAST_E4M3_WEIGHTS, 0)


@pytest.mark.parametrize("B,S,H,D,v_layout", [(4, 4096, 16, 128, None), (1, 4096, 4, 128, None), (2, 4096, 8, 64, None),
                                              (1, 4096, 8, 64, "bdhs"), (1, 4096, 4, 128, "bdhs")])
def test_fast_e4m3_weights_parity(fast_weights, B, S, H, D, v_layout):
    import torch
    f = fast_weights
    name = f.fmha_forward_kernel(f.CFK_FP8_E4M3, B, H, S, S, D, v_layout=f.CFK_V_BDHS if v_layout else f.CFK_V_BSHD)
    assert name.endswith("/direct"), name
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = _quant(q), _quant(k), _quant(v)
    kw = dict(q_descale=qs, k_descale=ks, v_descale=vs)
    vdev = to_dev(np.ascontiguousarray(vc.transpose(0, 3, 2, 1))) if v_layout else to_dev(vc)
    if v_layout: kw["v_layout"] = f.CFK_V_BDHS
    fast = pkg.fmha_forward(to_dev(qc), to_dev(kc), vdev, **kw)
    torch.cuda.synchronize()
    f.set_option(f.CFK_OPT_FAST_E4M3_WEIGHTS, 0)
    exact = pkg.fmha_forward(to_dev(qc), to_dev(kc), vdev, **kw)
    torch.cuda.synchronize()
    fast, exact = fast.float().cpu().numpy(), exact.float().cpu().numpy()
    pairs = sorted({(0, 0), (B - 1, H - 1)})
    ref = oracle.attention_f32(qf, kf, vf, bh_pairs=pairs)["O"]
    sel = ~np.isnan(ref)
    e_fast, e_exact = np.abs(fast[sel] - ref[sel]), np.abs(exact[sel] - ref[sel])
    rms = lambda e: float(np.sqrt((e.astype(np.float64) ** 2).mean()))
    print(f"e4m3 fast weights {name}: max-abs {e_fast.max():.3e} (default {e_exact.max():.3e}), rms {rms(e_fast):.3e} ({rms(e_exact):.3e})")
    assert not np.isnan(fast).any() and e_fast.max() <= TOL_FP8
    assert not np.array_equal(fast, exact)                 # the option did change the kernel that ran ...
    assert rms(e_fast) <= 1.35 * rms(e_exact)              # ... by about what a fifth of the codes one step off costs


@pytest.mark.parametrize("D", [64, 128])
def test_fast_e4m3_weights_second_pass(fast_weights, D):
    # weights beyond the e4m3 range come out of the conversion as 0x7F (NaN, seen in the row sum) or with bit 7 set (seen
    # in the OR of the P registers): climbing keys, then a single row whose score leaves the range by a wide margin
    import torch
    _climb_case(1, 256, 2, D, 4096)
    if D == 128: _climb_case(4, 4096, 16, 128, 4096, ramp=1.5, spike=1.0)   # the hand-scheduled build; some workgroups only
    B, S, H, Skv = 1, 256, 2, 4096
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=Skv)
    q[0, 77, 1] = 6.0 * k[0, 1000, 1]
    (qc, qs, qf), (kc, ks, kf), (vc, vs, vf) = _quant(q), _quant(k), _quant(v)
    o = pkg.fmha_forward(to_dev(qc), to_dev(kc), to_dev(vc), q_descale=qs, k_descale=ks, v_descale=vs)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    ref = oracle.attention_f32(qf, kf, vf)["O"]
    assert max_abs(got[0, 77, 1], vf[0, 1000, 1]) <= TOL_FP8
    assert not np.isnan(got).any() and max_abs(got, ref) <= TOL_FP8


def test_very_long_sequence():
    # 512 key tiles per work item on the hand-scheduled e4m3 kernel; every 1531st row of every head against the oracle
    B, S, H, D = 1, 32768, 2, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    got, (qf, kf, vf) = _run(q, k, v)
    ref = np.full(got.shape, np.nan, np.float32)
    oracle.attention_f32(qf, kf, vf, bh_pairs=[(0, 0), (0, 1)], row_start=5, row_step=1531, out=ref)
    sel = ~np.isnan(ref)
    err = max_abs(got[sel], ref[sel])
    print(f"e4m3 B={B} S={S} H={H} D={D}: checked {sel.sum()} elements, max-abs {err:.3e}")
    assert err <= TOL_FP8 and np.isfinite(got).all()
