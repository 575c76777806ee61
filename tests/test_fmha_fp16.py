"""GPU parity of the fp16 FMHA forward (through the C-ABI) against the CPU oracle on the same seeded inputs.
Gate: max-abs error <= 2e-3 against the fp32 host reference attention, plus the reference's own error-percentage
criterion (include/utils/random.hpp:54-90, thresholds src/fmha-pipeline/fmha_forward.cu:638-639)."""
import numpy as np
import pytest

import oracle
from _util import ERRPCT_FP16, TOL_FP16, climbing_keys, max_abs, pkg, subset_pairs, to_dev

pytestmark = pytest.mark.gpu


def _run(q, k, v, **kw):
    import torch
    q16, k16, v16 = (x.astype(np.float16) for x in (q, k, v))
    o = pkg.fmha_forward(to_dev(q16), to_dev(k16), to_dev(v16), **kw)
    torch.cuda.synchronize()
    return o.float().cpu().numpy(), (q16.astype(np.float32), k16.astype(np.float32), v16.astype(np.float32))


def _check_full(B, S, H, D, kind="gaussian", seqlen_kv=None, scale=None, climb=False):
    q, k, v = pkg.testbed.qkv(B, S, H, D, kind=kind, seqlen_kv=seqlen_kv)
    if kind != "gaussian":
        q, k = q / 8, k / 8  # keep scores moderate
    if climb:
        k, v = climbing_keys(k), v / 4
    got, (qf, kf, vf) = _run(q, k, v, softmax_scale=scale)
    ref = oracle.attention_f32(qf, kf, vf, alpha0=scale)["O"]
    err = max_abs(got, ref)
    ok, pct = oracle.verify_tensor(got, ref, ERRPCT_FP16)
    print(f"fp16 B={B} S={S}/{seqlen_kv or S} H={H} D={D} {kind}: max-abs {err:.3e}, error% {pct:.2e}")
    assert err <= TOL_FP16, err
    assert ok, pct


def test_config1_full_check():
    # benchmark configuration 1: B=1 H=8 S=512 D=64, scale 1/sqrt(64), full CPU check
    _check_full(1, 512, 8, 64, scale=1.0 / 8.0)


@pytest.mark.parametrize("B,S,H,D", [(2, 256, 3, 128), (1, 384, 2, 256), (3, 128, 5, 64), (1, 1024, 1, 128)])
def test_head_dims_and_ragged_grids(B, S, H, D):
    _check_full(B, S, H, D)


def test_rectangular_q_kv():
    _check_full(1, 256, 2, 128, seqlen_kv=640)
    _check_full(2, 512, 2, 64, seqlen_kv=128)


@pytest.mark.parametrize("B,S,H,D,Skv", [(1, 128, 1, 64, 64), (1, 128, 1, 128, 64), (2, 256, 2, 128, 192),
                                         (1, 256, 3, 64, 320), (1, 128, 2, 256, 32), (1, 128, 2, 256, 96)])
def test_shortest_and_odd_key_tile_counts(B, S, H, D, Skv):
    # one key tile (the pipeline is prologue + last step only), an odd number of tiles (the loop's other tail), and
    # the smallest problem the tiles allow: one workgroup, one (batch, head)
    _check_full(B, S, H, D, seqlen_kv=Skv)


@pytest.mark.parametrize("B,S,H,D,Skv", [(1, 256, 2, 64, 512), (2, 256, 2, 128, 384), (1, 128, 2, 256, 256), (1, 128, 1, 128, 64)])
def test_scores_that_climb_along_the_keys_move_the_reference_point(B, S, H, D, Skv):
    # the deferred rescale's slow path, many times per row; single-tile case: the reference point is only set
    _check_full(B, S, H, D, seqlen_kv=Skv, climb=True)


def test_integer_valued_inputs():
    _check_full(1, 256, 2, 64, kind="uniform_int")


def test_exact_arithmetic_pins_operand_layouts():
    # integer scores with scale*log2e = 1: P is a power of two (exact in fp16), V integer: only the fp16 output
    # rounds, so a wrong key <-> V-row association or a transposed operand cannot hide inside the tolerance
    rng = np.random.default_rng(11)
    for D in (64, 128, 256):
        B, S, H = 1, 384, 2
        q = np.zeros((B, S, H, D), np.float32)
        np.put_along_axis(q, rng.integers(0, D, (B, S, H, 4)), 1.0, axis=-1)
        k = rng.integers(-1, 2, (B, S, H, D)).astype(np.float32)
        v = rng.integers(-8, 9, (B, S, H, D)).astype(np.float32)
        got, (qf, kf, vf) = _run(q, k, v, softmax_scale=float(np.log(2.0)))
        ref = oracle.attention_f32(qf, kf, vf, alpha0=np.log(2.0))["O"]
        np.testing.assert_allclose(got, ref, rtol=1.5e-3, atol=2e-4)


def test_nondefault_scale():
    _check_full(1, 256, 2, 128, scale=0.05)


def test_row_max_and_row_sum_taps():
    # the reference's max-check / sum-check (fmha_forward.cu:655-676): kernel max is in the log2 domain,
    # kernel sum is not reciprocal
    import torch
    B, S, H, D = 2, 256, 2, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    rm = torch.full((B, H, S), -1.0, dtype=torch.float32, device="cuda:0")
    rs = torch.full((B, H, S), -1.0, dtype=torch.float32, device="cuda:0")
    got, (qf, kf, vf) = _run(q, k, v, row_max=rm, row_sum=rs)
    r = oracle.attention_f32(qf, kf, vf, want_stats=True)
    assert max_abs(got, r["O"]) <= TOL_FP16
    mi = rm.cpu().numpy() / oracle.LOG2E
    assert oracle.verify_tensor(mi, r["row_max"])[0]
    assert oracle.verify_tensor(1.0 / rs.cpu().numpy(), r["inv_sum"])[0]
    np.testing.assert_allclose(mi, r["row_max"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(1.0 / rs.cpu().numpy(), r["inv_sum"], rtol=1e-4)


@pytest.mark.parametrize("D,S", [(64, 256), (128, 256), (256, 256), (128, 160), (256, 96)])
def test_score_tap(D, S):
    # the reference's gemm-check-1 (fmha_forward.cu:640-653): pre-softmax scores against the oracle's, exact
    # products of fp16 values accumulated in fp32 (160 and 96 query rows: a last query tile that is partly filled)
    import torch
    B, H, Skv = 2, 2, 256
    q, k, v = pkg.testbed.qkv(B, S, H, D, seqlen_kv=Skv)
    sc = torch.full((B, H, S, Skv), -1.0, dtype=torch.float32, device="cuda:0")
    got, (qf, kf, vf) = _run(q, k, v, scores=sc)
    r = oracle.attention_f32(qf, kf, vf, want_scores=True)
    assert max_abs(got, r["O"]) <= TOL_FP16
    assert oracle.verify_tensor(sc.cpu().numpy(), r["S"])[0]
    np.testing.assert_allclose(sc.cpu().numpy(), r["S"], rtol=1e-4, atol=1e-4)


def test_kernel_matches_tiled_emulation_closely():
    # against the numpy emulation of the kernel-side algorithm (P rounded to fp16 per tile) the difference is
    # rounding noise of the fp16 output only
    B, S, H, D = 1, 256, 1, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    got, (qf, kf, vf) = _run(q, k, v)
    bn = pkg.fmha_forward_plan(pkg.CFK_FP16, B, H, S, S, D)[1]
    emu, _, _ = oracle.online_softmax_tiled(qf[0, :, 0], kf[0, :, 0], vf[0, :, 0], bn, oracle.LOG2E / np.sqrt(D))
    assert max_abs(got[0, :, 0], emu) <= 6e-4


def test_invariants_on_device():
    import torch
    B, S, H, D = 1, 512, 4, 128
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    base, _ = _run(q, k, v)
    # V = 1 -> O = 1 (rows of P sum to one)
    ones, _ = _run(q, k, np.ones_like(v))
    assert max_abs(ones, 1.0) <= 1e-3
    # a common permutation of the keys changes nothing beyond rounding
    perm = np.random.default_rng(5).permutation(S)
    permd, _ = _run(q, k[:, perm], v[:, perm])
    assert max_abs(base, permd) <= 1e-3
    # Q = 0 -> mean of V
    zero, (_, _, vf) = _run(np.zeros_like(q), k, v)
    assert max_abs(zero, np.broadcast_to(vf.mean(axis=1, keepdims=True), vf.shape)) <= 1e-3
    # output buffer is fully overwritten (the driver pre-fills O with -1, fmha_forward.cu:501-502)
    o = torch.full((B, S, H, D), -1.0, dtype=torch.float16, device="cuda:0")
    pkg.fmha_forward(to_dev(q.astype(np.float16)), to_dev(k.astype(np.float16)), to_dev(v.astype(np.float16)), o=o)
    torch.cuda.synchronize()
    assert max_abs(o.float().cpu().numpy(), base) == 0.0


def _subset_check(B, S, H, D, climb=False, **climb_kw):
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    if climb:
        k, v = climbing_keys(k, **climb_kw), v / 4
    got, (qf, kf, vf) = _run(q, k, v)
    pairs = subset_pairs(B, H)
    ref = oracle.attention_f32(qf, kf, vf, bh_pairs=pairs)["O"]
    all_pairs = [(b, h) for b in range(B) for h in range(H)]
    oracle.attention_f32(qf, kf, vf, bh_pairs=all_pairs, row_start=17, row_step=61, out=ref)
    sel = ~np.isnan(ref)
    assert sel.sum() >= len(pairs) * S * D
    err = max_abs(got[sel], ref[sel])
    ok, pct = oracle.verify_tensor(got[sel], ref[sel], ERRPCT_FP16)
    print(f"fp16 B={B} S={S} H={H} D={D}: checked {sel.sum()} elements, max-abs {err:.3e}, error% {pct:.2e}")
    assert err <= TOL_FP16 and ok
    assert not np.any(np.isnan(got)) and float(np.abs(got).max()) < 10.0


def test_config2_headline_shape_subset_check():
    # benchmark configuration 2: B=8 H=16 S=2048 D=128; four full (b,h) slices + every 61st row of every head
    _subset_check(8, 2048, 16, 128)


def test_headline_shapes_with_climbing_scores():
    # the kernels big problems get (256- and 128-row tiles on 16x16x32 MFMAs), on keys that keep moving the softmax
    # reference point
    _subset_check(8, 2048, 16, 128, climb=True)
    _subset_check(4, 2048, 16, 64, climb=True)


@pytest.mark.parametrize("B,S,H,D,ramp", [(8, 1024, 16, 128, 8.0), (8, 1024, 16, 128, 4.5), (4, 2048, 16, 64, 8.0),
                                          (2, 8192, 8, 256, 8.0)])
def test_weights_beyond_fp16_but_within_fp32(B, S, H, D, ramp):
    # No spike key: the scores climb 15 to 35 binades above the first tile's row max, so the weights taken against that
    # fixed reference point overflow fp16 (P) but not fp32 -- a sum of the fp32 weights stays finite, and the test that
    # sends a workgroup to the max-tracking loop has to go by its size.  Ramp 4.5: only some rows get that far.
    assert "kernel16p<" in pkg.fmha_forward_kernel(pkg.CFK_FP16, B, H, S, S, D)     # the fixed reference point is theirs
    _subset_check(B, S, H, D, climb=True, ramp=ramp, spike=1.0)


@pytest.mark.parametrize("scale", [1e-4, 0.012, 0.65, 12.0])
def test_unusual_softmax_scales_on_the_hand_scheduled_kernel(scale):
    # The hand-scheduled loops multiply Q by scale * log2(e) in fp16; scales that would push that product towards the
    # ends of the fp16 range are served by the kernel's other loop (0.012 * log2 e sits just above the limit of 2^-6,
    # 1e-4 below it; 0.65 * log2 e just below the limit of 1, 12 * log2 e above it: a softmax that is a hard max).
    B, S, H, D = 8, 1024, 16, 128
    assert "kernel16p<" in pkg.fmha_forward_kernel(pkg.CFK_FP16, B, H, S, S, D)
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    got, (qf, kf, vf) = _run(q, k, v, softmax_scale=scale)
    ref = oracle.attention_f32(qf, kf, vf, alpha0=scale, bh_pairs=[(0, 0), (B - 1, H - 1)])["O"]
    sel = ~np.isnan(ref)
    err = max_abs(got[sel], ref[sel])
    print(f"fp16 B={B} S={S} H={H} D={D} scale={scale}: max-abs {err:.3e}")
    # (a hard max returns single rows of V: the fp16 rounding of |O| up to 4.5 is 2e-3 by itself)
    assert err <= (TOL_FP16 if scale < 0.5 else 2.5e-3) and not np.isnan(got).any()


@pytest.mark.parametrize("B,S,H,D", [(1, 32768, 2, 128), (1, 32768, 3, 64), (1, 16384, 2, 256), (1, 65536, 1, 128)])
def test_very_long_sequences(B, S, H, D):
    # 256 to 1024 key tiles per work item: 64-bit tile addresses, row sums over tens of thousands of weights against one
    # fixed reference point; every 1531st row of every head against the oracle
    q, k, v = pkg.testbed.qkv(B, S, H, D)
    got, (qf, kf, vf) = _run(q, k, v)
    ref = np.full(got.shape, np.nan, np.float32)
    oracle.attention_f32(qf, kf, vf, bh_pairs=[(b, h) for b in range(B) for h in range(H)], row_start=5, row_step=1531, out=ref)
    sel = ~np.isnan(ref)
    err = max_abs(got[sel], ref[sel])
    print(f"fp16 B={B} S={S} H={H} D={D}: checked {sel.sum()} elements, max-abs {err:.3e}")
    assert sel.sum() >= (S // 1531) * H * D and err <= TOL_FP16 and np.isfinite(got).all()


def test_config3_long_sequence_large_head_subset_check():
    # benchmark configuration 3: B=2 H=8 S=8192 D=256
    _subset_check(2, 8192, 8, 256)
