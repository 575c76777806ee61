"""GPU parity of the dense GEMM (secondary bench, same tile engine) against the CPU oracle.
The reference checks its GEMM examples by equality on integer-valued inputs
(src/cutlass-gemm/gemm.cu:277-294, 329-359; src/cute-gemm-tma-gma/gemm.cu:645-651); so does this."""
import numpy as np
import pytest

import oracle
from _util import pkg, to_dev

pytestmark = pytest.mark.gpu


def _run(a, b, layout):
    import torch
    c = pkg.gemm_f16(to_dev(a.astype(np.float16)), to_dev(b.astype(np.float16)), layout=layout)
    torch.cuda.synchronize()
    return c.cpu().numpy()


@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 768, 320), (1024, 256, 1024)])
def test_integer_inputs_bit_exact(M, N, K, layout):
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-8, 9, (M, K)).astype(np.float32)
    b = rng.integers(-8, 9, (N, K)).astype(np.float32)       # logical B^T: b[n, k]
    want = oracle.gemm_f32(a, b).astype(np.float16)           # exact fp32 sums, one RNE rounding to fp16
    got = _run(a, b if layout == 0 else np.ascontiguousarray(b.T), layout)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("layout", [0, 1])
def test_uniform_inputs(layout):
    M, N, K = 512, 512, 2048
    a = pkg.testbed.uniform((M, K), 1).astype(np.float16)
    b = pkg.testbed.uniform((N, K), 2).astype(np.float16)
    want = oracle.gemm_f32(a.astype(np.float32), b.astype(np.float32))
    got = _run(a, b if layout == 0 else np.ascontiguousarray(b.T), layout).astype(np.float32)
    # fp32 accumulation in a different order + one fp16 rounding of |c| <~ 60
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)


def test_config5_row_sample():
    # benchmark configuration 5: M=N=K=8192, U(-1,1) fp16, fp32 accumulate, fp16 C; 24 sampled rows against the oracle
    import torch
    M = N = K = 8192
    a = pkg.testbed.uniform((M, K), 3).astype(np.float16)
    b = pkg.testbed.uniform((N, K), 4).astype(np.float16)
    c = pkg.gemm_f16(to_dev(a), to_dev(b))
    torch.cuda.synchronize()
    rows = np.sort(np.random.default_rng(9).choice(M, 24, replace=False)).astype(np.int32)
    rows[0], rows[-1] = 0, M - 1
    want = oracle.gemm_f32(a.astype(np.float32), b.astype(np.float32), rows=rows)
    got = c[torch.from_numpy(rows).long().cuda()].float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=1e-2)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_alpha_beta_batch_integer_inputs_bit_exact(dtype):
    # the CUTLASS-API example's run: D = alpha * A.B + beta * C on integer-valued operands in [-8, 8], checked for
    # EQUALITY (src/cutlass-gemm/gemm.cu:277-294, 318-359); plus the CuTe example's batch count L (gemm.cu:519-521).
    # Everything is an integer below 2^24 in fp32, so alpha = 2, beta = -3 keep the result exact before the final
    # rounding to the output type.
    import torch
    L, M, N, K = 3, 256, 512, 192
    rng = np.random.default_rng(17)
    a = rng.integers(-8, 9, (L, M, K)).astype(np.float32)
    b = rng.integers(-8, 9, (L, N, K)).astype(np.float32)
    c = rng.integers(-8, 9, (L, M, N)).astype(np.float32)
    want = np.stack([2.0 * oracle.gemm_f32(a[i], b[i]) - 3.0 * c[i] for i in range(L)]).astype(dtype)
    got = pkg.gemm(to_dev(a.astype(dtype)), to_dev(b.astype(dtype)), c=to_dev(c.astype(dtype)), alpha=2.0, beta=-3.0)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    # beta = 0 must not read C (NaNs there would otherwise leak), and D may alias C
    cn = to_dev(np.full((L, M, N), np.nan, dtype))
    got = pkg.gemm(to_dev(a.astype(dtype)), to_dev(b.astype(dtype)), c=cn, alpha=1.0, beta=0.0, out=cn)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), np.stack([oracle.gemm_f32(a[i], b[i]) for i in range(L)]).astype(dtype))


def test_fp32_uniform_inputs():
    # the CuTe example's type 1 (float operands, gemm.cu:677-684), U(-1,1) data (:482-485).  Both sides accumulate in
    # fp32 in different orders: |error| <~ sqrt(K) * 2^-24 * |terms|
    import torch
    M, N, K = 512, 256, 4096
    a = pkg.testbed.uniform((M, K), 5).astype(np.float32)
    b = pkg.testbed.uniform((N, K), 6).astype(np.float32)
    want = oracle.gemm_f32(a, b)
    got = pkg.gemm(to_dev(a), to_dev(b))
    torch.cuda.synchronize()
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-4, atol=2e-4)
    # pins the contraction-slot mapping of the fp32 path against a float64 product on a few rows
    ref64 = a[:8].astype(np.float64) @ b.astype(np.float64).T
    np.testing.assert_allclose(got[:8].cpu().numpy(), ref64, rtol=1e-4, atol=2e-4)


def test_error_paths():
    import torch
    x = torch.zeros((100, 64), dtype=torch.float16, device="cuda:0")
    with pytest.raises(pkg.CfkError) as e:
        pkg.gemm_f16(x, x)
    assert e.value.code == -2
    xf = torch.zeros((256, 64), dtype=torch.float32, device="cuda:0")
    with pytest.raises(pkg.CfkError) as e:      # the N-contiguous B layout is an fp16 layout
        pkg.gemm(xf, torch.zeros((64, 256), dtype=torch.float32, device="cuda:0"), layout=1)
    assert e.value.code == -2
