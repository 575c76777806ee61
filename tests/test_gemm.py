"""GPU parity of the dense fp16 GEMM (secondary bench, same tile engine) against the CPU oracle.
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
    # BASELINE config 5: M=N=K=8192, U(-1,1) fp16, fp32 accumulate, fp16 C; 24 sampled rows against the oracle
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


def test_error_paths():
    import torch
    x = torch.zeros((100, 64), dtype=torch.float16, device="cuda:0")
    with pytest.raises(pkg.CfkError) as e:
        pkg.gemm_f16(x, x)
    assert e.value.code == -2
