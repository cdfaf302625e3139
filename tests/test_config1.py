"""The CPU-runnable benchmark case (a single 4096 x 4096 fp16 matrix, values N(0, 0.02), unstructured
Bernoulli mask at density 0.5, torch CPU generator seed 0, x ~ N(0, 1) fp16): compress + multiply
through the CPU oracle against the dense fp32-accumulated product, and the HIP path against the
oracle on the same input (compressed arrays bit-exact, product within |err| <= 1e-3 + 1e-2 |want|).
"""
import numpy as np
import pytest
import torch

from oracle import macko_oracle as mo
from tests import helpers


def _inputs():
    g = torch.Generator(device="cpu")
    g.manual_seed(0)
    W = (torch.randn((4096, 4096), generator=g) * 0.02).half()
    W[torch.rand((4096, 4096), generator=g) >= 0.5] = 0
    x = torch.randn(4096, generator=g).half()
    return W.contiguous(), x


def test_cpu_path_against_dense_fp32_accumulation():
    W, x = _inputs()
    dense, xv = W.numpy(), x.numpy()
    values, deltas, row_ptr, n = mo.compress(dense)
    assert row_ptr[0] == 0 and row_ptr[-1] == n and len(values) == (n + 7) // 8 * 8
    # expected entry count: one per non-zero plus one padding entry per 16 zeros inside a gap
    assert abs(n - 8.39e6) < 0.02e6
    y = mo.spmv(values, deltas, row_ptr, 4096, 4096, xv).view(np.float16)
    want32 = (W.float() @ x.float()).numpy()            # dense, fp32 accumulation
    assert np.allclose(y.astype(np.float32), want32, rtol=1e-2, atol=1e-3)
    helpers.assert_close_fp16(y, helpers.dense_reference(dense, xv))


@pytest.mark.gpu
def test_hip_path_against_the_oracle():
    import macko_spmv

    W, x = _inputs()
    dense, xv = W.numpy(), x.numpy()
    want = mo.compress(dense)
    for device in ("cuda", "cpu"):
        c = macko_spmv.compress(W.to(device))
        assert np.array_equal(c[2].cpu().numpy(), want[2])
        assert np.array_equal(c[0].cpu().numpy().view(np.uint16), want[0])
        assert np.array_equal(c[1].cpu().numpy(), want[1])
    c = macko_spmv.compress(W.cuda())
    y = macko_spmv.multiply(c, x.cuda()).cpu().numpy()
    oracle_y = mo.spmv(want[0], want[1], want[2], 4096, 4096, xv).view(np.float16)
    assert np.allclose(y.astype(np.float32), oracle_y.astype(np.float32), rtol=1e-2, atol=1e-3)
    helpers.assert_close_fp16(y, helpers.dense_reference(dense, xv))
