"""GPU tests of the products that build their input vector while staging it: y = M rmsnorm(x) and
y = a M (silu(gate) * up) + b y.  Checked against (1) the dense float64 product of the same fp16
matrix with the fp16-rounded intermediate vector computed on the host, to the product's stated
tolerance |err| <= 1e-3 + 1e-2 * |want|, and (2) the unfused composition of the separate kernels.
"""
import ctypes

import numpy as np
import pytest
import torch

import macko_spmv
import macko_spmv_amd
from tests import helpers

pytestmark = pytest.mark.gpu


def _rmsnorm_host(x, w, eps):
    xf = x.astype(np.float64)
    inv = 1.0 / np.sqrt((xf * xf).mean() + eps)
    return (xf * inv * w.astype(np.float64)).astype(np.float16)


def _silu_mul_host(g, u):
    gf = g.astype(np.float64)
    return (gf / (1.0 + np.exp(-gf)) * u.astype(np.float64)).astype(np.float16)


SHAPES = [((1, 8), 1.0), ((5, 64), 0.5), ((300, 1000), 0.3), ((4096, 4096), 0.5), ((12288, 4096), 0.1),
          ((22016, 4096), 0.5), ((4096, 11008), 0.5), ((4096, 11008), 0.1), ((37, 30000), 0.2), ((20000, 64), 0.5),
          ((64, 512), 0.0)]


@pytest.mark.parametrize("shape,density", SHAPES)
def test_multiply_rmsnorm(shape, density):
    rows, cols = shape
    rng = np.random.default_rng(rows * 7 + cols)
    dense = helpers.row_pruned(rng, rows, cols, density) if rows * cols > 1 << 20 else \
        helpers.random_sparse(rng, rows, cols, density)
    x = rng.standard_normal(cols).astype(np.float16)
    w = (1.0 + 0.1 * rng.standard_normal(cols)).astype(np.float16)
    eps = 1e-5
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    xg, wg = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    print("rmsnorm case", shape, density, flush=True)
    y = macko_spmv.multiply_rmsnorm(c, xg, wg, eps)
    assert y.shape == (rows,) and y.dtype == torch.float16
    # the fp16 rounding of the normalised vector may differ from the host's in the last bit of a
    # few elements (fp32 vs float64 sum of squares): that is far inside the product's tolerance
    want = helpers.dense_reference(dense, _rmsnorm_host(x, w, eps))
    helpers.assert_close_fp16(y.cpu().numpy(), want)
    # against the separate kernels
    unfused = macko_spmv.multiply(c, torch.ops.macko_spmv.decode_rmsnorm(xg, wg, eps))
    assert torch.allclose(y.float(), unfused.float(), rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("shape,density", SHAPES)
def test_multiply_silu_mul_axpby(shape, density):
    rows, cols = shape
    rng = np.random.default_rng(rows * 11 + cols)
    dense = helpers.row_pruned(rng, rows, cols, density) if rows * cols > 1 << 20 else \
        helpers.random_sparse(rng, rows, cols, density)
    gu = rng.standard_normal(2 * cols).astype(np.float16)
    y0 = rng.standard_normal(rows).astype(np.float16)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    gug = torch.from_numpy(gu).cuda()
    gate, up = gug[:cols], gug[cols:]
    print("silu case", shape, density, flush=True)
    product = helpers.dense_reference(dense, _silu_mul_host(gu[:cols], gu[cols:]))
    # plain product: y is not read (filled with NaN to prove it)
    C = torch.full((rows,), float("nan"), dtype=torch.float16, device="cuda")
    out = macko_spmv.multiply_silu_mul_axpby(c, gate, up, C)
    assert out.data_ptr() == C.data_ptr()
    helpers.assert_close_fp16(C.cpu().numpy(), product)
    # same vector as the separate kernel builds, so the same sums in the same order; except for
    # matrices of short rows, where the plain product adds a row's entries in another order (it works
    # all the rows of a tile in one pass; the fused entry points have no such variant)
    unfused = macko_spmv.multiply(c, torch.ops.macko_spmv.decode_silu_mul(gate, up))
    if c[0].numel() >= 192 * rows:
        assert torch.equal(C, unfused)
    else:
        assert torch.allclose(C.float(), unfused.float(), rtol=2e-3, atol=2e-4)
    # with the residual folded in
    C = torch.from_numpy(y0.copy()).cuda()
    macko_spmv.multiply_silu_mul_axpby(c, gate, up, C, alpha=0.5, beta=-2.0)
    helpers.assert_close_fp16(C.cpu().numpy(), 0.5 * product - 2.0 * y0.astype(np.float64), rel=1e-2, abs_=4e-3)


def test_fused_input_argument_checks_and_c_abi():
    lib = ctypes.CDLL(macko_spmv_amd.HIP_LIBRARY_PATH)
    vp, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float
    lib.macko_spmv_f16_rmsnorm.argtypes = [vp, vp, vp, vp, vp, f32, vp, i32, i32, i64, vp]
    lib.macko_spmv_f16_silu_mul_axpby.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i64, f32, f32, vp]
    rng = np.random.default_rng(5)
    rows, cols = 200, 1024
    dense = helpers.random_sparse(rng, rows, cols, 0.3)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    x = torch.from_numpy(rng.standard_normal(cols + 8).astype(np.float16)).cuda()
    w = torch.ones(cols + 8, dtype=torch.float16, device="cuda")
    y = torch.empty(rows, dtype=torch.float16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    P = c[0].numel()

    def rms(xp, wp, n_cols=cols):
        return lib.macko_spmv_f16_rmsnorm(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), xp, wp, 1e-5,
                                          y.data_ptr(), rows, n_cols, P, stream)

    assert rms(x.data_ptr(), w.data_ptr()) == 0
    torch.cuda.synchronize()
    want = helpers.dense_reference(dense, _rmsnorm_host(x[:cols].cpu().numpy(), w[:cols].cpu().numpy(), 1e-5))
    helpers.assert_close_fp16(y.cpu().numpy(), want)
    assert rms(x.data_ptr() + 2, w.data_ptr()) == -1          # x not 16-byte aligned
    assert rms(x.data_ptr(), w.data_ptr() + 8) == -1          # weight not 16-byte aligned
    assert rms(x.data_ptr(), None) == -1
    assert lib.macko_spmv_f16_silu_mul_axpby(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), x.data_ptr(),
                                             w.data_ptr() + 4, y.data_ptr(), rows, cols, P, 1.0, 0.0, stream) == -1
    # a column count that is not a multiple of 8 is refused by the operator as well
    odd = macko_spmv.compress(torch.from_numpy(helpers.random_sparse(rng, 10, 1004, 0.3)).cuda())
    with pytest.raises(RuntimeError):
        macko_spmv.multiply_rmsnorm(odd, x[:1004].contiguous(), w[:1004].contiguous(), 1e-5)
    # a vector too long for LDS is refused
    wide = macko_spmv.compress(torch.from_numpy(helpers.random_sparse(rng, 4, 90000, 0.01)).cuda())
    xl = torch.zeros(90000, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        macko_spmv.multiply_rmsnorm(wide, xl, xl, 1e-5)
