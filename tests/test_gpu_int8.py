"""GPU parity tests of the int8 values variant: HIP compressor bit-exact against the CPU oracle,
products within |err| <= 1e-3 + 1e-2 * |want| of the dense float64 product, through the torch
operators and directly through the C ABI.
"""
import ctypes

import numpy as np
import pytest
import torch

import macko_spmv_amd as mk
from oracle import macko_oracle as mo
from tests import helpers

pytestmark = pytest.mark.gpu


def _random_int8(rng, rows, cols, density):
    m = rng.integers(-128, 128, (rows, cols)).astype(np.int8)
    m[rng.random((rows, cols)) >= density] = 0
    return m


def _assert_bit_exact(compressed, dense_np):
    want = mo.compress_int8(dense_np)
    values, deltas, row_ptr = (t.cpu().numpy() for t in compressed[:3])
    assert compressed[3] == dense_np.shape[0] and compressed[4] == dense_np.shape[1]
    assert np.array_equal(row_ptr, want[2]), "row_indices differ"
    assert values.dtype == np.int8 and values.shape == want[0].shape and np.array_equal(values, want[0])
    assert deltas.shape == want[1].shape and np.array_equal(deltas, want[1]), "deltas differ"


@pytest.mark.parametrize("device", ["cpu", "cuda"])
def test_compressor_small_shapes(device):
    rng = np.random.default_rng(2024)
    for _ in range(60):
        rows = int(rng.integers(1, 40))
        cols = int(rng.integers(1, 1500))
        dense = _random_int8(rng, rows, cols, float(rng.choice([0, 0.003, 0.02, 0.1, 0.3, 0.5, 0.9, 1.0])))
        c = mk.compress_int8(torch.from_numpy(dense).to(device))
        assert c[0].device.type == device
        _assert_bit_exact(c, dense)


@pytest.mark.parametrize("gap", [14, 15, 16, 17, 31, 32, 33, 511, 512, 513, 1023, 1024])
def test_compressor_gap_edges(gap):
    dense = np.zeros((4, 1100), dtype=np.int8)
    dense[0, 0] = 1
    dense[0, min(gap + 1, 1099)] = 2
    dense[1, min(gap, 1099)] = 3
    dense[2, 1099 - min(gap, 1099)] = 4
    _assert_bit_exact(mk.compress_int8(torch.from_numpy(dense).cuda()), dense)


@pytest.mark.parametrize("shape,density", [((1024, 4096), 0.5), ((333, 4099), 0.1), ((4096, 515), 0.02),
                                           ((64, 20000), 0.3), ((512, 1024), 0.0)])
def test_compressor_mid_shapes(shape, density):
    rng = np.random.default_rng(5)
    dense = _random_int8(rng, shape[0], shape[1], density)
    _assert_bit_exact(mk.compress_int8(torch.from_numpy(dense).cuda()), dense)


def _check_product(dense, x, compressed=None):
    c = compressed if compressed is not None else mk.compress_int8(torch.from_numpy(dense).cuda())
    y = mk.multiply_int8(c, torch.from_numpy(x).cuda())
    assert y.dtype == torch.float16 and y.shape == (dense.shape[0],)
    want = dense.astype(np.float64) @ x.astype(np.float64)[: dense.shape[1]]
    helpers.assert_close_fp16(y.cpu().numpy(), want)
    return c, y


@pytest.mark.parametrize("shape,density", [((1, 1), 1.0), ((3, 17), 0.5), ((65, 511), 0.3), ((64, 513), 0.9),
                                           ((1000, 1000), 0.05), ((4096, 4096), 0.5), ((11008, 4096), 0.1),
                                           ((4096, 11008), 0.3), ((37, 30000), 0.2), ((20000, 64), 0.5), ((5, 90000), 0.1),
                                           ((256, 2048), 0.0)])
def test_multiply_against_dense_float64(shape, density):
    rng = np.random.default_rng(shape[0] * 31 + shape[1])
    dense = _random_int8(rng, shape[0], shape[1], density)
    x = (rng.standard_normal(shape[1]) * 0.01).astype(np.float16)
    _check_product(dense, x)


def test_multiply_matches_oracle_and_keeps_trailing_padding():
    rng = np.random.default_rng(3)
    dense = _random_int8(rng, 300, 700, 0.1)
    dense[5] = 0  # an all-zero row still stores 43 padding entries
    x = (rng.standard_normal(700) * 0.01).astype(np.float16)
    c, y = _check_product(dense, x)
    row_ptr = c[2].cpu().numpy()
    assert row_ptr[6] - row_ptr[5] == 700 // 16
    values, deltas = c[0].cpu().numpy(), c[1].cpu().numpy()
    want = mo.spmv_int8(values, deltas, row_ptr, 300, 700, x).view(np.float16)
    # same fp32 accumulation, different summation order
    assert np.allclose(y.cpu().numpy().astype(np.float32), want.astype(np.float32), rtol=1e-2, atol=1e-3)


def test_multiply_axpby_and_c_abi():
    rng = np.random.default_rng(8)
    rows, cols = 777, 3001
    dense = _random_int8(rng, rows, cols, 0.25)
    x = (rng.standard_normal(cols) * 0.01).astype(np.float16)
    y0 = rng.standard_normal(rows).astype(np.float16)
    c = mk.compress_int8(torch.from_numpy(dense).cuda())
    want = dense.astype(np.float64) @ x.astype(np.float64)
    C = torch.from_numpy(y0.copy()).cuda()
    out = mk.multiply_int8_axpby(c, torch.from_numpy(x).cuda(), C, alpha=0.5, beta=-2.0)
    assert out.data_ptr() == C.data_ptr()
    helpers.assert_close_fp16(C.cpu().numpy(), 0.5 * want - 2.0 * y0.astype(np.float64))

    # the same product straight through the C ABI
    lib = ctypes.CDLL(mk.HIP_LIBRARY_PATH)
    vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
    lib.macko_spmv_i8f16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i64, vp]
    lib.macko_compress_i8_count.argtypes = [vp, i32, i32, vp, vp]
    lib.macko_compress_i8_fill.argtypes = [vp, i32, i32, vp, vp, vp, i64, vp]
    stream = torch.cuda.current_stream().cuda_stream
    M = torch.from_numpy(dense).cuda()
    row_ptr = torch.empty(rows + 1, dtype=torch.int32, device="cuda")
    assert lib.macko_compress_i8_count(M.data_ptr(), rows, cols, row_ptr.data_ptr(), stream) == 0
    n = int(row_ptr[rows].item())
    P = (n + 7) // 8 * 8
    values = torch.full((P,), 99, dtype=torch.int8, device="cuda")      # garbage on purpose:
    deltas = torch.full((P // 2,), 0xAB, dtype=torch.uint8, device="cuda")  # fill overwrites all of it
    assert lib.macko_compress_i8_fill(M.data_ptr(), rows, cols, row_ptr.data_ptr(), values.data_ptr(),
                                      deltas.data_ptr(), P, stream) == 0
    assert torch.equal(values, c[0]) and torch.equal(deltas, c[1]) and torch.equal(row_ptr, c[2])
    xg = torch.from_numpy(x).cuda()
    y = torch.empty(rows, dtype=torch.float16, device="cuda")
    assert lib.macko_spmv_i8f16(values.data_ptr(), deltas.data_ptr(), row_ptr.data_ptr(), xg.data_ptr(),
                                y.data_ptr(), rows, cols, P, stream) == 0
    torch.cuda.synchronize()
    helpers.assert_close_fp16(y.cpu().numpy(), want)
    # misaligned values pointer is rejected before anything is launched
    assert lib.macko_spmv_i8f16(values.data_ptr() + 1, deltas.data_ptr(), row_ptr.data_ptr(), xg.data_ptr(),
                                y.data_ptr(), rows, cols, P, stream) == -1


def test_linearity_full_size():
    # size-independent property at a full Llama shape: M(a*x1 + x2) = a*M x1 + M x2 within tolerance
    torch.manual_seed(0)
    rows, cols = 11008, 4096
    M = torch.randint(-127, 128, (rows, cols), dtype=torch.int8, device="cuda")
    M[torch.rand((rows, cols), device="cuda") > 0.5] = 0
    c = mk.compress_int8(M)
    x1 = (torch.randn(cols, device="cuda") * 0.01).half()
    x2 = (torch.randn(cols, device="cuda") * 0.01).half()
    y1 = mk.multiply_int8(c, x1).float()
    y2 = mk.multiply_int8(c, x2).float()
    y12 = mk.multiply_int8(c, (2 * x1.float() + x2.float()).half()).float()
    ref = M.float() @ (2 * x1.float() + x2.float()).half().float()
    assert torch.allclose(y12, ref, rtol=1e-2, atol=2e-3 * ref.abs().max().item())
    assert torch.allclose(y12, 2 * y1 + y2, rtol=2e-2, atol=5e-3 * ref.abs().max().item())
