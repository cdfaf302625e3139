"""GPU parity tests: the HIP path against the CPU oracle, the upstream known-answer vectors and
size-independent properties.  Everything here calls the product through the C ABI -- directly
with ctypes, or through the torch operator that forwards to it.

Bars: compressed arrays bit-exact; products within |err| <= 1e-3 + 1e-2 * |want| of the dense
float64 product of the same fp16 data (the tolerance stated for this path), and within
rtol = atol = 1e-3 of torch's fp16 dense product where the upstream tests use that bar.
"""
import ctypes

import numpy as np
import pytest
import torch

import macko_spmv
import macko_spmv_amd
from oracle import macko_numpy as mn
from oracle import macko_oracle as mo
from tests import helpers

pytestmark = pytest.mark.gpu


def _np_tuple(compressed):
    return (compressed[0].cpu().numpy().view(np.uint16), compressed[1].cpu().numpy(),
            compressed[2].cpu().numpy(), compressed[3], compressed[4])


def _assert_bit_exact(compressed, dense_np):
    values, deltas, row_ptr, rows, cols = _np_tuple(compressed)
    want = mo.compress(dense_np)
    assert rows == dense_np.shape[0] and cols == dense_np.shape[1]
    assert np.array_equal(row_ptr, want[2]), "row_indices differ"
    assert values.shape == want[0].shape and np.array_equal(values, want[0]), "values differ"
    assert deltas.shape == want[1].shape and np.array_equal(deltas, want[1]), "deltas differ"


# ---- compressor ----------------------------------------------------------------------------

@pytest.mark.parametrize("device", ["cpu", "cuda"])
@pytest.mark.parametrize("case", helpers.load_kat(), ids=lambda c: c["name"])
def test_compressor_known_answers(case, device):
    # tests/test_macko_spmv.py:43-103 of the upstream package, both device routes
    M = torch.from_numpy(case["dense"]).to(device)
    compressed = macko_spmv.compress(M)
    assert len(compressed) == 5
    assert compressed[0].device.type == device and compressed[0].dtype == torch.float16
    assert compressed[1].dtype == torch.uint8 and compressed[2].dtype == torch.int32
    assert torch.equal(compressed[0].cpu(), torch.from_numpy(case["values"]))
    assert torch.equal(compressed[1].cpu(), torch.from_numpy(case["deltas"]))
    assert torch.equal(compressed[2].cpu(), torch.from_numpy(case["row_indices"]))
    assert compressed[3] == case["rows"] and compressed[4] == case["cols"]


def test_compressor_bit_exact_small_shapes():
    rng = np.random.default_rng(2024)
    for t in range(120):
        rows = int(rng.integers(1, 40))
        cols = int(rng.integers(1, 1400))
        density = float(rng.choice([0, 0.003, 0.02, 0.1, 0.3, 0.5, 0.9, 1.0]))
        bits = helpers.random_sparse(rng, rows, cols, density).view(np.uint16).copy()
        for special in (0x8000, 0x8000, 0x8000, 0x7E00, 0xFC00, 0x7C00, 0x0001, 0x8001, 0xFE01):
            if rng.random() < 0.5:
                bits[rng.integers(0, rows), rng.integers(0, cols)] = special
        M = torch.from_numpy(bits.view(np.float16)).cuda()
        print("compress case", t, rows, cols, density, flush=True)
        _assert_bit_exact(macko_spmv.compress(M), bits)


@pytest.mark.parametrize("gap", [14, 15, 16, 17, 31, 32, 33, 48, 600])
def test_compressor_gap_edges(gap):
    cols = gap + 40
    m = np.zeros((4, cols), dtype=np.float16)
    m[0, 0] = 1
    m[0, gap + 1] = 2          # exactly `gap` zeros between two non-zeros
    m[1, gap] = 3              # `gap` leading zeros
    m[2, cols - 1 - gap] = 4   # `gap` trailing zeros: no padding entries may remain
    _assert_bit_exact(macko_spmv.compress(torch.from_numpy(m).cuda()), m)


@pytest.mark.parametrize("shape,density", [((512, 4096), 0.5), ((1000, 1111), 0.1), ((333, 8192), 0.3),
                                           ((64, 49152), 0.1), ((2048, 515), 0.02), ((4096, 4096), 0.5)])
def test_compressor_bit_exact_mid_shapes(shape, density):
    rng = np.random.default_rng(hash(shape) & 0xFFFF)
    m = helpers.random_sparse(rng, shape[0], shape[1], density)
    _assert_bit_exact(macko_spmv.compress(torch.from_numpy(m).cuda()), m)


def test_compressor_row_pruned_and_skewed():
    rng = np.random.default_rng(11)
    m = helpers.row_pruned(rng, 512, 4096, 0.1)
    _assert_bit_exact(macko_spmv.compress(torch.from_numpy(m).cuda()), m)
    m, _ = helpers.skewed(rng, 1024, 4096)
    _assert_bit_exact(macko_spmv.compress(torch.from_numpy(m).cuda()), m)


def test_compress_decompress_round_trip_full_size():
    # config-3 size: compress on the GPU, decode on the GPU, compare with the input
    torch.manual_seed(3)
    rows, cols = 28672, 8192
    M = (torch.randn((rows, cols), device="cuda", dtype=torch.float16) * 0.02)
    M = M * (torch.rand((rows, cols), device="cuda") < 0.3)
    M = M.contiguous()
    compressed = macko_spmv.compress(M)
    back = macko_spmv.decompress(compressed)
    # +0.0 turns -0 into +0 (a padding entry keeps the sign of the zero it sits on)
    assert torch.equal((back + 0.0).view(torch.int16), (M + 0.0).view(torch.int16))
    values, deltas, row_ptr = compressed[:3]
    n = int(row_ptr[-1])
    assert values.numel() % 8 == 0 and n <= values.numel() < n + 8 and deltas.numel() * 2 == values.numel()
    assert int(row_ptr[0]) == 0 and bool((row_ptr[1:] >= row_ptr[:-1]).all())
    nnz = int((M != 0).sum())
    pads = int((values[:n] == 0).sum())
    assert n == nnz + pads


# ---- multiply ------------------------------------------------------------------------------

def _check_product(dense_np, x_np, compressed=None, label=""):
    rows, cols = dense_np.shape
    M = torch.from_numpy(dense_np).cuda()
    x = torch.from_numpy(x_np).cuda()
    if compressed is None:
        compressed = macko_spmv.compress(M)
    print("multiply case", label, rows, cols, flush=True)
    y = macko_spmv.multiply(compressed, x)
    assert y.shape == (rows,) and y.dtype == torch.float16 and y.is_cuda
    y_np = y.cpu().numpy()
    helpers.assert_close_fp16(y_np, helpers.dense_reference(dense_np, x_np))
    # and against the oracle product from the same compressed arrays
    values, deltas, row_ptr, _, _ = _np_tuple(compressed)
    y_oracle = mo.spmv(values, deltas, row_ptr, rows, cols, x_np).view(np.float16)
    assert np.allclose(y_np.astype(np.float32), y_oracle.astype(np.float32), rtol=1e-2, atol=1e-3)
    return y


def test_multiply_sample_matrix():
    # tests/test_macko_spmv.py:106-112 (default allclose tolerances against the fp16 dense product)
    case = helpers.load_kat()[0]
    M = torch.from_numpy(case["dense"]).cuda()
    torch.manual_seed(0)
    V = torch.rand((case["cols"],), device="cuda", dtype=torch.float16)
    got = macko_spmv.multiply(macko_spmv.compress(M), V)
    assert torch.allclose(M @ V, got, rtol=1e-3, atol=1e-3)
    want = helpers.dense_reference(case["dense"], V.cpu().numpy())
    helpers.assert_close_fp16(got.cpu().numpy(), want)


@pytest.mark.parametrize("density", [1.0, 0.5, 0.1, 0.01, 0.001, 0.0])
@pytest.mark.parametrize("seed", [0, 1])
def test_multiply_upstream_random_sweep(density, seed):
    # tests/test_macko_spmv.py:115-135: 4096 x 8192, U[0,1) values, rtol = atol = 1e-3 vs fp16 M @ V
    torch.manual_seed(seed)
    M_cpu = torch.rand((4096, 8192), dtype=torch.float16, device="cpu")
    M_cpu[torch.rand_like(M_cpu) > density] = 0
    M = M_cpu.cuda()
    V = torch.rand((8192,), device="cuda", dtype=torch.float16)
    compressed = macko_spmv.compress(M)
    got = macko_spmv.multiply(compressed, V)
    assert torch.allclose(M @ V, got, rtol=1e-3, atol=1e-3), f"Fail at {seed} {density}"
    want = (M_cpu.double() @ V.cpu().double()).numpy()
    helpers.assert_close_fp16(got.cpu().numpy(), want)


def test_all_zero_matrix_gives_empty_arrays_and_zero_product():
    M = torch.zeros((300, 777), dtype=torch.float16, device="cuda")
    M[5, 5] = -0.0
    compressed = macko_spmv.compress(M)
    assert compressed[0].numel() == 0 and compressed[1].numel() == 0
    assert torch.equal(compressed[2].cpu(), torch.zeros(301, dtype=torch.int32))
    V = torch.full((777,), float("inf"), dtype=torch.float16, device="cuda")
    y = macko_spmv.multiply(compressed, V)
    assert y.shape == (300,) and not y.any()


def test_multiply_small_and_ragged_shapes():
    rng = np.random.default_rng(77)
    for t in range(80):
        rows = int(rng.integers(1, 200))
        cols = int(rng.integers(1, 3000))
        density = float(rng.choice([0, 0.005, 0.05, 0.3, 0.5, 1.0]))
        dense = helpers.random_sparse(rng, rows, cols, density, scale=1.0)
        x = rng.standard_normal(cols).astype(np.float16)
        _check_product(dense, x, label=f"ragged{t} d={density}")


@pytest.mark.parametrize("shape", [(4096, 4096), (11008, 4096), (4096, 11008)])
@pytest.mark.parametrize("density", [0.1, 0.5, 0.9])
def test_multiply_llama_shapes_row_pruned(shape, density):
    rng = np.random.default_rng(shape[0] * 7 + int(density * 10))
    dense = helpers.row_pruned(rng, shape[0], shape[1], density)
    x = rng.standard_normal(shape[1]).astype(np.float16)
    _check_product(dense, x, label=f"llama {shape} d={density}")


def test_multiply_long_vector_and_few_rows():
    rng = np.random.default_rng(5)
    for rows, cols, density in [(96, 49152, 0.3), (3, 70000, 0.2), (1, 81000, 1.0), (7, 100000, 0.05)]:
        dense = helpers.random_sparse(rng, rows, cols, density, scale=0.05)
        x = rng.standard_normal(cols).astype(np.float16)
        _check_product(dense, x, label=f"long {rows}x{cols}")


def test_multiply_skewed_rows():
    rng = np.random.default_rng(4)
    dense, _ = helpers.skewed(rng, 14336, 4096)
    x = rng.standard_normal(4096).astype(np.float16)
    _check_product(dense, x, label="skewed 14336x4096")


def test_multiply_rows_of_wildly_different_length():
    rng = np.random.default_rng(8)
    dense = np.zeros((300, 6000), dtype=np.float16)
    for r in range(300):
        k = [0, 1, 2, 7, 8, 9, 63, 64, 65, 511, 512, 513, 1000, 6000][r % 14]
        cols = rng.choice(6000, size=k, replace=False)
        dense[r, cols] = rng.standard_normal(k).astype(np.float16)
    x = rng.standard_normal(6000).astype(np.float16)
    _check_product(dense, x, label="wild")


def test_multiply_rows_not_more_than_waves():
    # ownership by proportional row share: one row per wave, with empty rows in between, few rows
    # over many tiles (most waves idle), and exactly as many rows as the launch has waves
    rng = np.random.default_rng(21)
    for rows, cols, density in [(4096, 600, 0.3), (4096, 3000, 0.05), (300, 40000, 0.3), (4095, 2049, 0.5),
                                (17, 30000, 0.9), (2048, 8192, 0.2)]:
        dense = helpers.random_sparse(rng, rows, cols, density, scale=0.05)
        dense[rng.random(rows) < 0.1] = 0  # empty rows, also first / last now and then
        dense[0] = 0
        x = rng.standard_normal(cols).astype(np.float16)
        _check_product(dense, x, label=f"row share {rows}x{cols}")


def test_multiply_row_lengths_sorted():
    # row lengths grow monotonically, so the proportional row guess is far off for every wave and
    # the search runs through its second window and the 64-ary rounds
    rng = np.random.default_rng(22)
    for rows, cols in [(9000, 2048), (20000, 512), (5000, 4096)]:
        density = np.linspace(0.002, 0.9, rows) ** 2
        dense = (rng.standard_normal((rows, cols), dtype=np.float32) * 0.05).astype(np.float16)
        dense[rng.random((rows, cols)) >= density[:, None]] = 0
        x = rng.standard_normal(cols).astype(np.float16)
        _check_product(dense, x, label=f"sorted rows {rows}x{cols}")
        _check_product(dense[::-1].copy(), x, label=f"sorted rows reversed {rows}x{cols}")


@pytest.mark.parametrize("rows,cols,density", [(257, 1500, 0.3), (4096, 4096, 0.5), (11008, 4096, 0.1),
                                               (64, 20000, 0.2), (300, 515, 0.9), (1000, 70000, 0.05),
                                               (33, 90000, 0.1), (512, 512, 0.0)])
def test_multiply_batched(rows, cols, density):
    # every vector of the batch against the dense float64 product and against the single-vector path;
    # batch sizes cover the 8-, 4-, 2- and 1-vector launches and their combinations, and LDS limits
    # (20000 columns: four vectors per launch; 70000: two; 90000: one)
    rng = np.random.default_rng(rows + cols)
    dense = helpers.random_sparse(rng, rows, cols, density, scale=0.05)
    if rows > 40:
        dense[3] = 0
        dense[-1] = 0
    compressed = macko_spmv.compress(torch.from_numpy(dense).cuda())
    for batch in (1, 2, 3, 4, 5, 7, 8, 9, 15):
        X = rng.standard_normal((batch, cols)).astype(np.float16)
        Xg = torch.from_numpy(X).cuda()
        print("batched case", rows, cols, density, batch, flush=True)
        Y = macko_spmv.multiply_batched(compressed, Xg)
        assert Y.shape == (batch, rows) and Y.dtype == torch.float16
        Y_np = Y.cpu().numpy()
        for b in range(batch):
            helpers.assert_close_fp16(Y_np[b], helpers.dense_reference(dense, X[b]))
            single = macko_spmv.multiply(compressed, Xg[b]).cpu().numpy()
            assert np.allclose(Y_np[b].astype(np.float32), single.astype(np.float32), rtol=1e-2, atol=1e-3)


def test_multiply_batched_strided_through_c_abi():
    # leading dimensions larger than cols / rows, odd ldx (unaligned vectors take the scalar copy)
    rng = np.random.default_rng(77)
    rows, cols, batch, ldx, ldy = 500, 1001, 6, 1013, 512
    dense = helpers.random_sparse(rng, rows, cols, 0.3, scale=0.05)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    X = rng.standard_normal((batch, ldx)).astype(np.float16)
    Xg = torch.from_numpy(X).cuda()
    Yg = torch.full((batch, ldy), 7.0, dtype=torch.float16, device="cuda")
    lib = ctypes.CDLL(macko_spmv_amd.HIP_LIBRARY_PATH)
    vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
    lib.macko_spmv_f16_batched.argtypes = [vp, vp, vp, vp, vp, i32, i32, i64, i32, i64, i64, vp]
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.macko_spmv_f16_batched(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), Xg.data_ptr(), Yg.data_ptr(),
                                    rows, cols, c[0].numel(), batch, ldx, ldy, stream)
    assert rc == 0
    torch.cuda.synchronize()
    Y = Yg.cpu().numpy()
    for b in range(batch):
        helpers.assert_close_fp16(Y[b, :rows], helpers.dense_reference(dense, X[b, :cols]))
    assert (Y[:, rows:] == 7.0).all()  # nothing written past the rows
    # leading dimensions smaller than the matrix are rejected before any launch
    assert lib.macko_spmv_f16_batched(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), Xg.data_ptr(), Yg.data_ptr(),
                                      rows, cols, c[0].numel(), batch, cols - 1, ldy, stream) == -1


def test_multiply_x_longer_than_cols_and_unaligned():
    rng = np.random.default_rng(9)
    dense = helpers.random_sparse(rng, 128, 1001, 0.4, scale=1.0)
    x_full = rng.standard_normal(1001 + 9).astype(np.float16)
    M = torch.from_numpy(dense).cuda()
    compressed = macko_spmv.compress(M)
    xg = torch.from_numpy(x_full).cuda()
    for off in (0, 1, 3, 8):
        V = xg[off:off + 1001 + (0 if off else 9)]
        assert V.is_contiguous()
        got = macko_spmv.multiply(compressed, V).cpu().numpy()
        helpers.assert_close_fp16(got, helpers.dense_reference(dense, x_full[off:off + 1001]))
    got2d = macko_spmv.multiply(compressed, xg[:1001].reshape(1, -1)).cpu().numpy()
    helpers.assert_close_fp16(got2d, helpers.dense_reference(dense, x_full[:1001]))


def test_multiply_linearity_full_size():
    # y(a*x1 + x2) against a*y(x1) + y(x2) on a config-3 shape, too big for the CPU oracle
    torch.manual_seed(1)
    rows, cols = 8192, 28672
    M = torch.randn((rows, cols), device="cuda", dtype=torch.float16) * 0.02
    M = (M * (torch.rand((rows, cols), device="cuda") < 0.1)).contiguous()
    compressed = macko_spmv.compress(M)
    x1 = torch.randn(cols, device="cuda", dtype=torch.float16)
    x2 = torch.randn(cols, device="cuda", dtype=torch.float16)
    y1 = macko_spmv.multiply(compressed, x1).float()
    y2 = macko_spmv.multiply(compressed, x2).float()
    y12 = macko_spmv.multiply(compressed, (2 * x1 + x2)).float()
    want = (M.float() @ (2 * x1 + x2).float())
    assert torch.allclose(y12, want, rtol=1e-2, atol=2e-3)
    assert torch.allclose(y12, 2 * y1 + y2, rtol=2e-2, atol=5e-3)
    dense_y = (M.float() @ x1.float())
    assert torch.allclose(y1, dense_y, rtol=1e-2, atol=1e-3)


def test_multiply_axpby():
    rng = np.random.default_rng(21)
    dense = helpers.random_sparse(rng, 500, 2000, 0.3, scale=1.0)
    x = rng.standard_normal(2000).astype(np.float16)
    y0 = rng.standard_normal(500).astype(np.float16)
    compressed = macko_spmv.compress(torch.from_numpy(dense).cuda())
    C = torch.from_numpy(y0.copy()).cuda()
    macko_spmv.multiply_axpby(compressed, torch.from_numpy(x).cuda(), C, alpha=0.5, beta=-2.0)
    want = 0.5 * helpers.dense_reference(dense, x) - 2.0 * y0.astype(np.float64)
    helpers.assert_close_fp16(C.cpu().numpy(), want, rel=1e-2, abs_=4e-3)


def test_c_abi_direct_call():
    lib = ctypes.CDLL(macko_spmv_amd.HIP_LIBRARY_PATH)
    vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
    lib.macko_spmv_f16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i64, vp]
    lib.macko_compress_f16_count.argtypes = [vp, i32, i32, vp, vp]
    lib.macko_compress_f16_fill.argtypes = [vp, i32, i32, vp, vp, vp, i64, vp]
    rng = np.random.default_rng(31)
    rows, cols = 777, 3333
    dense = helpers.random_sparse(rng, rows, cols, 0.25, scale=1.0)
    x = rng.standard_normal(cols).astype(np.float16)
    M = torch.from_numpy(dense).cuda()
    xg = torch.from_numpy(x).cuda()
    stream = torch.cuda.current_stream().cuda_stream
    row_ptr = torch.empty(rows + 1, dtype=torch.int32, device="cuda")
    assert lib.macko_compress_f16_count(M.data_ptr(), rows, cols, row_ptr.data_ptr(), stream) == 0
    n = int(row_ptr[-1])
    P = (n + 7) // 8 * 8
    values = torch.empty(P, dtype=torch.float16, device="cuda")
    deltas = torch.empty(P // 2, dtype=torch.uint8, device="cuda")
    assert lib.macko_compress_f16_fill(M.data_ptr(), rows, cols, row_ptr.data_ptr(), values.data_ptr(),
                                       deltas.data_ptr(), P, stream) == 0
    _assert_bit_exact((values, deltas, row_ptr, rows, cols), dense)
    y = torch.empty(rows, dtype=torch.float16, device="cuda")
    assert lib.macko_spmv_f16(values.data_ptr(), deltas.data_ptr(), row_ptr.data_ptr(), xg.data_ptr(),
                              y.data_ptr(), rows, cols, P, stream) == 0
    torch.cuda.synchronize()
    helpers.assert_close_fp16(y.cpu().numpy(), helpers.dense_reference(dense, x))


def test_opcheck_and_compile():
    # tests/test_macko_spmv.py:142-178
    torch.manual_seed(0)
    M_cpu = torch.rand((4096, 8192), dtype=torch.float16, device="cpu")
    M_cpu[torch.rand_like(M_cpu) > 0.5] = 0
    M = M_cpu.cuda()
    V = torch.rand((8192,), device="cuda", dtype=torch.float16)
    compressed = macko_spmv.compress(M)
    args = (*compressed, V)
    expected = M @ V
    torch.library.opcheck(torch.ops.macko_spmv.multiply, args)
    compiled = torch.compile(macko_spmv.multiply, mode="reduce-overhead", fullgraph=True)
    for _ in range(4):  # warm-up runs, graph capture, replays
        out = compiled(compressed, V)
        assert torch.allclose(expected, out, rtol=1e-3, atol=1e-3)
    f_c = torch.compile(lambda x: macko_spmv.multiply(compressed, x + 1) - 1, mode="reduce-overhead",
                        fullgraph=True)
    for _ in range(4):
        out = f_c(V)
        assert torch.allclose((M @ (V + 1)) - 1, out, rtol=1e-3, atol=2e-3)


def test_opcheck_of_the_additional_operators():
    # schema, fake implementation and aliasing annotations of everything beyond the upstream operator
    torch.manual_seed(1)
    ops = torch.ops.macko_spmv
    M = torch.randn((300, 700), dtype=torch.float16, device="cuda")
    M[torch.rand_like(M.float()) > 0.3] = 0
    c = macko_spmv.compress(M)
    V = torch.randn(700, device="cuda", dtype=torch.float16)
    X = torch.randn(5, 700, device="cuda", dtype=torch.float16)
    C = torch.randn(300, device="cuda", dtype=torch.float16)
    torch.library.opcheck(ops.multiply_batched, (*c, X))
    torch.library.opcheck(ops.multiply_axpby, (*c, V, C, 0.5, 2.0))
    torch.library.opcheck(ops.decompress, tuple(c))
    Q = torch.randint(-100, 100, (300, 700), dtype=torch.int8, device="cuda")
    Q[torch.rand((300, 700), device="cuda") > 0.3] = 0
    c8 = macko_spmv.compress_int8(Q)
    torch.library.opcheck(ops.multiply_int8, (*c8, V))
    torch.library.opcheck(ops.multiply_int8_axpby, (*c8, V, C, 0.5, 2.0))
    compiled = torch.compile(lambda X: macko_spmv.multiply_batched(c, X * 2), mode="reduce-overhead", fullgraph=True)
    want = (X.float() * 2) @ M.float().t()
    for _ in range(3):
        assert torch.allclose(compiled(X).float(), want, rtol=1e-2, atol=2e-2)


def test_vmap_over_the_vector_like_the_upstream_llm_layer():
    # python_scripts/util_run_pruned_llm.py:109-118: torch.vmap(f, in_dims=-2, out_dims=-2) over (1, t, C)
    torch.manual_seed(2)
    M = torch.randn((300, 700), dtype=torch.float16, device="cuda")
    M[torch.rand_like(M.float()) > 0.3] = 0
    c = macko_spmv.compress(M)
    lifted = torch.vmap(lambda x: macko_spmv.multiply(c, x), in_dims=-2, out_dims=-2)
    x = torch.randn(1, 6, 700, device="cuda", dtype=torch.float16)
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")   # no fall-back to a loop over the batch: one batched product
        out = lifted(x)
    assert out.shape == (6, 300)
    assert torch.allclose(out.float(), x[0].float() @ M.float().t(), rtol=1e-2, atol=2e-2)


# ---- the upstream flow: compress on the host tensor, move the tuple, multiply ----------------------

@pytest.mark.parametrize("shape,density", [((257, 1500), 0.3), ((64, 4096), 0.5), ((1000, 333), 0.05)])
def test_cpu_compress_move_to_device_multiply(shape, density):
    # src/macko_spmv/__init__.py:110-117 (move_to_device) between :120-131 (compress of a CPU tensor)
    # and :134-149 (multiply): the route an upstream user takes when the dense matrix lives on the host
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    dense = helpers.random_sparse(rng, shape[0], shape[1], density)
    dense[3] = 0
    x = rng.standard_normal(shape[1]).astype(np.float16)
    c_cpu = macko_spmv.compress(torch.from_numpy(dense))
    assert all(t.device.type == "cpu" for t in c_cpu[:3])
    _assert_bit_exact(c_cpu, dense)
    c_gpu = macko_spmv.move_to_device(c_cpu, "cuda")
    assert all(t.is_cuda for t in c_gpu[:3]) and c_gpu[3:] == c_cpu[3:]
    # the moved tuple is what compress() gives for the same matrix on the GPU, bit for bit
    direct = macko_spmv.compress(torch.from_numpy(dense).cuda())
    for moved, made in zip(c_gpu[:3], direct[:3]):
        assert moved.dtype == made.dtype and torch.equal(moved, made)
    y = macko_spmv.multiply(c_gpu, torch.from_numpy(x).cuda()).cpu().numpy()
    values, deltas, row_ptr, _ = mo.compress(dense)
    want = mo.spmv(values, deltas, row_ptr, shape[0], shape[1], x).view(np.float16)
    assert np.allclose(y.astype(np.float32), want.astype(np.float32), rtol=1e-2, atol=1e-3)
    helpers.assert_close_fp16(y, helpers.dense_reference(dense, x))
    # and back: nothing changes on the way
    back = macko_spmv.move_to_device(c_gpu, "cpu")
    for a, b in zip(back[:3], c_cpu[:3]):
        assert a.device.type == "cpu" and torch.equal(a, b)
    assert back[3:] == c_cpu[3:]


def test_upstream_binding_names():
    # the two pybind modules of the upstream package as attributes of the module
    # (src/macko_spmv/__init__.py:36 `__compressor_lib`, :90 `__multiply_lib`, used at :124 and :141)
    rng = np.random.default_rng(5)
    dense = helpers.random_sparse(rng, 48, 700, 0.25)
    x = torch.from_numpy(rng.standard_normal(700).astype(np.float16)).cuda()
    compressor = getattr(macko_spmv, "__compressor_lib")
    multiplier = getattr(macko_spmv, "__multiply_lib")
    c = compressor.cpu_compress(torch.from_numpy(dense).cuda())
    assert len(c) == 5 and c[3] == 48 and c[4] == 700
    _assert_bit_exact(c, dense)
    y = multiplier.macko_spmv_launcher(c[0], c[1], c[2], c[3], c[4], x)
    assert y.dtype == torch.float16 and y.shape == (48,)
    assert torch.equal(y, macko_spmv.multiply(c, x))
    helpers.assert_close_fp16(y.cpu().numpy(), helpers.dense_reference(dense, x.cpu().numpy()))


def test_compress_refuses_graph_capture():
    # compress() has to read the entry count back in the middle of the call; under stream capture it
    # says so, the capture survives, and a product captured next to it still replays correctly
    rng = np.random.default_rng(11)
    dense = helpers.random_sparse(rng, 96, 640, 0.3)
    M = torch.from_numpy(dense).cuda()
    x = torch.from_numpy(rng.standard_normal(640).astype(np.float16)).cuda()
    c = macko_spmv.compress(M)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        y_eager = macko_spmv.multiply(c, x)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            with pytest.raises(RuntimeError, match="cannot be captured"):
                macko_spmv.compress(M)
            y_graph = macko_spmv.multiply(c, x)
        for _ in range(3):
            graph.replay()
            stream.synchronize()
            assert torch.equal(y_graph, y_eager)
    torch.cuda.current_stream().wait_stream(stream)
