"""GPU parity tests for what the first test files leave open: matrices with fewer rows than the GPU
has waves (rows split between the waves of a workgroup), row ends next to Inf / NaN entries of x, and
the largest configurations, which only the GPU itself can check (round trips, the dense fp32 product,
entry counts).

Bars: compressed arrays bit-exact; products within |err| <= 1e-3 + 1e-2 * |want| of the dense
float64 (or, at the largest sizes, fp32-accumulated) product of the same fp16 data.
"""
import ctypes

import numpy as np
import pytest
import torch

import macko_spmv
import macko_spmv_amd
from oracle import macko_oracle as mo
from tests import helpers

pytestmark = pytest.mark.gpu


def _oracle_product(compressed, x_np):
    values = compressed[0].cpu().numpy().view(np.uint16)
    return mo.spmv(values, compressed[1].cpu().numpy(), compressed[2].cpu().numpy(), compressed[3], compressed[4],
                   x_np).view(np.float16)


def _check(dense, x, label):
    print("case", label, dense.shape, flush=True)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    y = macko_spmv.multiply(c, torch.from_numpy(x).cuda()).cpu().numpy()
    helpers.assert_close_fp16(y, helpers.dense_reference(dense, x))
    assert np.allclose(y.astype(np.float32), _oracle_product(c, x).astype(np.float32), rtol=1e-2, atol=1e-3)
    return c


# ---- few, long rows: workgroups own the rows, their waves split them ---------------------------------

@pytest.mark.parametrize("rows,cols,density", [(1024, 8192, 0.5), (512, 16384, 0.5), (512, 16384, 0.1),
                                               (64, 49152, 0.5), (64, 49152, 0.1), (2000, 12288, 0.3),
                                               (300, 40000, 0.3), (17, 30000, 0.9), (1, 81000, 1.0),
                                               (7, 100000, 0.3), (96, 49152, 0.3), (255, 9000, 0.7),
                                               (257, 9000, 0.7), (1500, 6000, 1.0)])
def test_rows_split_between_waves(rows, cols, density):
    rng = np.random.default_rng(rows * 31 + cols)
    dense = helpers.random_sparse(rng, rows, cols, density, scale=0.05)
    x = rng.standard_normal(cols).astype(np.float16)
    _check(dense, x, "split")
    # empty rows at the start, at the end and in between; one row much longer than the others
    if rows >= 7:
        dense[0] = 0
        dense[-1] = 0
        dense[rng.random(rows) < 0.15] = 0
        dense[rows // 2] = (rng.standard_normal(cols) * 0.05).astype(np.float16)
        _check(dense, x, "split, empty rows")


def test_rows_split_between_waves_row_lengths_vary_wildly():
    rng = np.random.default_rng(91)
    rows, cols = 600, 20000
    density = np.linspace(0.0005, 0.95, rows) ** 2
    dense = (rng.standard_normal((rows, cols), dtype=np.float32) * 0.05).astype(np.float16)
    dense[rng.random((rows, cols)) >= density[:, None]] = 0
    x = rng.standard_normal(cols).astype(np.float16)
    _check(dense, x, "split, sorted row lengths")
    _check(dense[::-1].copy(), x, "split, sorted row lengths reversed")
    perm = rng.permutation(rows)
    _check(dense[perm].copy(), x, "split, shuffled row lengths")


def test_rows_split_between_waves_other_entry_points():
    # the same few-row shapes through the epilogue, int8, batched and fused-input entry points
    rng = np.random.default_rng(7)
    rows, cols = 384, 16384
    dense = helpers.random_sparse(rng, rows, cols, 0.4, scale=0.05)
    dense[5] = 0
    x = rng.standard_normal(cols).astype(np.float16)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    xg = torch.from_numpy(x).cuda()
    want = helpers.dense_reference(dense, x)
    # y = alpha * M x + beta * y
    y0 = rng.standard_normal(rows).astype(np.float16)
    C = torch.from_numpy(y0.copy()).cuda()
    macko_spmv.multiply_axpby(c, xg, C, alpha=0.5, beta=-2.0)
    helpers.assert_close_fp16(C.cpu().numpy(), 0.5 * want - 2.0 * y0.astype(np.float64), rel=1e-2, abs_=4e-3)
    # several vectors per pass (16384 columns: four vectors per launch, then two, then one)
    X = rng.standard_normal((7, cols)).astype(np.float16)
    Y = macko_spmv.multiply_batched(c, torch.from_numpy(X).cuda()).cpu().numpy()
    for b in range(7):
        helpers.assert_close_fp16(Y[b], helpers.dense_reference(dense, X[b]))
    # int8 values
    q = np.clip(np.round(dense.astype(np.float32) * 400), -127, 127).astype(np.int8)
    c8 = macko_spmv.compress_int8(torch.from_numpy(q).cuda())
    y8 = macko_spmv.multiply_int8(c8, xg).cpu().numpy().astype(np.float64)
    want8 = q.astype(np.float64) @ x.astype(np.float64)
    assert np.all(np.abs(y8 - want8) <= 1e-3 + 1e-2 * np.abs(want8) + 2 ** -11 * np.abs(want8))
    # input produced while it is staged: RMS norm, SiLU gate
    w = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float16)
    normed = macko_spmv.multiply_rmsnorm(c, xg, torch.from_numpy(w).cuda(), 1e-5).cpu().numpy()
    xf = x.astype(np.float64)
    n_host = (xf / np.sqrt((xf ** 2).mean() + 1e-5) * w.astype(np.float64)).astype(np.float16)
    helpers.assert_close_fp16(normed, helpers.dense_reference(dense, n_host), rel=2e-2, abs_=2e-3)
    up = rng.standard_normal(cols).astype(np.float16)
    acc = torch.from_numpy(y0.copy()).cuda()
    macko_spmv.multiply_silu_mul_axpby(c, xg, torch.from_numpy(up).cuda(), acc, 1.0, 1.0)
    gated = (xf / (1 + np.exp(-xf)) * up.astype(np.float64)).astype(np.float16)
    helpers.assert_close_fp16(acc.cpu().numpy(), helpers.dense_reference(dense, gated) + y0.astype(np.float64),
                              rel=2e-2, abs_=4e-3)


# ---- row ends next to Inf / NaN in x --------------------------------------------------------------------

def _poisoned_case(rng, rows, cols, blocks):
    """Matrix whose rows end right in front of a block of columns that no stored entry (non-zero or
    padding entry) ever touches, and an x that is Inf / NaN exactly on those columns."""
    dense = np.zeros((rows, cols), dtype=np.float16)
    starts = [b for b, _ in blocks]
    for r in range(rows):
        end = starts[r % len(starts)]            # this row's last non-zero sits at column end - 1
        lo = 0
        for b, width in blocks:                   # columns between the blocks, up to `end`
            hi = min(b, end)
            if hi > lo:
                k = max(2, int((hi - lo) * rng.uniform(0.05, 0.9)))
                cols_r = rng.choice(np.arange(lo, hi), size=min(k, hi - lo), replace=False)
                dense[r, cols_r] = (rng.standard_normal(cols_r.size) * 0.1).astype(np.float16)
                # both neighbours of a block are non-zero, so the gap across it stays below 16 columns
                dense[r, hi - 1] = 0.5
                dense[r, lo] = 0.25
            lo = b + width
            if lo >= end:
                break
    x = rng.standard_normal(cols).astype(np.float16)
    for i, (b, width) in enumerate(blocks):
        x[b:b + width] = [np.inf, -np.inf, np.nan][i % 3]
    assert not dense[:, np.concatenate([np.arange(b, b + w) for b, w in blocks])].any()
    return dense, x


@pytest.mark.parametrize("rows,cols", [(700, 3000), (5000, 1200), (40, 30000)])
def test_row_ends_next_to_inf_and_nan(rows, cols):
    # Entries that are masked off at a row's end would read the columns right behind the row's last
    # entry; multiplied by a masked (zero) value an Inf or NaN there would still poison the sum.
    rng = np.random.default_rng(rows + cols)
    blocks = [(cols // 5, 9), (cols // 2 + 3, 8), (cols - 40, 12)]
    dense, x = _poisoned_case(rng, rows, cols, blocks)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    want_oracle = _oracle_product(c, x).astype(np.float32)
    assert np.isfinite(want_oracle).all(), "the checker itself reads no poisoned column"
    xg = torch.from_numpy(x).cuda()
    y = macko_spmv.multiply(c, xg).cpu().numpy().astype(np.float32)
    assert np.isfinite(y).all(), f"{(~np.isfinite(y)).sum()} rows poisoned"
    assert np.allclose(y, want_oracle, rtol=1e-2, atol=1e-3)
    finite_x = np.where(np.isfinite(x), x, 0).astype(np.float16)
    helpers.assert_close_fp16(y, helpers.dense_reference(dense, finite_x))
    # epilogue, several vectors, int8 values
    y0 = rng.standard_normal(rows).astype(np.float16)
    C = torch.from_numpy(y0.copy()).cuda()
    macko_spmv.multiply_axpby(c, xg, C, alpha=2.0, beta=1.0)
    got = C.cpu().numpy().astype(np.float32)
    assert np.isfinite(got).all()
    helpers.assert_close_fp16(got, 2.0 * helpers.dense_reference(dense, finite_x) + y0.astype(np.float64),
                              rel=1e-2, abs_=4e-3)
    X = np.stack([x, x[::-1].copy(), x])
    X[1] = rng.standard_normal(cols).astype(np.float16)
    Y = macko_spmv.multiply_batched(c, torch.from_numpy(X).cuda()).cpu().numpy().astype(np.float32)
    assert np.isfinite(Y).all()
    assert np.allclose(Y[0], want_oracle, rtol=1e-2, atol=1e-3) and np.allclose(Y[2], want_oracle, rtol=1e-2, atol=1e-3)
    q = np.clip(np.round(dense.astype(np.float32) * 200), -127, 127).astype(np.int8)
    q[(q == 0) & (dense != 0)] = 1
    c8 = macko_spmv.compress_int8(torch.from_numpy(q).cuda())
    y8 = macko_spmv.multiply_int8(c8, xg).cpu().numpy().astype(np.float64)
    # the int8 format keeps the padding entries behind a row's last non-zero (one every 16 columns),
    # and those do multiply the poisoned columns they sit on: compare with the checker, NaN for NaN
    want8 = mo.spmv_int8(c8[0].cpu().numpy(), c8[1].cpu().numpy(), c8[2].cpu().numpy(), rows, cols, x).view(np.float16)
    want8 = want8.astype(np.float64)
    same_nan = np.isnan(y8) == np.isnan(want8)
    assert same_nan.all()
    ok = ~np.isnan(want8)
    assert np.allclose(y8[ok], want8[ok], rtol=1e-2, atol=1e-3)


# ---- the largest configurations ---------------------------------------------------------------------------

def _padding_entries(M, block=1024):
    """Number of padding entries the format stores for M: one per 16 zeros in every gap in front of a
    non-zero (trailing zeros of a row store nothing)."""
    rows, cols = M.shape
    total = 0
    col = torch.arange(cols, device=M.device, dtype=torch.int32)
    for r0 in range(0, rows, block):
        nz = M[r0:r0 + block] != 0
        idx = torch.where(nz, col[None, :], torch.full_like(col, -1)[None, :])
        prev = torch.cummax(idx, dim=1).values            # last non-zero at or before every column
        prev = torch.cat((torch.full_like(prev[:, :1], -1), prev[:, :-1]), dim=1)   # ... strictly before
        gap = col[None, :] - prev - 1
        total += int((gap[nz] // 16).sum())
    return total


@pytest.mark.parametrize("rows,cols", [(12288, 49152), (49152, 12288), (28672, 8192)])
@pytest.mark.parametrize("density", [0.1, 0.5])
def test_large_configuration_round_trip_and_product(rows, cols, density):
    g = torch.Generator(device="cuda")
    g.manual_seed(rows + int(100 * density))
    M = (torch.randn((rows, cols), device="cuda", dtype=torch.float32, generator=g) * 0.02).half()
    M = (M * (torch.rand((rows, cols), device="cuda", generator=g) < density)).contiguous()
    x = torch.randn(cols, device="cuda", generator=g).half()
    print("large case", rows, cols, density, flush=True)
    compressed = macko_spmv.compress(M)
    values, deltas, row_ptr = compressed[:3]
    n = int(row_ptr[-1])
    assert values.numel() % 8 == 0 and n <= values.numel() < n + 8 and deltas.numel() * 2 == values.numel()
    assert int(row_ptr[0]) == 0 and bool((row_ptr[1:] >= row_ptr[:-1]).all())
    nnz = int((M != 0).sum())
    assert n == nnz + _padding_entries(M)
    assert int((values[:n] == 0).sum()) == n - nnz        # exactly the padding entries hold a zero
    back = macko_spmv.decompress(compressed)
    assert torch.equal((back + 0.0).view(torch.int16), (M + 0.0).view(torch.int16))
    del back
    y = macko_spmv.multiply(compressed, x).float()
    want = M.float() @ x.float()
    assert torch.allclose(y, want, rtol=1e-2, atol=1e-3)
    # the C ABI directly, into a buffer with a guard element behind it
    lib = ctypes.CDLL(macko_spmv_amd.HIP_LIBRARY_PATH)
    vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
    lib.macko_spmv_f16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i64, vp]
    out = torch.full((rows + 1,), 7.0, dtype=torch.float16, device="cuda")
    rc = lib.macko_spmv_f16(values.data_ptr(), deltas.data_ptr(), row_ptr.data_ptr(), x.data_ptr(), out.data_ptr(),
                            rows, cols, values.numel(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(out[:rows].float(), y) and float(out[rows]) == 7.0


# ---- a malformed matrix: entries that decode to columns beyond `cols` --------------------------------

@pytest.mark.parametrize("rows,wide,cols", [(300, 900, 600), (64, 40000, 30000)])
def test_columns_beyond_cols_leave_the_other_rows_alone(rows, wide, cols):
    """A well-formed matrix never decodes a column >= cols.  For one that does, upstream clamps the
    column to cols - 1 (kernels.cuh:104-105); here the product of such a row is unspecified, but
    the call must return normally and every row whose entries all lie inside `cols` must be right.
    Built by compressing a wider matrix and passing a smaller column count."""
    rng = np.random.default_rng(rows + cols)
    dense = helpers.random_sparse(rng, rows, wide, 0.2)
    dense[::3, cols:] = 0  # every third row stays inside `cols`
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    x = rng.standard_normal(cols).astype(np.float16)
    print("case malformed", rows, wide, cols, flush=True)
    y = macko_spmv.multiply((c[0], c[1], c[2], rows, cols), torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    y = y.cpu().numpy()
    want = helpers.dense_reference(dense[::3, :cols], x)
    helpers.assert_close_fp16(y[::3], want)
    # the next call on the same stream is unaffected
    good = macko_spmv.compress(torch.from_numpy(np.ascontiguousarray(dense[:, :cols])).cuda())
    y2 = macko_spmv.multiply(good, torch.from_numpy(x).cuda()).cpu().numpy()
    helpers.assert_close_fp16(y2, helpers.dense_reference(dense[:, :cols], x))
