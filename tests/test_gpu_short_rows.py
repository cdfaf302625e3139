"""GPU parity tests for matrices of short rows (a few to a few dozen stored entries a row, many rows
per wave): the product then works all the rows of a 512-entry tile in one pass instead of row by row.
The shapes below are chosen so that this variant is the one launched (mean row length below 192
entries and at least six rows per wave of the launch); what they exercise is named per case.

Bars: compressed arrays bit-exact with the oracle's; products within |err| <= 1e-3 + 1e-2 * |want|
of the dense float64 product of the same fp16 data, and within rtol 1e-2 / atol 1e-3 of the oracle's
product where the oracle finishes in seconds.
"""
import numpy as np
import pytest
import torch

import macko_spmv
from oracle import macko_oracle as mo
from tests import helpers

pytestmark = pytest.mark.gpu


def _check(dense, x, label, oracle=True):
    print("case", label, dense.shape, flush=True)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    y = macko_spmv.multiply(c, torch.from_numpy(x).cuda()).cpu().numpy()
    helpers.assert_close_fp16(y, helpers.dense_reference(dense, x))
    if oracle:
        values = c[0].cpu().numpy().view(np.uint16)
        want = mo.spmv(values, c[1].cpu().numpy(), c[2].cpu().numpy(), c[3], c[4], x).view(np.float16)
        assert np.allclose(y.astype(np.float32), want.astype(np.float32), rtol=1e-2, atol=1e-3)
    return c


@pytest.mark.parametrize("rows,cols,density", [
    (20000, 300, 0.02),    # 6 entries a row: more than 64 rows end in a tile, the row window slides inside it
    (20000, 300, 0.05),
    (5000, 64, 0.5),       # half a tile per wave
    (30000, 40, 0.3),
    (50000, 16, 0.2),      # 3 entries a row, every fifth row or so empty
    (100000, 8, 0.05),     # mostly empty rows
    (65536, 512, 0.2),     # 100 entries a row, several tiles per wave
    (40000, 1, 1.0),       # one entry a row
    (12000, 2000, 0.05),   # 100 entries a row with long gaps (padding entries)
])
def test_short_rows(rows, cols, density):
    rng = np.random.default_rng(rows + 7 * cols)
    dense = helpers.random_sparse(rng, rows, cols, density, scale=0.05)
    x = rng.standard_normal(cols).astype(np.float16)
    _check(dense, x, "short rows", oracle=rows * cols <= 6_000_000)


def test_short_rows_with_empty_stretches_and_long_rows_between():
    # rows of about 15 entries; every 500th row full (3000 entries: it spans several tiles, begins and
    # ends inside tiles it shares with short rows); stretches of empty rows, also at both ends
    rng = np.random.default_rng(5)
    rows, cols = 20000, 3000
    dense = helpers.random_sparse(rng, rows, cols, 0.005, scale=0.05)
    dense[::500] = (rng.standard_normal((rows // 500, cols)) * 0.05).astype(np.float16)
    dense[0:70] = 0
    dense[-130:] = 0
    dense[7000:7300] = 0
    dense[rng.random(rows) < 0.1] = 0
    x = rng.standard_normal(cols).astype(np.float16)
    _check(dense, x, "short rows, long rows between", oracle=False)
    # row lengths 0, 1, 2, ... 63, 0, 1, ...: every alignment of a row's start and end within a lane
    rows, cols = 30000, 64
    dense = np.zeros((rows, cols), dtype=np.float16)
    for r in range(rows):
        dense[r, :r % 64] = 0.01 * ((r + np.arange(r % 64)) % 13 - 6)
    x = rng.standard_normal(cols).astype(np.float16)
    _check(dense, x, "short rows, every length", oracle=True)


def test_short_rows_other_entry_points():
    rng = np.random.default_rng(11)
    rows, cols = 24000, 256
    dense = helpers.random_sparse(rng, rows, cols, 0.08, scale=0.05)
    dense[100:140] = 0
    x = rng.standard_normal(cols).astype(np.float16)
    xg = torch.from_numpy(x).cuda()
    c = _check(dense, x, "short rows, plain")
    want = helpers.dense_reference(dense, x)
    # y = alpha * M x + beta * y
    y0 = rng.standard_normal(rows).astype(np.float16)
    C = torch.from_numpy(y0.copy()).cuda()
    macko_spmv.multiply_axpby(c, xg, C, alpha=0.5, beta=-2.0)
    helpers.assert_close_fp16(C.cpu().numpy(), 0.5 * want - 2.0 * y0.astype(np.float64), rel=1e-2, abs_=4e-3)
    # int8 values
    q = np.clip(np.round(dense.astype(np.float32) * 400), -127, 127).astype(np.int8)
    c8 = macko_spmv.compress_int8(torch.from_numpy(q).cuda())
    y8 = macko_spmv.multiply_int8(c8, xg).cpu().numpy().astype(np.float64)
    want8 = q.astype(np.float64) @ x.astype(np.float64)
    assert np.all(np.abs(y8 - want8) <= 1e-3 + 1e-2 * np.abs(want8) + 2 ** -11 * np.abs(want8))
    # several vectors per pass
    X = rng.standard_normal((3, cols)).astype(np.float16)
    Y = macko_spmv.multiply_batched(c, torch.from_numpy(X).cuda()).cpu().numpy()
    for b in range(3):
        helpers.assert_close_fp16(Y[b], helpers.dense_reference(dense, X[b]))


def test_short_rows_keep_inf_and_nan_to_the_rows_that_read_them():
    # x is Inf / NaN on the last columns; only rows with a stored entry there may see it.  Rows that
    # end before those columns stay finite, whatever their neighbours in the tile sum to.
    rng = np.random.default_rng(13)
    rows, cols = 30000, 200
    dense = helpers.random_sparse(rng, rows, cols, 0.06, scale=0.05)
    dense[:, 190:] = 0
    dense[:, 189] = 0.5                      # every row's last entry in front of the block: no padding entry beyond
    touched = rng.random(rows) < 0.2
    which = rng.integers(190, 200, size=rows)
    for r in np.nonzero(touched)[0]:
        dense[r, 190:which[r] + 1] = 0.25    # contiguous from 190 on, so that no padding entry is needed
    x = rng.standard_normal(cols).astype(np.float16)
    x[190:194] = np.inf
    x[194:197] = -np.inf
    x[197:] = np.nan
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    y = macko_spmv.multiply(c, torch.from_numpy(x).cuda()).cpu().numpy()
    with np.errstate(invalid="ignore", over="ignore"):
        products = dense.astype(np.float64) * x.astype(np.float64)[None, :]
        want = np.where(dense != 0, products, 0.0).sum(axis=1)   # stored entries only: 0 * Inf is not stored
    assert np.isfinite(want[~touched]).all() and not np.isfinite(want[touched]).any()
    assert np.isfinite(y[~touched]).all()
    helpers.assert_close_fp16(y[~touched], want[~touched])
    got = y[touched].astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want[touched]))
    assert np.array_equal(got[~np.isnan(got)], want[touched][~np.isnan(want[touched])])  # the same infinities
