"""Pins the int8 part of the CPU oracle.  The upstream tests hold no int8 vector, so the pins are:
the sequential C restatement against an independent per-column NumPy statement; the special case
that reduces to the fp16 compressor (which IS pinned by upstream known answers); invariants;
round trips; a brute-force entry count; the product against dense float64.
"""
import numpy as np
import pytest

from oracle import macko_numpy as mn
from oracle import macko_oracle as mo
from tests import helpers


def _random_int8(rng, rows, cols, density):
    m = rng.integers(-128, 128, (rows, cols)).astype(np.int8)
    m[rng.random((rows, cols)) >= density] = 0
    return m


def _matrices():
    rng = np.random.default_rng(4321)
    out = []
    for _ in range(250):
        rows = int(rng.integers(1, 9))
        cols = int(rng.integers(1, 300))
        out.append(_random_int8(rng, rows, cols, float(rng.choice([0, 0.01, 0.05, 0.1, 0.3, 0.5, 0.9, 1.0]))))
    for gap in (14, 15, 16, 17, 30, 31, 32, 33, 47, 48):
        m = np.zeros((3, 70), dtype=np.int8)
        m[0, 0] = 1
        m[0, gap + 1] = -2
        m[1, gap] = 3
        m[2, 69 - gap] = -128
        out.append(m)
    out.append(np.zeros((4, 40), dtype=np.int8))   # all zero: 2 padding entries per row
    out.append(np.zeros((3, 15), dtype=np.int8))   # all zero and too short for any entry
    out.append(np.zeros((2, 16), dtype=np.int8))   # exactly one padding entry per row
    out.append(np.full((2, 8), 7, dtype=np.int8))
    return out


def test_sequential_c_matches_per_column_statement():
    for dense in _matrices():
        a = mo.compress_int8(dense)
        b = mn.compress_int8_closed_form(dense)
        assert a[3] == b[3]
        for x, y in zip(a[:3], b[:3]):
            assert x.dtype == y.dtype and np.array_equal(x, y)


def test_reduces_to_the_fp16_format_when_rows_end_on_a_non_zero():
    # no trailing padding entries exist then, so row_ptr and the nibbles must be those of the fp16
    # compressor (pinned by the upstream known answers) on the same non-zero pattern
    rng = np.random.default_rng(7)
    for _ in range(100):
        rows, cols = int(rng.integers(1, 9)), int(rng.integers(1, 200))
        dense = _random_int8(rng, rows, cols, float(rng.choice([0.02, 0.1, 0.5])))
        dense[:, -1] = 5
        as_half = dense.astype(np.float16)
        v8, d8, r8, n8 = mo.compress_int8(dense)
        v16, d16, r16, n16 = mo.compress(as_half)
        assert n8 == n16 and np.array_equal(r8, r16) and np.array_equal(d8, d16)
        assert np.array_equal(v8.astype(np.float16).view(np.uint16), v16)


def test_trailing_padding_entries_are_kept():
    dense = np.zeros((2, 50), dtype=np.int8)
    dense[0, 3] = 9
    values, deltas, row_ptr, n = mo.compress_int8(dense)
    # row 0: the 9 at column 3 (nibble 3), then padding at 19 and 35; row 1: padding at 15, 31, 47
    assert row_ptr.tolist() == [0, 3, 6] and n == 6
    assert mn.unpack_nibbles(deltas, 6).tolist() == [3, 15, 15, 15, 15, 15]
    assert values[:6].tolist() == [9, 0, 0, 0, 0, 0]
    _, cols_of = mn.entry_columns(deltas, row_ptr)
    assert cols_of.tolist() == [3, 19, 35, 15, 31, 47]


def test_invariants_round_trip_and_count():
    for dense in _matrices():
        rows, cols = dense.shape
        values, deltas, row_ptr, n = mo.compress_int8(dense)
        assert row_ptr[0] == 0 and row_ptr[-1] == n and np.all(np.diff(row_ptr) >= 0)
        assert values.size % 8 == 0 and n <= values.size < n + 8 and deltas.size * 2 == values.size
        assert not values[n:].any() and not mn.unpack_nibbles(deltas, values.size)[n:].any()
        assert np.array_equal(mo.decode_int8(values, deltas, row_ptr, rows, cols), dense)
        # brute force: walk every row with a zero counter
        want = 0
        for r in range(rows):
            run = 0
            for c in range(cols):
                if dense[r, c] != 0 or run == 15:
                    want += 1
                    run = 0
                else:
                    run += 1
        assert n == want
        if n:
            nib = mn.unpack_nibbles(deltas, n)
            assert np.all(nib[values[:n] == 0] == 15)  # a stored zero is a padding entry


@pytest.mark.parametrize("density", [1.0, 0.5, 0.1, 0.01, 0.0])
def test_product_against_dense_float64(density):
    rng = np.random.default_rng(11)
    rows, cols = 48, 900
    dense = _random_int8(rng, rows, cols, density)
    x = (rng.standard_normal(cols) * 0.05).astype(np.float16)
    values, deltas, row_ptr, _ = mo.compress_int8(dense)
    y = mo.spmv_int8(values, deltas, row_ptr, rows, cols, x).view(np.float16)
    want = dense.astype(np.float64) @ x.astype(np.float64)
    helpers.assert_close_fp16(y, want)
    y0 = rng.standard_normal(rows).astype(np.float16)
    y2 = mo.spmv_int8(values, deltas, row_ptr, rows, cols, x, alpha=0.25, beta=-1.5, y_bits=y0).view(np.float16)
    helpers.assert_close_fp16(y2, 0.25 * want - 1.5 * y0.astype(np.float64))
