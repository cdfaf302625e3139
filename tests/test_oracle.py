"""Pins the CPU oracle (oracle/macko_oracle.c, oracle/macko_numpy.py) before anything trusts it.

Checks, in order: the two known-answer vectors the upstream tests hold; the sequential C
restatement against an independent closed-form NumPy statement; structural invariants of the
format; compress -> decode round trips; the oracle product against a dense float64 product; the
hand-written fp16 conversions against NumPy's, exhaustively.
"""
import numpy as np
import pytest

from oracle import macko_numpy as mn
from oracle import macko_oracle as mo
from tests import helpers


@pytest.mark.parametrize("case", helpers.load_kat(), ids=lambda c: c["name"])
def test_known_answer_vectors(case):
    for compress in (mo.compress, lambda d: mn.compress_closed_form(np.asarray(d).view(np.uint16))):
        values, deltas, row_ptr, n = compress(case["dense"])
        assert np.array_equal(values, case["values"].view(np.uint16))
        assert np.array_equal(deltas, case["deltas"])
        assert np.array_equal(row_ptr, case["row_indices"])
        assert n == case["row_indices"][-1]


def test_known_answer_decoded_by_hand():
    # row 0 of the 5x32 vector: nibbles 0,0,6,3,15,0 -> columns 0,1,8,12,28(pad),29
    case = helpers.load_kat()[0]
    rows_of, cols_of = mn.entry_columns(case["deltas"], case["row_indices"])
    assert cols_of[:6].tolist() == [0, 1, 8, 12, 28, 29]
    assert rows_of[:6].tolist() == [0] * 6
    # row 4 starts at entry 13, an odd nibble slot (high half of byte 6)
    assert cols_of[13:22].tolist() == [4, 5, 7, 13, 23, 26, 28, 29, 31]


def _special_matrices():
    rng = np.random.default_rng(1234)
    out = []
    for t in range(250):
        rows = int(rng.integers(1, 9))
        cols = int(rng.integers(1, 300))
        density = float(rng.choice([0, 0.01, 0.05, 0.1, 0.3, 0.5, 0.9, 1.0]))
        bits = helpers.random_sparse(rng, rows, cols, density).view(np.uint16).copy()
        for special in (0x8000, 0x8000, 0x7E00, 0xFC00, 0x7C00, 0x0001, 0x8001, 0xFE01):
            if rng.random() < 0.5:
                bits[rng.integers(0, rows), rng.integers(0, cols)] = special
        out.append(bits)
    # gaps of exactly 15, 16, 31, 32, 33 zeros; rows ending right after a padding slot
    for gap in (14, 15, 16, 17, 30, 31, 32, 33, 47, 48):
        m = np.zeros((3, 70), dtype=np.uint16)
        m[0, 0] = 0x3C00
        m[0, gap + 1] = 0x4000
        m[1, gap] = 0x3C00          # first non-zero after `gap` leading zeros
        m[2, 69 - gap] = 0x3C00     # followed by `gap` trailing zeros
        out.append(m)
    out.append(np.zeros((4, 40), dtype=np.uint16))            # nothing stored at all
    out.append(np.full((2, 8), 0x3C00, dtype=np.uint16))      # n is a multiple of 8
    out.append(np.full((1, 1), 0x3C00, dtype=np.uint16))
    last_empty = np.zeros((3, 33), dtype=np.uint16)
    last_empty[0, 32] = 0x3C00
    out.append(last_empty)
    return out


def test_sequential_c_matches_closed_form_and_invariants():
    for bits in _special_matrices():
        rows, cols = bits.shape
        a = mo.compress(bits)
        b = mn.compress_closed_form(bits)
        for x, y in zip(a[:3], b[:3]):
            assert np.array_equal(x, y)
        assert a[3] == b[3]
        mn.check_invariants(a[0], a[1], a[2], rows, cols)


def test_round_trip():
    for bits in _special_matrices():
        rows, cols = bits.shape
        values, deltas, row_ptr, _ = mo.compress(bits)
        dec_c = mo.decode(values, deltas, row_ptr, rows, cols)
        dec_np = mn.decode(values, deltas, row_ptr, rows, cols)
        assert np.array_equal(dec_c, dec_np)
        want = bits.copy()
        want[(want & 0x7FFF) > 0x7C00] = 0x7FFF  # NaNs come back canonical
        stored = (want & 0x7FFF) != 0
        assert np.array_equal(dec_c[stored], want[stored])
        # zeros come back as zeros; only zeros sitting in a padding slot keep their sign bit
        assert not (dec_c[~stored] & 0x7FFF).any()


def test_entry_count_formula():
    # n = sum over non-zeros of 1 + (gap >> 4); checked by brute force on one row
    rng = np.random.default_rng(7)
    for _ in range(100):
        cols = int(rng.integers(1, 400))
        row = helpers.random_sparse(rng, 1, cols, float(rng.choice([0.02, 0.1, 0.5])))
        nz = np.flatnonzero(row[0] != 0)
        expect = 0
        prev = -1
        for c in nz:
            expect += 1 + ((c - prev - 1) >> 4)
            prev = c
        assert mo.compress(row)[3] == expect


@pytest.mark.parametrize("density", [1.0, 0.5, 0.1, 0.01, 0.0])
def test_oracle_product_against_dense_float64(density):
    rng = np.random.default_rng(99)
    rows, cols = 64, 1000
    dense = helpers.random_sparse(rng, rows, cols, density)
    x = rng.standard_normal(cols).astype(np.float16)
    values, deltas, row_ptr, _ = mo.compress(dense)
    y = mo.spmv(values, deltas, row_ptr, rows, cols, x).view(np.float16)
    want = helpers.dense_reference(dense, x)
    helpers.assert_close_fp16(y, want)
    # and the float64 product taken straight from the compressed arrays is the dense one
    got64 = mn.spmv_fp64(values, deltas, row_ptr, rows, cols, x.view(np.uint16))
    assert np.allclose(got64, want, rtol=1e-12, atol=1e-12)
    # dense baseline routine agrees too
    helpers.assert_close_fp16(mo.dense_gemv(dense, x).view(np.float16), want)


def test_oracle_axpby():
    rng = np.random.default_rng(5)
    rows, cols = 16, 256
    dense = helpers.random_sparse(rng, rows, cols, 0.3)
    x = rng.standard_normal(cols).astype(np.float16)
    y0 = rng.standard_normal(rows).astype(np.float16)
    values, deltas, row_ptr, _ = mo.compress(dense)
    y = mo.spmv(values, deltas, row_ptr, rows, cols, x, alpha=0.5, beta=2.0, y_bits=y0).view(np.float16)
    want = 0.5 * helpers.dense_reference(dense, x) + 2.0 * y0.astype(np.float64)
    helpers.assert_close_fp16(y, want)


def test_column_clamp_matches_reference_rule():
    # a malformed entry past the last column multiplies x[cols-1] (kernels.cuh:104-105)
    values = np.array([0x3C00, 0, 0, 0, 0, 0, 0, 0], dtype=np.uint16)  # 1.0
    deltas = np.array([15, 0, 0, 0], dtype=np.uint8)                  # column 15
    row_ptr = np.array([0, 1], dtype=np.int32)
    x = np.arange(4, dtype=np.float16)
    y = mo.spmv(values, deltas, row_ptr, 1, 4, x).view(np.float16)
    assert y[0] == np.float16(3.0)


def test_half_conversions_exhaustive():
    all_bits = np.arange(65536, dtype=np.uint16)
    as_float = all_bits.view(np.float16).astype(np.float32)
    for h in range(65536):
        f = mo.half_to_float(h)
        if np.isnan(as_float[h]):
            assert np.isnan(f)
            assert mo.float_to_half(f) == 0x7FFF
        else:
            assert f == float(as_float[h])
            assert mo.float_to_half(f) == h
    rng = np.random.default_rng(3)
    mags = np.float32(10.0) ** rng.integers(-9, 6, 5000).astype(np.float32)
    with np.errstate(over="ignore"):
        for f in rng.standard_normal(5000).astype(np.float32) * mags:
            assert mo.float_to_half(f) == int(np.array([f]).astype(np.float16).view(np.uint16)[0])
