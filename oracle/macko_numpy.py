"""Closed-form NumPy statements of the MACKO formats (fp16, int8).  TEST INFRASTRUCTURE ONLY.

An independent second statement of what the upstream compressor emits
(src/macko_spmv/cuda/cpu_compressor.cuh:6-73), used to cross-check the sequential C
restatement in macko_oracle.c and the HIP compressor.  Nothing under macko_spmv_amd/ imports it.

Closed form.  In one row let the non-zeros sit at columns c_0 < c_1 < ... and let p be the
previous non-zero's column (-1 before the first).  With g = c - p - 1 zeros in between, the row
stores (g >> 4) padding entries at columns p+16, p+32, ... {nibble 15, value = the element
found there, i.e. a zero whose sign bit is kept: -0.0 stays 0x8000, cpu_compressor.cuh:36}
followed by the non-zero itself with nibble (g & 15).  Nothing is stored after the last non-zero; an all-zero row stores nothing.
Entry j of the whole matrix keeps its nibble in byte j // 2, low half when j is even.  Arrays are
zero-padded to a multiple of 8 entries.  "Non-zero" means non-zero as a float: -0.0 is a zero,
NaN is not; a stored NaN becomes 0x7fff (CUDA float->half conversion; parity unpinned).

All arrays carry fp16 as raw uint16 bit patterns so comparisons are bit-exact.
"""
import numpy as np


def compress_closed_form(dense_bits):
    """dense_bits: uint16 [R, C] -> (values uint16 [P], deltas uint8 [P//2], row_ptr int32 [R+1], n)."""
    dense_bits = np.ascontiguousarray(dense_bits, dtype=np.uint16)
    rows, cols = dense_bits.shape
    nz_r, nz_c = np.nonzero((dense_bits & 0x7FFF) != 0)  # row-major order
    nz_r = nz_r.astype(np.int64)
    nz_c = nz_c.astype(np.int64)
    first_in_row = np.ones(nz_r.shape, dtype=bool)
    first_in_row[1:] = nz_r[1:] != nz_r[:-1]
    prev = np.empty_like(nz_c)
    prev[1:] = nz_c[:-1]
    prev[first_in_row] = -1
    gap = nz_c - prev - 1
    pads = gap >> 4
    per_nz = pads + 1
    n = int(per_nz.sum())
    row_counts = np.bincount(nz_r, weights=per_nz, minlength=rows).astype(np.int64)
    row_ptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(row_counts, out=row_ptr[1:])
    padded = (n + 7) // 8 * 8
    nibbles = np.full(padded, 15, dtype=np.uint8)
    values = np.zeros(padded, dtype=np.uint16)
    nibbles[n:] = 0
    pos = np.cumsum(per_nz) - 1  # slot of each non-zero; its pads sit right before it
    nibbles[pos] = (gap & 15).astype(np.uint8)
    v = dense_bits[nz_r, nz_c]
    is_nan = (v & 0x7FFF) > 0x7C00
    v = np.where(is_nan, np.uint16(0x7FFF), v)
    values[pos] = v
    # padding entries copy the (signed) zero found at their own column p + 16*j
    total_pads = int(pads.sum())
    if total_pads:
        owner = np.repeat(np.arange(nz_c.size), pads)
        first_pad = np.cumsum(pads) - pads
        j = np.arange(total_pads) - first_pad[owner] + 1
        pad_col = prev[owner] + 16 * j
        pad_slot = pos[owner] - pads[owner] + (j - 1)
        values[pad_slot] = dense_bits[nz_r[owner], pad_col]
    deltas = (nibbles[0::2] | (nibbles[1::2] << 4)).astype(np.uint8)
    return values, deltas, row_ptr.astype(np.int32), n


def compress_int8_closed_form(dense):
    """int8 [R, C] -> (values int8 [P], deltas uint8 [P//2], row_ptr int32 [R+1], n).

    Per-column statement of compress_rows_int8_cpu (cpu_compressor.cuh:75-117): with p the column
    of the previous non-zero of the row (-1 before the first), column x stores an entry when its
    element is non-zero, or when x - p is a positive multiple of 16 (a padding entry, nibble 15,
    value 0).  A non-zero carries nibble (x - p - 1) & 15.  Unlike the fp16 format the padding
    entries behind the last non-zero of a row stay.
    """
    dense = np.ascontiguousarray(dense, dtype=np.int8)
    rows, cols = dense.shape
    nz = dense != 0
    col_idx = np.broadcast_to(np.arange(cols, dtype=np.int64), (rows, cols))
    last_nz_incl = np.maximum.accumulate(np.where(nz, col_idx, -1), axis=1)
    prev = np.full((rows, cols), -1, dtype=np.int64)
    prev[:, 1:] = last_nz_incl[:, :-1]
    dist = col_idx - prev
    is_entry = nz | (dist % 16 == 0)
    nib = np.where(nz, (dist - 1) & 15, 15).astype(np.uint8)
    row_counts = is_entry.sum(axis=1)
    row_ptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(row_counts, out=row_ptr[1:])
    n = int(row_ptr[-1])
    padded = (n + 7) // 8 * 8
    nibbles = np.zeros(padded, dtype=np.uint8)
    values = np.zeros(padded, dtype=np.int8)
    nibbles[:n] = nib[is_entry]  # boolean indexing walks row-major
    values[:n] = dense[is_entry]
    deltas = (nibbles[0::2] | (nibbles[1::2] << 4)).astype(np.uint8)
    return values, deltas, row_ptr.astype(np.int32), n


def unpack_nibbles(deltas, count):
    deltas = np.asarray(deltas, dtype=np.uint8)
    out = np.empty(deltas.size * 2, dtype=np.int64)
    out[0::2] = deltas & 0xF
    out[1::2] = deltas >> 4
    return out[:count]


def entry_columns(deltas, row_ptr):
    """Column of every stored entry (kernels.cuh:97-103: running nibble sum + index in row)."""
    row_ptr = np.asarray(row_ptr, dtype=np.int64)
    n = int(row_ptr[-1])
    nib = unpack_nibbles(deltas, n)
    step = nib + 1
    csum = np.cumsum(step)
    rows_of = np.repeat(np.arange(row_ptr.size - 1), np.diff(row_ptr))
    base = np.concatenate(([0], csum))[row_ptr[:-1]]  # running sum before the row's first entry
    cols = csum - base[rows_of] - 1
    return rows_of, cols


def decode(values, deltas, row_ptr, rows, cols):
    """Back to dense uint16 [rows, cols]."""
    rows_of, col_of = entry_columns(deltas, row_ptr)
    n = rows_of.size
    dense = np.zeros((rows, cols), dtype=np.uint16)
    if n:
        assert col_of.max() < cols and col_of.min() >= 0
        dense[rows_of, col_of] = np.asarray(values, dtype=np.uint16)[:n]
    return dense


def check_invariants(values, deltas, row_ptr, rows, cols):
    """Structural facts every compressed matrix satisfies; raises AssertionError otherwise."""
    values = np.asarray(values, dtype=np.uint16)
    deltas = np.asarray(deltas, dtype=np.uint8)
    row_ptr = np.asarray(row_ptr, dtype=np.int64)
    assert row_ptr.shape == (rows + 1,)
    assert row_ptr[0] == 0
    assert np.all(np.diff(row_ptr) >= 0)
    n = int(row_ptr[-1])
    padded = values.size
    assert padded % 8 == 0 and n <= padded < n + 8
    assert deltas.size * 2 == padded
    assert not values[n:].any() and not unpack_nibbles(deltas, padded)[n:].any()
    if n == 0:
        return
    nib = unpack_nibbles(deltas, n)
    rows_of, col_of = entry_columns(deltas, row_ptr)
    assert col_of.min() >= 0 and col_of.max() < cols
    is_zero = (values[:n] & 0x7FFF) == 0
    # a stored (signed) zero is a padding entry and carries nibble 15
    assert np.all(nib[is_zero] == 15)
    # every non-empty row ends on a non-zero
    ends = row_ptr[1:][np.diff(row_ptr) > 0] - 1
    assert not is_zero[ends].any()


def spmv_fp64(values, deltas, row_ptr, rows, cols, x_bits):
    """Exact-ish product from the compressed arrays: float64 accumulation, not rounded."""
    rows_of, col_of = entry_columns(deltas, row_ptr)
    n = rows_of.size
    v = np.asarray(values, dtype=np.uint16)[:n].view(np.float16).astype(np.float64)
    xv = np.asarray(x_bits, dtype=np.uint16).view(np.float16).astype(np.float64)
    out = np.zeros(rows, dtype=np.float64)
    if n:
        np.add.at(out, rows_of, v * xv[col_of])
    return out
