"""ctypes front end of libmacko_oracle.so (macko_oracle.c).  TEST INFRASTRUCTURE ONLY.

Loaded by tests/, the smoke check and the benchmark's cpu_baseline leg; never by the product
package.  All fp16 data crosses this boundary as NumPy uint16 bit patterns.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmacko_oracle.so")
_lib = None


def build(force=False):
    """Compile macko_oracle.c with the Makefile next to it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE, "libmacko_oracle.so"], check=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    vp, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float
    lib.macko_oracle_compress_f16.restype = i64
    lib.macko_oracle_compress_f16.argtypes = [vp, i32, i32, vp, vp, vp, i64, ctypes.POINTER(i64)]
    lib.macko_oracle_count_f16.restype = i64
    lib.macko_oracle_count_f16.argtypes = [vp, i32, i32, vp]
    lib.macko_oracle_decode_f16.restype = ctypes.c_int
    lib.macko_oracle_decode_f16.argtypes = [vp, vp, vp, i32, i32, vp]
    lib.macko_oracle_spmv_f16.restype = None
    lib.macko_oracle_spmv_f16.argtypes = [vp, vp, vp, vp, vp, i32, i32, f32, f32, ctypes.c_int]
    lib.macko_oracle_dense_gemv_f16.restype = None
    lib.macko_oracle_dense_gemv_f16.argtypes = [vp, vp, vp, i32, i32]
    lib.macko_oracle_compress_i8.restype = i64
    lib.macko_oracle_compress_i8.argtypes = [vp, i32, i32, vp, vp, vp, i64, ctypes.POINTER(i64)]
    lib.macko_oracle_decode_i8.restype = ctypes.c_int
    lib.macko_oracle_decode_i8.argtypes = [vp, vp, vp, i32, i32, vp]
    lib.macko_oracle_spmv_i8.restype = None
    lib.macko_oracle_spmv_i8.argtypes = [vp, vp, vp, vp, vp, i32, i32, f32, f32, ctypes.c_int]
    lib.macko_oracle_float_to_half.restype = ctypes.c_uint16
    lib.macko_oracle_float_to_half.argtypes = [f32]
    lib.macko_oracle_half_to_float.restype = f32
    lib.macko_oracle_half_to_float.argtypes = [ctypes.c_uint16]
    _lib = lib
    return lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _u16(a):
    a = np.asarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    return np.ascontiguousarray(a, dtype=np.uint16)


def compress(dense_bits):
    """uint16/float16 [R, C] -> (values uint16 [P], deltas uint8 [P//2], row_ptr int32 [R+1], n)."""
    lib = _load()
    dense_bits = _u16(dense_bits)
    rows, cols = dense_bits.shape
    row_ptr = np.zeros(rows + 1, dtype=np.int32)
    n = lib.macko_oracle_count_f16(_p(dense_bits), rows, cols, _p(row_ptr))
    cap = (n + 7) // 8 * 8 + 16  # trailing pads of the last row may transiently overshoot n
    # worst transient overshoot: one row's trailing pads = cols // 16
    cap += (cols // 16 + 2) // 2 * 2
    values = np.zeros(cap, dtype=np.uint16)
    deltas = np.zeros(cap // 2, dtype=np.uint8)
    row_ptr2 = np.zeros(rows + 1, dtype=np.int32)
    padded = ctypes.c_int64(0)
    n2 = lib.macko_oracle_compress_f16(_p(dense_bits), rows, cols, _p(row_ptr2), _p(values), _p(deltas),
                                       cap, ctypes.byref(padded))
    assert n2 == n, (n, n2)
    assert np.array_equal(row_ptr, row_ptr2)
    p = padded.value
    return values[:p].copy(), deltas[: p // 2].copy(), row_ptr2, int(n)


def compress_one_walk(dense_bits):
    """The compressor as the upstream launcher runs it (cpu_compressor_torch_launcher.cuh:6-39): outputs
    sized for the worst case (rows * cols entries), one walk over the matrix.  Returns
    (values, deltas, row_ptr, n, seconds spent inside the C function)."""
    import time

    lib = _load()
    dense_bits = _u16(dense_bits)
    rows, cols = dense_bits.shape
    cap = rows * cols + 8
    values = np.zeros(cap, dtype=np.uint16)
    deltas = np.zeros(cap // 2, dtype=np.uint8)
    row_ptr = np.zeros(rows + 1, dtype=np.int32)
    padded = ctypes.c_int64(0)
    t0 = time.perf_counter()
    n = lib.macko_oracle_compress_f16(_p(dense_bits), rows, cols, _p(row_ptr), _p(values), _p(deltas), cap,
                                      ctypes.byref(padded))
    seconds = time.perf_counter() - t0
    assert n >= 0
    p = padded.value
    return values[:p].copy(), deltas[: p // 2].copy(), row_ptr, int(n), seconds


def decode(values, deltas, row_ptr, rows, cols):
    lib = _load()
    values = _u16(values)
    deltas = np.ascontiguousarray(deltas, dtype=np.uint8)
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    dense = np.zeros((rows, cols), dtype=np.uint16)
    rc = lib.macko_oracle_decode_f16(_p(values), _p(deltas), _p(row_ptr), rows, cols, _p(dense))
    if rc != 0:
        raise ValueError("an entry decodes to a column outside the matrix")
    return dense


def spmv(values, deltas, row_ptr, rows, cols, x_bits, alpha=1.0, beta=None, y_bits=None):
    """fp32-accumulated product rounded to fp16 bits (uint16 [rows])."""
    lib = _load()
    values = _u16(values)
    deltas = np.ascontiguousarray(deltas, dtype=np.uint8)
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    x_bits = _u16(x_bits).reshape(-1)
    assert x_bits.size >= cols
    y = np.zeros(rows, dtype=np.uint16) if y_bits is None else _u16(y_bits).copy()
    lib.macko_oracle_spmv_f16(_p(values), _p(deltas), _p(row_ptr), _p(x_bits), _p(y), rows, cols,
                              float(alpha), 0.0 if beta is None else float(beta), 0 if beta is None else 1)
    return y


def compress_int8(dense):
    """int8 [R, C] -> (values int8 [P], deltas uint8 [P//2], row_ptr int32 [R+1], n)."""
    lib = _load()
    dense = np.ascontiguousarray(dense, dtype=np.int8)
    rows, cols = dense.shape
    cap = rows * cols + 8
    values = np.zeros(cap, dtype=np.int8)
    deltas = np.zeros(cap // 2, dtype=np.uint8)
    row_ptr = np.zeros(rows + 1, dtype=np.int32)
    padded = ctypes.c_int64(0)
    n = lib.macko_oracle_compress_i8(_p(dense), rows, cols, _p(row_ptr), _p(values), _p(deltas), cap,
                                     ctypes.byref(padded))
    assert n >= 0
    p = padded.value
    return values[:p].copy(), deltas[: p // 2].copy(), row_ptr, int(n)


def decode_int8(values, deltas, row_ptr, rows, cols):
    lib = _load()
    values = np.ascontiguousarray(values, dtype=np.int8)
    deltas = np.ascontiguousarray(deltas, dtype=np.uint8)
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    dense = np.zeros((rows, cols), dtype=np.int8)
    rc = lib.macko_oracle_decode_i8(_p(values), _p(deltas), _p(row_ptr), rows, cols, _p(dense))
    if rc != 0:
        raise ValueError("an entry decodes to a column outside the matrix")
    return dense


def spmv_int8(values, deltas, row_ptr, rows, cols, x_bits, alpha=1.0, beta=None, y_bits=None):
    """int8 values x fp16 vector, fp32 accumulate, fp16 bits out (uint16 [rows])."""
    lib = _load()
    values = np.ascontiguousarray(values, dtype=np.int8)
    deltas = np.ascontiguousarray(deltas, dtype=np.uint8)
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    x_bits = _u16(x_bits).reshape(-1)
    assert x_bits.size >= cols
    y = np.zeros(rows, dtype=np.uint16) if y_bits is None else _u16(y_bits).copy()
    lib.macko_oracle_spmv_i8(_p(values), _p(deltas), _p(row_ptr), _p(x_bits), _p(y), rows, cols,
                             float(alpha), 0.0 if beta is None else float(beta), 0 if beta is None else 1)
    return y


def dense_gemv(dense_bits, x_bits):
    lib = _load()
    dense_bits = _u16(dense_bits)
    x_bits = _u16(x_bits).reshape(-1)
    rows, cols = dense_bits.shape
    y = np.zeros(rows, dtype=np.uint16)
    lib.macko_oracle_dense_gemv_f16(_p(dense_bits), _p(x_bits), _p(y), rows, cols)
    return y


def float_to_half(f):
    return int(_load().macko_oracle_float_to_half(float(f)))


def half_to_float(h):
    return float(_load().macko_oracle_half_to_float(int(h)))
