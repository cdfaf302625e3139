/*
 * macko_oracle.c -- CPU restatement of the MACKO fp16 compress / decode / multiply path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP product path.
 * Only the test-suite, the smoke check and the CPU-baseline leg of the benchmark
 * may load it; nothing under macko_spmv_amd/ calls into it.
 *
 * Each function cites the reference file:line (paths relative to the upstream
 * checkout) whose behaviour it restates.
 *
 * Pinning status
 *   macko_oracle_compress_f16   pinned: both known-answer vectors of the upstream
 *                               tests (tests/test_macko_spmv.py:5-69, :72-103), an
 *                               independent closed-form statement (macko_numpy.py),
 *                               format invariants and compress->decode round trips.
 *                               NaN payload canonicalisation (-> 0x7fff) follows CUDA's
 *                               float->half conversion and is PARITY UNPINNED: no
 *                               upstream fixture holds a NaN.
 *   macko_oracle_decode_f16     pinned by round trip against dense inputs and by the
 *                               two known-answer vectors decoded by hand.
 *   macko_oracle_spmv_f16       pinned against a dense fp64 mat-vec (textbook
 *                               reduction) within the fp16 tolerance the tests state.
 *   macko_oracle_compress_i8    the upstream tests hold no int8 vector.  Pinned by: an
 *                               independent closed-form statement (macko_numpy.py); the
 *                               special case that reduces to the fp16 compressor (rows whose
 *                               last column is non-zero have no trailing padding entries, so
 *                               row_ptr and nibbles must equal those of the known-answer-pinned
 *                               fp16 compressor on the same non-zero pattern); format
 *                               invariants; compress->decode round trips; a brute-force
 *                               entry count.
 *   macko_oracle_spmv_i8        pinned against a dense fp64 mat-vec within the fp16
 *                               tolerance, and by exact agreement with a float64 product
 *                               taken from the decoded arrays.
 *
 * Plain C99, no dependencies beyond libc/libm.  Half precision is handled as raw
 * uint16_t bit patterns so the file builds with any gcc.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define MACKO_GAP_LIMIT 15u /* largest gap a 4-bit delta can store (cpu_compressor.cuh:27) */
#define MACKO_CHUNK 8       /* arrays are padded to a multiple of 8 entries (cpu_compressor.cuh:69) */

/* ---- IEEE binary16 <-> binary32, bit exact -------------------------------------------- */

static float half_bits_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t out;
    if (exp == 0) {
        if (man == 0) {
            out = sign;
        } else { /* subnormal half: renormalise */
            int shift = 0;
            while ((man & 0x400u) == 0) {
                man <<= 1;
                ++shift;
            }
            man &= 0x3ffu;
            out = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 0x1fu) {
        out = sign | 0x7f800000u | (man << 13);
    } else {
        out = sign | ((exp + (127 - 15)) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &out, sizeof f);
    return f;
}

/* Round-to-nearest-even.  A NaN becomes 0x7fff (sign dropped), which is what CUDA's
 * host and device float->half conversions produce; the upstream compressor stores every
 * value through such a conversion (cpu_compressor.cuh:26,36). */
static uint16_t float_to_half_bits(float f)
{
    uint32_t x;
    memcpy(&x, &f, sizeof x);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7fffffffu;
    if (mag > 0x7f800000u)
        return 0x7fffu;
    if (mag == 0x7f800000u)
        return (uint16_t)(sign | 0x7c00u);
    if (mag >= 0x477ff000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    if (mag < 0x33000001u) /* below half of the smallest subnormal -> 0 */
        return (uint16_t)sign;
    int32_t e = (int32_t)(mag >> 23) - 127;
    uint32_t m = (mag & 0x7fffffu) | 0x800000u;
    uint32_t shift;
    uint32_t base;
    if (e < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - e));
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7fffffu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u)))
        ++q;
    return (uint16_t)(sign | (base + q)); /* a mantissa carry bumps the exponent correctly */
}

uint16_t macko_oracle_float_to_half(float f) { return float_to_half_bits(f); }
float macko_oracle_half_to_float(uint16_t h) { return half_bits_to_float(h); }

/* ---- nibble access: entry j lives in byte j/2, low nibble when j is even
 *      (cpu_compressor.cuh:29-35) -------------------------------------------------------- */

static void nibble_store(uint8_t *deltas, int64_t j, unsigned v)
{
    uint8_t *b = deltas + (j >> 1);
    if (j & 1)
        *b = (uint8_t)((*b & 0x0fu) | (v << 4));
    else
        *b = (uint8_t)v; /* starting a fresh byte clears its high nibble too */
}

static unsigned nibble_load(const uint8_t *deltas, int64_t j)
{
    return (deltas[j >> 1] >> ((j & 1) * 4)) & 0xfu;
}

/*
 * Compress a dense row-major fp16 matrix.  Follows compress_rows_cpu
 * (src/macko_spmv/cuda/cpu_compressor.cuh:6-73):
 *   - walk every row left to right keeping the number of zeros since the last stored
 *     entry; store an entry when the element is non-zero as a float (so -0.0 is a zero and
 *     NaN is not) or when that count has reached 15 (:24-46);
 *   - after the row, take back every entry stored after the row's last non-zero (:48-64);
 *   - row_ptr[r+1] is the running entry count (:66);
 *   - the arrays end at the count rounded up to a multiple of 8, zero filled (:68-72).
 *
 * `capacity` is the number of entries `values` can hold (`deltas` holds capacity/2 bytes,
 * capacity even).  rows*cols+8 always suffices.  Returns the unpadded entry count n, or -1
 * when capacity is too small.  *padded receives ceil(n/8)*8.
 */
int64_t macko_oracle_compress_f16(const uint16_t *dense, int32_t rows, int32_t cols,
                                  int32_t *row_ptr, uint16_t *values, uint8_t *deltas,
                                  int64_t capacity, int64_t *padded)
{
    int64_t n = 0;
    row_ptr[0] = 0;
    for (int32_t r = 0; r < rows; ++r) {
        const uint16_t *row = dense + (size_t)r * (size_t)cols;
        unsigned gap = 0;
        int64_t keep = n; /* entry count just after the row's last non-zero so far */
        for (int32_t c = 0; c < cols; ++c) {
            float v = half_bits_to_float(row[c]);
            int nonzero = (v != 0.0f);
            if (nonzero || gap == MACKO_GAP_LIMIT) {
                if (n >= capacity)
                    return -1;
                nibble_store(deltas, n, gap);
                values[n] = float_to_half_bits(v);
                ++n;
                gap = 0;
                if (nonzero)
                    keep = n;
            } else {
                ++gap;
            }
        }
        for (int64_t j = keep; j < n; ++j) { /* trailing padding entries are withdrawn */
            nibble_store(deltas, j, 0);
            values[j] = 0;
        }
        n = keep;
        row_ptr[r + 1] = (int32_t)n;
    }
    int64_t p = (n + MACKO_CHUNK - 1) / MACKO_CHUNK * MACKO_CHUNK;
    if (p > capacity)
        return -1;
    for (int64_t j = n; j < p; ++j) {
        nibble_store(deltas, j, 0);
        values[j] = 0;
    }
    if (padded)
        *padded = p;
    return n;
}

/* Entry count only (no output arrays): the same walk as above. */
int64_t macko_oracle_count_f16(const uint16_t *dense, int32_t rows, int32_t cols, int32_t *row_ptr)
{
    int64_t n = 0;
    row_ptr[0] = 0;
    for (int32_t r = 0; r < rows; ++r) {
        const uint16_t *row = dense + (size_t)r * (size_t)cols;
        unsigned gap = 0;
        int64_t pending = 0; /* padding entries not yet confirmed by a later non-zero */
        for (int32_t c = 0; c < cols; ++c) {
            if ((row[c] & 0x7fffu) != 0) {
                n += pending + 1;
                pending = 0;
                gap = 0;
            } else if (gap == MACKO_GAP_LIMIT) {
                ++pending;
                gap = 0;
            } else {
                ++gap;
            }
        }
        row_ptr[r + 1] = (int32_t)n;
    }
    return n;
}

/*
 * Decode back to a dense row-major matrix.  Column rule from the multiply kernel
 * (src/macko_spmv/cuda/kernels.cuh:97-103): inside a row the k-th entry sits at column
 * (sum of the nibbles of entries 0..k) + k.  Returns 0, or -1 when an entry decodes to a
 * column outside [0, cols).
 */
int macko_oracle_decode_f16(const uint16_t *values, const uint8_t *deltas, const int32_t *row_ptr,
                            int32_t rows, int32_t cols, uint16_t *dense)
{
    memset(dense, 0, (size_t)rows * (size_t)cols * sizeof(uint16_t));
    for (int32_t r = 0; r < rows; ++r) {
        int64_t col = -1;
        for (int64_t j = row_ptr[r]; j < row_ptr[r + 1]; ++j) {
            col += (int64_t)nibble_load(deltas, j) + 1;
            if (col >= cols)
                return -1;
            dense[(size_t)r * (size_t)cols + (size_t)col] = values[j];
        }
    }
    return 0;
}

/*
 * y = fp16(alpha * (M x) [+ beta * y]).  Follows macko_spmv<reuse_value_from_c>
 * (src/macko_spmv/cuda/kernels.cuh:34-124): per row an fp32 accumulator over
 * float(value) * float(x[col]) (:106-107, contracted to an FMA by the device compiler),
 * column clamped to [0, cols-1] (:104-105), result rounded to fp16 (:115-121).  The upstream
 * kernel sums in a lane-interleaved order; this restatement sums left to right, which the
 * tolerance-based parity bar allows.
 */
void macko_oracle_spmv_f16(const uint16_t *values, const uint8_t *deltas, const int32_t *row_ptr,
                           const uint16_t *x, uint16_t *y, int32_t rows, int32_t cols,
                           float alpha, float beta, int use_beta)
{
    for (int32_t r = 0; r < rows; ++r) {
        float acc = 0.0f;
        int64_t col = -1;
        for (int64_t j = row_ptr[r]; j < row_ptr[r + 1]; ++j) {
            col += (int64_t)nibble_load(deltas, j) + 1;
            int64_t cc = col >= cols ? cols - 1 : col;
            if (cc < 0)
                cc = 0;
            acc = fmaf(half_bits_to_float(values[j]), half_bits_to_float(x[cc]), acc);
        }
        float out = alpha * acc;
        if (use_beta)
            out += beta * half_bits_to_float(y[r]);
        y[r] = float_to_half_bits(out);
    }
}

/* Dense fp32-accumulated mat-vec on the uncompressed matrix: the CPU path a user of the
 * upstream package has for the product itself (tests/test_macko_spmv.py:110,124 use the
 * dense product as the expected result).  Used only as a timed baseline. */
void macko_oracle_dense_gemv_f16(const uint16_t *dense, const uint16_t *x, uint16_t *y,
                                 int32_t rows, int32_t cols)
{
    for (int32_t r = 0; r < rows; ++r) {
        const uint16_t *row = dense + (size_t)r * (size_t)cols;
        float acc = 0.0f;
        for (int32_t c = 0; c < cols; ++c)
            acc = fmaf(half_bits_to_float(row[c]), half_bits_to_float(x[c]), acc);
        y[r] = float_to_half_bits(acc);
    }
}

/* ---- int8 values variant --------------------------------------------------------------- */

/*
 * Compress a dense row-major int8 matrix.  Follows compress_rows_int8_cpu
 * (src/macko_spmv/cuda/cpu_compressor.cuh:75-117): the same walk as the fp16 compressor
 * (entry when the element is non-zero or 15 zeros have been skipped, :94-110), but the
 * padding entries behind a row's last non-zero are KEPT (there is no withdrawal step), so an
 * all-zero row of C columns stores C/16 padding entries.  row_ptr[r+1] is the running count
 * (:111); arrays end at the count rounded up to a multiple of 8 (:113-117), zero filled
 * (calloc, :82-83).  Same capacity / return convention as macko_oracle_compress_f16.
 */
int64_t macko_oracle_compress_i8(const int8_t *dense, int32_t rows, int32_t cols, int32_t *row_ptr,
                                 int8_t *values, uint8_t *deltas, int64_t capacity, int64_t *padded)
{
    int64_t n = 0;
    row_ptr[0] = 0;
    for (int32_t r = 0; r < rows; ++r) {
        const int8_t *row = dense + (size_t)r * (size_t)cols;
        unsigned gap = 0;
        for (int32_t c = 0; c < cols; ++c) {
            if (row[c] != 0 || gap == MACKO_GAP_LIMIT) {
                if (n >= capacity)
                    return -1;
                nibble_store(deltas, n, gap);
                values[n] = row[c];
                ++n;
                gap = 0;
            } else {
                ++gap;
            }
        }
        row_ptr[r + 1] = (int32_t)n;
    }
    int64_t p = (n + MACKO_CHUNK - 1) / MACKO_CHUNK * MACKO_CHUNK;
    if (p > capacity)
        return -1;
    for (int64_t j = n; j < p; ++j) {
        nibble_store(deltas, j, 0);
        values[j] = 0;
    }
    if (padded)
        *padded = p;
    return n;
}

/* Decode of the int8 arrays: the column rule of macko_spmv_int8
 * (src/macko_spmv/cuda/kernels.cuh:196-197), identical to the fp16 one. */
int macko_oracle_decode_i8(const int8_t *values, const uint8_t *deltas, const int32_t *row_ptr,
                           int32_t rows, int32_t cols, int8_t *dense)
{
    memset(dense, 0, (size_t)rows * (size_t)cols);
    for (int32_t r = 0; r < rows; ++r) {
        int64_t col = -1;
        for (int64_t j = row_ptr[r]; j < row_ptr[r + 1]; ++j) {
            col += (int64_t)nibble_load(deltas, j) + 1;
            if (col >= cols)
                return -1;
            dense[(size_t)r * (size_t)cols + (size_t)col] = values[j];
        }
    }
    return 0;
}

/*
 * y = fp16(alpha * (M x) [+ beta * y]) for int8 values and an fp16 vector.  Follows
 * macko_spmv_int8<reuse_value_from_c> (src/macko_spmv/cuda/kernels.cuh:126-216): fp32
 * accumulator over float(value) * float(x[col]) (:198-202), column clamped to [0, cols-1]
 * (:199-200), result rounded to fp16 (:208-215).  Summed left to right (the upstream order is
 * lane-interleaved; the parity bar is tolerance based).
 */
void macko_oracle_spmv_i8(const int8_t *values, const uint8_t *deltas, const int32_t *row_ptr,
                          const uint16_t *x, uint16_t *y, int32_t rows, int32_t cols, float alpha,
                          float beta, int use_beta)
{
    for (int32_t r = 0; r < rows; ++r) {
        float acc = 0.0f;
        int64_t col = -1;
        for (int64_t j = row_ptr[r]; j < row_ptr[r + 1]; ++j) {
            col += (int64_t)nibble_load(deltas, j) + 1;
            int64_t cc = col >= cols ? cols - 1 : col;
            if (cc < 0)
                cc = 0;
            acc = fmaf((float)values[j], half_bits_to_float(x[cc]), acc);
        }
        float out = alpha * acc;
        if (use_beta)
            out += beta * half_bits_to_float(y[r]);
        y[r] = float_to_half_bits(out);
    }
}
