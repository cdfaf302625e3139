/*
 * macko_hip.h -- C ABI of libmacko_hip.so: MACKO fp16 sparse matrix-vector product and
 * compressor for AMD gfx950 (MI355X).
 *
 * Plain pointers and sizes only.  Every pointer is a DEVICE pointer unless said otherwise.
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).  No entry point
 * allocates, frees or keeps caller-visible memory; nothing synchronises unless said otherwise.
 * Return value: 0 on success, a positive hipError_t from the HIP runtime, or one of the
 * negative MACKO_E_* codes below.  macko_hip_error_string() explains either kind.
 *
 * Compressed matrix ("the 5-tuple" of the upstream Python API, src/macko_spmv/__init__.py:120-131):
 *   values   fp16  [P]      stored entries (non-zeros and padding entries), P a multiple of 8
 *   deltas   uint8 [P/2]    4-bit column gaps, entry j in byte j/2, low nibble when j is even
 *   row_ptr  int32 [rows+1] entry index where each row starts; row_ptr[rows] = n <= P < n + 8
 *   rows, cols
 * Column of the k-th entry of a row = (sum of the nibbles of its entries 0..k) + k.
 */
#ifndef MACKO_HIP_H
#define MACKO_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Entry points are the only symbols the library exports. */
#if defined(__GNUC__)
#define MACKO_API __attribute__((visibility("default")))
#else
#define MACKO_API
#endif

#define MACKO_E_INVALID_ARGUMENT (-1) /* null pointer, negative size, rows*cols >= 2^31 ... */
#define MACKO_E_NO_DEVICE (-2)        /* no usable HIP device */

/* ABI version of this header (bumped on incompatible change). */
MACKO_API int macko_hip_abi_version(void);

/* Human-readable text for a return code of this library.  Never NULL; static storage. */
MACKO_API const char *macko_hip_error_string(int code);

/*
 * y[r] = fp16( sum_k fp32(values[k]) * fp32(x[col_k]) ) for every row r, fp32 accumulation.
 *
 * Replaces the kernel launch in macko_spmv_launcher
 * (src/macko_spmv/cuda/kernels_torch_launchers.cuh:15-45, kernel src/macko_spmv/cuda/kernels.cuh:34-124,
 * alpha = 1, beta ignored).  Asynchronous on `stream`; safe to capture in a HIP graph.
 *
 *   padded_entries = P = number of fp16 elements in `values` (0 allowed: y is zero-filled)
 *   x   fp16 [>= cols], 2-byte aligned (16-byte alignment is faster)
 *   y   fp16 [rows], written for every row
 */
MACKO_API int macko_spmv_f16(const void *values, const void *deltas, const int32_t *row_ptr,
                   const void *x, void *y, int32_t rows, int32_t cols,
                   int64_t padded_entries, void *stream);

/*
 * y[r] = fp16( alpha * (M x)[r] + beta * fp32(y[r]) ).
 *
 * Replaces the macko_spmv<true> instantiation that the upstream C benchmark launches
 * (src/macko_spmv/cuda/kernels.cuh:113-118, c_benchmarking/benchmark.cu:92-105).
 */
MACKO_API int macko_spmv_f16_axpby(const void *values, const void *deltas, const int32_t *row_ptr,
                         const void *x, void *y, int32_t rows, int32_t cols,
                         int64_t padded_entries, float alpha, float beta, void *stream);

/*
 * Prepared cuts ("plan") for macko_spmv_f16 / macko_spmv_f16_axpby.  No counterpart in the reference:
 * its kernel owns one row per warp (src/macko_spmv/cuda/kernels.cuh:34-56) and has nothing to look
 * up.  Here a launch deals whole rows to a fixed number of waves by stored entries, and every wave
 * finds its first row in row_ptr when the kernel starts.  Where rows are about equally long that
 * search takes one probe; where they are not (row lengths spread over orders of magnitude) it takes
 * whole workgroups one or two more round trips to memory per launch.  A plan holds the result of
 * that search for one matrix: build it once after compressing, pass it with every product.
 *
 *   macko_spmv_plan_entries  *entries = int32 elements a plan for this shape holds on the current
 *                            device, 0 if products of this shape take none (no stored entries, fewer
 *                            rows than waves, or a vector too long for LDS).
 *   macko_spmv_plan_build    fills plan[0 .. plan_entries) from row_ptr; plan 16-byte aligned, device
 *                            memory; plan_entries must be what macko_spmv_plan_entries returns.
 *                            Asynchronous on `stream`.
 *   macko_spmv_f16_planned, macko_spmv_f16_axpby_planned
 *                            as macko_spmv_f16 / macko_spmv_f16_axpby.  A plan of another size than this
 *                            launch needs (plan_entries 0, another device, another shape) is ignored
 *                            and the rows are searched as usual; results are the same either way,
 *                            bit for bit.  A plan built from another row_ptr is the caller's error,
 *                            like a wrong row_ptr.
 */
MACKO_API int macko_spmv_plan_entries(int32_t rows, int32_t cols, int64_t padded_entries, int32_t *entries);
MACKO_API int macko_spmv_plan_build(const int32_t *row_ptr, int32_t rows, int32_t cols,
                          int64_t padded_entries, int32_t *plan, int32_t plan_entries, void *stream);
MACKO_API int macko_spmv_f16_planned(const void *values, const void *deltas, const int32_t *row_ptr,
                           const int32_t *plan, int32_t plan_entries, const void *x, void *y,
                           int32_t rows, int32_t cols, int64_t padded_entries, void *stream);
MACKO_API int macko_spmv_f16_axpby_planned(const void *values, const void *deltas, const int32_t *row_ptr,
                                 const int32_t *plan, int32_t plan_entries, const void *x, void *y,
                                 int32_t rows, int32_t cols, int64_t padded_entries, float alpha,
                                 float beta, void *stream);

/*
 * Compressor, step 1 of 2.  Reads the dense row-major fp16 matrix `dense` [rows, cols] and
 * writes row_ptr[0..rows] (int32, device).  Asynchronous.  The caller then reads
 * n = row_ptr[rows] back (one 4-byte copy + stream sync), sizes values/deltas to
 * P = ceil(n/8)*8 and calls step 2.
 *
 * Steps 1+2 together replace compress_rows_cpu (src/macko_spmv/cuda/cpu_compressor.cuh:6-73)
 * and emit bit-identical arrays.
 */
MACKO_API int macko_compress_f16_count(const void *dense, int32_t rows, int32_t cols,
                             int32_t *row_ptr, void *stream);

/*
 * Step 1 with the total handed over: as macko_compress_f16_count, and when row_ptr is complete
 * the kernel also stores n = row_ptr[rows] to *total (a release store of system scope).  `total`
 * is any int32 the GPU can write; given page-locked host memory that the caller has set to -1, a
 * host thread can watch that word change instead of copying n back and synchronizing the stream,
 * which takes several microseconds less.  total == NULL behaves as macko_compress_f16_count.
 * No upstream counterpart (upstream's compressor runs on the host).
 */
MACKO_API int macko_compress_f16_count_total(const void *dense, int32_t rows, int32_t cols,
                                             int32_t *row_ptr, int32_t *total, void *stream);

/*
 * Compressor, step 2 of 2.  Fills values [P] (16-byte aligned) and deltas [P/2] (4-byte
 * aligned) from `dense` and the row_ptr produced by step 1; both arrays are fully written,
 * tail zero-filled, whatever they held before.  P must be ceil(row_ptr[rows]/8)*8.
 * Asynchronous.
 */
MACKO_API int macko_compress_f16_fill(const void *dense, int32_t rows, int32_t cols,
                            const int32_t *row_ptr, void *values, void *deltas,
                            int64_t padded_entries, void *stream);

/*
 * Y[b, :] = M X[b, :] for b < batch.  X is [batch, ldx] and Y [batch, ldy], row-major fp16 with
 * ldx >= cols and ldy >= rows (elements).  The matrix is streamed once per group of up to eight
 * vectors (as many as fit next to each other in LDS), the rest like macko_spmv_f16.  No
 * counterpart in the upstream package, whose LLM runner maps the single-vector operator over
 * the batch dimension (python_scripts/util_run_pruned_llm.py:112-118).
 */
MACKO_API int macko_spmv_f16_batched(const void *values, const void *deltas, const int32_t *row_ptr,
                           const void *x, void *y, int32_t rows, int32_t cols,
                           int64_t padded_entries, int32_t batch, int64_t ldx, int64_t ldy,
                           void *stream);

/*
 * Products whose input vector is produced on the fly while it is staged for the product, so a
 * decode step needs no launch for the producer.  No counterpart in the upstream package, whose
 * LLM runner leaves these parts to stock modules (python_scripts/util_run_pruned_llm.py:136-160).
 * Both need cols % 8 == 0, 16-byte aligned vector operands, and a vector that fits in LDS
 * (cols <= 81,000 or so); MACKO_E_INVALID_ARGUMENT otherwise.
 *
 * macko_spmv_f16_rmsnorm:        y = M n,  n[i] = fp16(x[i] * rsqrt(mean(x^2) + eps) * norm_weight[i])
 * macko_spmv_f16_silu_mul_axpby: y = alpha * M g + beta * y,  g[i] = fp16(silu(gate[i]) * up[i]);
 *                                with alpha == 1 and beta == 0, y is not read.
 */
MACKO_API int macko_spmv_f16_rmsnorm(const void *values, const void *deltas, const int32_t *row_ptr,
                           const void *x, const void *norm_weight, float eps, void *y,
                           int32_t rows, int32_t cols, int64_t padded_entries, void *stream);
MACKO_API int macko_spmv_f16_silu_mul_axpby(const void *values, const void *deltas, const int32_t *row_ptr,
                                  const void *gate, const void *up, void *y, int32_t rows,
                                  int32_t cols, int64_t padded_entries, float alpha, float beta,
                                  void *stream);

/*
 * int8 values variant.  Same arrays, except that `values` holds int8 [P] (8-byte aligned) and
 * `dense` is a row-major int8 matrix.  The compressor pair replaces compress_rows_int8_cpu
 * (src/macko_spmv/cuda/cpu_compressor.cuh:75-117), which differs from the fp16 one in keeping
 * the padding entries behind a row's last non-zero; the products replace
 * macko_spmv_int8<false> / <true> (src/macko_spmv/cuda/kernels.cuh:126-216; launched by
 * c_benchmarking/benchmark.cu:106-118): y = fp16(alpha * sum float(value) * float(x[col])
 * [+ beta * y]), fp32 accumulation.
 */
MACKO_API int macko_compress_i8_count(const void *dense, int32_t rows, int32_t cols,
                            int32_t *row_ptr, void *stream);
/* int8 twin of macko_compress_f16_count_total. */
MACKO_API int macko_compress_i8_count_total(const void *dense, int32_t rows, int32_t cols,
                                            int32_t *row_ptr, int32_t *total, void *stream);
MACKO_API int macko_compress_i8_fill(const void *dense, int32_t rows, int32_t cols,
                           const int32_t *row_ptr, void *values, void *deltas,
                           int64_t padded_entries, void *stream);
MACKO_API int macko_spmv_i8f16(const void *values, const void *deltas, const int32_t *row_ptr,
                     const void *x, void *y, int32_t rows, int32_t cols,
                     int64_t padded_entries, void *stream);
MACKO_API int macko_spmv_i8f16_axpby(const void *values, const void *deltas, const int32_t *row_ptr,
                           const void *x, void *y, int32_t rows, int32_t cols,
                           int64_t padded_entries, float alpha, float beta, void *stream);

/*
 * Inverse of the compressor: writes the dense row-major fp16 matrix [rows, cols] (every
 * element written; `dense` 2-byte aligned).  Uses the decode rule of the multiply kernel
 * (src/macko_spmv/cuda/kernels.cuh:97-103); the upstream package has no such function, it is
 * provided for round-trip checks at sizes a CPU decode cannot reach.  padded_entries = P bounds
 * what is read of values / deltas.  Launches kernels only (no memset), so it may be captured.
 */
MACKO_API int macko_decompress_f16(const void *values, const void *deltas, const int32_t *row_ptr,
                         int32_t rows, int32_t cols, int64_t padded_entries, void *dense,
                         void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MACKO_HIP_H */
