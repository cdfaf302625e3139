/*
 * macko_decode.h -- C ABI of the glue kernels the batch-1 decode harness runs between the
 * matrix-vector products (libmacko_hip.so).  None of them has a counterpart in the upstream
 * package: its harness (python_scripts/util_run_pruned_llm.py:136-160) runs stock Hugging Face
 * modules for these parts.  They exist so that a decode step on MI355X is dominated by the
 * projections rather than by dozens of launch-bound framework kernels.
 *
 * All pointers are device pointers; activations fp16, tables fp32; `position` points at one
 * int64 in device memory (read by the kernel, so a captured graph can be replayed per token);
 * `stream` is a hipStream_t passed as void*.  Return codes as in macko_hip.h.
 */
#ifndef MACKO_DECODE_H
#define MACKO_DECODE_H

#include <stdint.h>

#include "macko_hip.h" /* MACKO_API, return codes */

#ifdef __cplusplus
extern "C" {
#endif

/* y[i] = x[i] * rsqrt(mean(x^2) + eps) * weight[i], i < n. */
MACKO_API int macko_decode_rmsnorm_f16(const void *x, const void *weight, void *y, int32_t n, float eps,
                             void *stream);

/*
 * Rotary embedding (rotate-half pairing: element i with i + head_dim/2) of q and k at
 * *position; writes the rotated q to q_out and appends the rotated k and v to the caches
 * [n_heads, max_len, head_dim] at that position.  cos_table / sin_table: [max_len, head_dim/2].
 */
MACKO_API int macko_decode_rope_append_f16(const void *q, const void *k, const void *v,
                                 const float *cos_table, const float *sin_table,
                                 const int64_t *position, void *q_out, void *k_cache,
                                 void *v_cache, int32_t n_heads, int32_t head_dim,
                                 int32_t max_len, void *stream);

/*
 * Single-query attention per head over cache positions 0..*position:
 * out = softmax(scale * q K^T) V.  head_dim <= 256 and a multiple of 8, max_len <= 4096,
 * both caches 16-byte aligned.
 */
MACKO_API int macko_decode_attention_f16(const void *q, const void *k_cache, const void *v_cache,
                               const int64_t *position, void *out, int32_t n_heads,
                               int32_t head_dim, int32_t max_len, float scale, void *stream);

/*
 * macko_decode_rope_append_f16 followed by macko_decode_attention_f16 in one launch: q, k, v are
 * the raw projections of the current token, the caches receive the rotated k and v at *position,
 * out is the attention output.  Same limits as the two separate calls.
 */
MACKO_API int macko_decode_rope_attention_f16(const void *q, const void *k, const void *v,
                                    const float *cos_table, const float *sin_table,
                                    const int64_t *position, void *k_cache, void *v_cache,
                                    void *out, int32_t n_heads, int32_t head_dim, int32_t max_len,
                                    float scale, void *stream);

/* out[i] = silu(gate[i]) * up[i], i < n. */
MACKO_API int macko_decode_silu_mul_f16(const void *gate, const void *up, void *out, int32_t n,
                              void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MACKO_DECODE_H */
