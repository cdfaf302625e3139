// Glue kernels of the batch-1 decode harness (gfx950, wave64): everything a Llama-architecture
// decode step does between the projections, one launch each, so that the step is dominated by the
// matrix-vector products it is there to measure.  The upstream harness runs stock Hugging Face
// modules for these parts (python_scripts/util_run_pruned_llm.py:136-160); there is no upstream
// kernel to mirror.  All activations are fp16, all arithmetic fp32.  The current position is read
// from device memory so a captured HIP graph can be replayed for every token.

#include "macko_common.h"
#include "macko_decode.h"

namespace macko {
namespace {

__device__ __forceinline__ float h2f(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f2h(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }

// Sum over the workgroup (blockDim.x a multiple of 64, at most 1024); every thread gets the total.
// `scratch` is 16 floats that no other reduction of the same kernel uses (so no barrier is needed
// in front of the write).
__device__ __forceinline__ float block_sum(float v, float *scratch)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    const float w = wave_sum(v);
    if (lane == 0) scratch[wave] = w;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < n_waves; ++i) total += scratch[i];
    return total;
}

__device__ __forceinline__ float block_max(float v, float *scratch)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    float m = v;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if (lane == 0) scratch[wave] = m;
    __syncthreads();
    float total = scratch[0];
    for (int i = 1; i < n_waves; ++i) total = fmaxf(total, scratch[i]);
    return total;
}

// y = x * rsqrt(mean(x^2) + eps) * w, one workgroup.
__global__ void __launch_bounds__(1024) rmsnorm_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ w,
                                                       uint16_t *__restrict__ y, int n, float eps)
{
    __shared__ float scratch[16];
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = h2f(x[i]);
        ss += v * v;
    }
    const float inv = rsqrtf(block_sum(ss, scratch) / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += blockDim.x) y[i] = f2h(h2f(x[i]) * inv * h2f(w[i]));
}

// Rotary embedding of q and k (rotate-half convention: element i pairs with i + head_dim/2), k and
// v appended to the caches at the current position.  One workgroup per head, head_dim/2 threads.
// q, k, v: [n_heads * head_dim]; cos, sin: [max_len, head_dim/2] fp32; caches [n_heads, max_len, head_dim].
__global__ void rope_append_kernel(const uint16_t *__restrict__ q, const uint16_t *__restrict__ k,
                                   const uint16_t *__restrict__ v, const float *__restrict__ cos_table,
                                   const float *__restrict__ sin_table, const long long *__restrict__ position,
                                   uint16_t *__restrict__ q_out, uint16_t *__restrict__ k_cache,
                                   uint16_t *__restrict__ v_cache, int head_dim, int max_len)
{
    const int head = blockIdx.x, i = threadIdx.x, half = head_dim >> 1;
    long long pos = position[0];
    pos = pos < 0 ? 0 : (pos >= max_len ? max_len - 1 : pos);
    const float c = cos_table[pos * half + i], s = sin_table[pos * half + i];
    const size_t in = (size_t)head * head_dim;
    const size_t slot = ((size_t)head * max_len + (size_t)pos) * head_dim;
    const float q0 = h2f(q[in + i]), q1 = h2f(q[in + i + half]);
    q_out[in + i] = f2h(q0 * c - q1 * s);
    q_out[in + i + half] = f2h(q1 * c + q0 * s);
    const float k0 = h2f(k[in + i]), k1 = h2f(k[in + i + half]);
    k_cache[slot + i] = f2h(k0 * c - k1 * s);
    k_cache[slot + i + half] = f2h(k1 * c + k0 * s);
    v_cache[slot + i] = v[in + i];
    v_cache[slot + i + half] = v[in + i + half];
}

// Single-query attention over positions 0..position of one head per workgroup (512 threads):
// scores, softmax, weighted sum of v.  head_dim <= 256 and a multiple of 8; max_len <= kMaxLen.
// With ROPE the kernel first does what rope_append_kernel does for its head (q, k, v are then the
// raw projections; the rotated q is rounded to fp16 as if it had been written out), so a decode
// step needs one launch for both.  The row it appends is used from LDS, not read back.
// The kernel is latency-bound (a head's cache is a few hundred KB), so what matters is how few
// dependent memory round trips there are: HD = head_dim as a compile-time constant lets a thread
// issue all loads of its k row at once (HD = 0: any head_dim, loops of runtime length), and the k
// row of a thread's first position and the v pieces of its first kVPre positions are requested
// before anything else is computed, together with q, k, v of the new token.
constexpr int kAttnThreads = 512;
constexpr int kMaxLen = 4096;
constexpr int kVPre = 8;
template <bool ROPE, int HD>
__global__ void __launch_bounds__(kAttnThreads) attention_kernel(const uint16_t *__restrict__ q,
                                                                  const uint16_t *__restrict__ k_new,
                                                                  const uint16_t *__restrict__ v_new,
                                                                  const float *__restrict__ cos_table,
                                                                  const float *__restrict__ sin_table,
                                                                  uint16_t *k_cache, uint16_t *v_cache,
                                                                  const long long *__restrict__ position,
                                                                  uint16_t *__restrict__ out, int head_dim_arg,
                                                                  int max_len, float scale)
{
    __shared__ float scores[kMaxLen];
    __shared__ __attribute__((aligned(16))) float qs[256];
    __shared__ __attribute__((aligned(16))) uint16_t ks[256];  // the appended row (ROPE only)
    __shared__ __attribute__((aligned(16))) uint16_t vs[256];
    __shared__ float partial[kAttnThreads * 8];  // groups x head_dim
    __shared__ float max_scratch[16], sum_scratch[16];
    const int head_dim = HD ? HD : head_dim_arg;
    const int head = blockIdx.x, tid = threadIdx.x;
    long long pos = position[0];
    pos = pos < 0 ? 0 : (pos >= max_len ? max_len - 1 : pos);
    const int len = (int)pos + 1;
    const int own = ROPE ? (int)pos : -1;  // the row this launch appends
    const uint16_t *kh = k_cache + (size_t)head * max_len * head_dim;
    const uint16_t *vh = v_cache + (size_t)head * max_len * head_dim;
    const int lanes_per_row = head_dim >> 3;
    const int groups = kAttnThreads / lanes_per_row;
    const int g = tid / lanes_per_row, j = tid - g * lanes_per_row;

    // ---- cache loads that depend on nothing computed here -------------------------------------------
    constexpr int NV = HD > 0 ? HD / 8 : 1;
    u32x4 kpre[NV];
    if (HD > 0) {
        const bool fetch = tid < len && tid != own;
        const u32x4 *row = reinterpret_cast<const u32x4 *>(kh + (size_t)tid * head_dim);
#pragma unroll
        for (int jj = 0; jj < NV; ++jj) kpre[jj] = fetch ? row[jj] : u32x4{0, 0, 0, 0};
    }
    u32x4 vpre[kVPre];
#pragma unroll
    for (int u = 0; u < kVPre; ++u) {
        const int pu = g + u * groups;
        const bool fetch = g < groups && pu < len && pu != own;
        vpre[u] = fetch ? reinterpret_cast<const u32x4 *>(vh + (size_t)pu * head_dim)[j] : u32x4{0, 0, 0, 0};
    }

    // ---- q (rotated with ROPE), and the new cache row -------------------------------------------------
    if (ROPE) {
        const int half = head_dim >> 1;
        if (tid < half) {
            const int i = tid;
            const float c = cos_table[pos * half + i], s = sin_table[pos * half + i];
            const size_t in = (size_t)head * head_dim;
            const size_t slot = ((size_t)head * max_len + (size_t)pos) * head_dim;
            const float q0 = h2f(q[in + i]), q1 = h2f(q[in + i + half]);
            qs[i] = h2f(f2h(q0 * c - q1 * s)) * scale;
            qs[i + half] = h2f(f2h(q1 * c + q0 * s)) * scale;
            const float k0 = h2f(k_new[in + i]), k1 = h2f(k_new[in + i + half]);
            const uint16_t r0 = f2h(k0 * c - k1 * s), r1 = f2h(k1 * c + k0 * s);
            const uint16_t v0 = v_new[in + i], v1 = v_new[in + i + half];
            ks[i] = r0;
            ks[i + half] = r1;
            vs[i] = v0;
            vs[i + half] = v1;
            k_cache[slot + i] = r0;
            k_cache[slot + i + half] = r1;
            v_cache[slot + i] = v0;
            v_cache[slot + i + half] = v1;
        }
    } else if (tid < head_dim) {
        qs[tid] = h2f(q[(size_t)head * head_dim + tid]) * scale;
    }
    __syncthreads();

    // ---- scores -----------------------------------------------------------------------------------------
    auto dot8 = [&](const u32x4 kv, int jj, float acc) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            acc += h2f((uint16_t)(kv[e] & 0xffffu)) * qs[8 * jj + 2 * e];
            acc += h2f((uint16_t)(kv[e] >> 16)) * qs[8 * jj + 2 * e + 1];
        }
        return acc;
    };
    float local_max = -3.0e38f;
    for (int p = tid; p < len; p += kAttnThreads) {
        float acc = 0.f;
        if (p == own) {
            for (int jj = 0; jj < lanes_per_row; ++jj) acc = dot8(reinterpret_cast<const u32x4 *>(ks)[jj], jj, acc);
        } else if (HD > 0) {
            if (p != tid) {  // beyond the row requested up front
                const u32x4 *row = reinterpret_cast<const u32x4 *>(kh + (size_t)p * head_dim);
#pragma unroll
                for (int jj = 0; jj < NV; ++jj) kpre[jj] = row[jj];
            }
#pragma unroll
            for (int jj = 0; jj < NV; ++jj) acc = dot8(kpre[jj], jj, acc);
        } else {
            const u32x4 *row = reinterpret_cast<const u32x4 *>(kh + (size_t)p * head_dim);
            for (int jj = 0; jj < lanes_per_row; ++jj) acc = dot8(row[jj], jj, acc);
        }
        scores[p] = acc;
        local_max = fmaxf(local_max, acc);
    }
    const float m = block_max(local_max, max_scratch);
    float local_sum = 0.f;
    for (int p = tid; p < len; p += kAttnThreads) {
        const float e = __expf(scores[p] - m);
        scores[p] = e;
        local_sum += e;
    }
    const float inv = 1.0f / block_sum(local_sum, sum_scratch);  // also orders the scores[] writes

    // ---- weighted sum of v: a thread owns 8 consecutive dims (one 16-byte piece per position) of the
    //      positions p = g, g + groups, ...; the groups' partial sums meet in LDS --------------------------
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto add_row = [&](const u32x4 vv, float wgt) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            acc[2 * e] += wgt * h2f((uint16_t)(vv[e] & 0xffffu));
            acc[2 * e + 1] += wgt * h2f((uint16_t)(vv[e] >> 16));
        }
    };
    if (g < groups) {
#pragma unroll
        for (int u = 0; u < kVPre; ++u) {
            const int pu = g + u * groups;
            if (pu < len) add_row(pu == own ? reinterpret_cast<const u32x4 *>(vs)[j] : vpre[u], scores[pu]);
        }
        for (int p = g + kVPre * groups; p < len; p += 4 * groups) {
            u32x4 vv[4];
            float wgt[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int pu = p + u * groups;
                const bool ok = pu < len;
                vv[u] = !ok ? u32x4{0, 0, 0, 0}
                            : (pu == own ? reinterpret_cast<const u32x4 *>(vs)[j]
                                         : reinterpret_cast<const u32x4 *>(vh + (size_t)pu * head_dim)[j]);
                wgt[u] = ok ? scores[pu] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) add_row(vv[u], wgt[u]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) partial[g * head_dim + 8 * j + e] = acc[e];
    }
    __syncthreads();
    if (tid < head_dim) {
        float total = 0.f;
        for (int gg = 0; gg < groups; ++gg) total += partial[gg * head_dim + tid];
        out[(size_t)head * head_dim + tid] = f2h(total * inv);
    }
}

template <bool ROPE>
void launch_attention(const void *q, const void *k, const void *v, const float *cos_table, const float *sin_table,
                      void *k_cache, void *v_cache, const int64_t *position, void *out, int n_heads, int head_dim,
                      int max_len, float scale, hipStream_t stream)
{
#define MACKO_ATTN(HD_)                                                                                         \
    hipLaunchKernelGGL((attention_kernel<ROPE, HD_>), dim3(n_heads), dim3(kAttnThreads), 0, stream,             \
                       (const uint16_t *)q, (const uint16_t *)k, (const uint16_t *)v, cos_table, sin_table,      \
                       (uint16_t *)k_cache, (uint16_t *)v_cache, (const long long *)position, (uint16_t *)out,   \
                       head_dim, max_len, scale)
    if (head_dim == 128)
        MACKO_ATTN(128);
    else if (head_dim == 64)
        MACKO_ATTN(64);
    else
        MACKO_ATTN(0);
#undef MACKO_ATTN
}

// out[i] = silu(gate[i]) * up[i]
__global__ void silu_mul_kernel(const uint16_t *__restrict__ gate, const uint16_t *__restrict__ up,
                                uint16_t *__restrict__ out, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float gv = h2f(gate[i]);
        out[i] = f2h(gv / (1.0f + __expf(-gv)) * h2f(up[i]));
    }
}

}  // namespace
}  // namespace macko

extern "C" int macko_decode_rmsnorm_f16(const void *x, const void *weight, void *y, int32_t n, float eps, void *stream)
{
    using namespace macko;
    if (x == nullptr || weight == nullptr || y == nullptr || n <= 0) return MACKO_E_INVALID_ARGUMENT;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(1), dim3(1024), 0, as_stream(stream), (const uint16_t *)x,
                       (const uint16_t *)weight, (uint16_t *)y, n, eps);
    return (int)hipGetLastError();
}

extern "C" int macko_decode_rope_append_f16(const void *q, const void *k, const void *v, const float *cos_table,
                                            const float *sin_table, const int64_t *position, void *q_out,
                                            void *k_cache, void *v_cache, int32_t n_heads, int32_t head_dim,
                                            int32_t max_len, void *stream)
{
    using namespace macko;
    if (!q || !k || !v || !cos_table || !sin_table || !position || !q_out || !k_cache || !v_cache)
        return MACKO_E_INVALID_ARGUMENT;
    if (n_heads <= 0 || head_dim <= 0 || (head_dim & 1) || head_dim > 2048 || max_len <= 0)
        return MACKO_E_INVALID_ARGUMENT;
    hipLaunchKernelGGL(rope_append_kernel, dim3(n_heads), dim3(head_dim / 2), 0, as_stream(stream),
                       (const uint16_t *)q, (const uint16_t *)k, (const uint16_t *)v, cos_table, sin_table,
                       (const long long *)position, (uint16_t *)q_out, (uint16_t *)k_cache, (uint16_t *)v_cache,
                       head_dim, max_len);
    return (int)hipGetLastError();
}

extern "C" int macko_decode_attention_f16(const void *q, const void *k_cache, const void *v_cache,
                                          const int64_t *position, void *out, int32_t n_heads, int32_t head_dim,
                                          int32_t max_len, float scale, void *stream)
{
    using namespace macko;
    if (!q || !k_cache || !v_cache || !position || !out) return MACKO_E_INVALID_ARGUMENT;
    if (n_heads <= 0 || head_dim <= 0 || head_dim > 256 || (head_dim & 7) || max_len <= 0 || max_len > kMaxLen)
        return MACKO_E_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(k_cache) & 15) || (reinterpret_cast<uintptr_t>(v_cache) & 15))
        return MACKO_E_INVALID_ARGUMENT;
    launch_attention<false>(q, nullptr, nullptr, nullptr, nullptr, const_cast<void *>(k_cache),
                            const_cast<void *>(v_cache), position, out, n_heads, head_dim, max_len, scale,
                            as_stream(stream));
    return (int)hipGetLastError();
}

extern "C" int macko_decode_rope_attention_f16(const void *q, const void *k, const void *v, const float *cos_table,
                                               const float *sin_table, const int64_t *position, void *k_cache,
                                               void *v_cache, void *out, int32_t n_heads, int32_t head_dim,
                                               int32_t max_len, float scale, void *stream)
{
    using namespace macko;
    if (!q || !k || !v || !cos_table || !sin_table || !position || !k_cache || !v_cache || !out)
        return MACKO_E_INVALID_ARGUMENT;
    if (n_heads <= 0 || head_dim <= 0 || head_dim > 256 || (head_dim & 7) || max_len <= 0 || max_len > kMaxLen)
        return MACKO_E_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(k_cache) & 15) || (reinterpret_cast<uintptr_t>(v_cache) & 15))
        return MACKO_E_INVALID_ARGUMENT;
    launch_attention<true>(q, k, v, cos_table, sin_table, k_cache, v_cache, position, out, n_heads, head_dim,
                           max_len, scale, as_stream(stream));
    return (int)hipGetLastError();
}

extern "C" int macko_decode_silu_mul_f16(const void *gate, const void *up, void *out, int32_t n, void *stream)
{
    using namespace macko;
    if (!gate || !up || !out || n <= 0) return MACKO_E_INVALID_ARGUMENT;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((n + 255) / 256), dim3(256), 0, as_stream(stream),
                       (const uint16_t *)gate, (const uint16_t *)up, (uint16_t *)out, n);
    return (int)hipGetLastError();
}
