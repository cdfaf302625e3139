// MACKO fp16 sparse matrix-vector product for gfx950 (wave64).
//
// Work split.  The launch has W = gridDim.x * (BLOCK/64) waves.  Wave w owns the rows whose
// first entry index lies in [w*P/W, (w+1)*P/W): contiguous whole rows, balanced by stored
// entries, found by a 64-wide search of row_ptr.  No two waves share a row, so there is no
// cross-wave reduction and no scratch memory.
//
// Per row a wave walks the row's 8-entry chunks 64 at a time (one chunk per lane: one 128-bit
// value load and one 32-bit delta load), D such passes in flight.  Columns come from a DPP
// prefix sum over per-lane nibble sums plus v_dot8_u32_u4 for the running sum inside a lane; the
// dense vector is gathered from LDS, where the workgroup staged it once.  fp32 accumulation,
// one DPP reduction per row, fp16 store.
//
// Behaviour restated from src/macko_spmv/cuda/kernels.cuh:34-124 of the upstream package.

#include "macko_common.h"

namespace macko {
namespace {

constexpr int kLdsFront = 16;   // zero bytes in front of x in LDS (masked head entries read here)
constexpr int kLdsBack = 64;    // zero bytes behind x (masked tail entries read here)

struct SpmvArgs {
    const u32 *values;      // fp16 pairs
    const u32 *deltas;      // 8 nibbles per word
    const int *row_ptr;
    const uint16_t *x;
    uint16_t *y;
    int rows;
    int cols;
    long long padded;       // P
    float alpha;
    float beta;
};

__device__ __forceinline__ float half_bits_to_float(uint16_t h)
{
    return (float)__builtin_bit_cast(_Float16, h);
}

__device__ __forceinline__ uint16_t float_to_half_bits(float f)
{
    return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// Smallest r in [0, rows] with row_ptr[r] >= target (rows if there is none), for two targets
// at once.  All 64 lanes probe together; `guess` centres the first probe window, which hits
// when rows carry similar entry counts.  Every value here is wave-uniform.
__device__ __forceinline__ void wave_lower_bound2(const int *__restrict__ row_ptr, int rows, int lane,
                                                  const int target[2], const int guess[2], int out[2])
{
    int lo[2], hi[2];
    int probe[2], win[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        int w0 = guess[k] - 32;
        int wmax = rows - 63;
        w0 = w0 > wmax ? wmax : w0;
        w0 = w0 < 0 ? 0 : w0;
        win[k] = w0;
        int idx = w0 + lane;
        probe[k] = idx <= rows ? row_ptr[idx] : 0x7fffffff;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        unsigned long long m = __ballot(probe[k] >= target[k]);
        if (m == 0) {  // everything probed is below the target
            lo[k] = win[k] + 64 > rows ? rows : win[k] + 64;
            hi[k] = rows;
        } else {
            int f = __builtin_ctzll(m);
            if (f == 0) {  // the answer is at or before the window start
                lo[k] = 0;
                hi[k] = win[k];
            } else {
                lo[k] = hi[k] = win[k] + f > rows ? rows : win[k] + f;
            }
        }
    }
    while (lo[0] < hi[0] || lo[1] < hi[1]) {
        int step[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            step[k] = (hi[k] - lo[k] + 63) >> 6;
            int idx = lo[k] + lane * step[k];
            probe[k] = (lo[k] < hi[k] && idx < hi[k]) ? row_ptr[idx] : 0x7fffffff;
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            if (lo[k] < hi[k]) {
                unsigned long long m = __ballot(probe[k] >= target[k]);
                if (m == 0) {
                    lo[k] = lo[k] + 63 * step[k] + 1;
                } else {
                    int f = __builtin_ctzll(m);
                    int at = lo[k] + f * step[k];
                    if (f > 0) lo[k] = lo[k] + (f - 1) * step[k] + 1;
                    if (at < hi[k]) hi[k] = at;
                }
                if (lo[k] > hi[k]) lo[k] = hi[k];
            }
        }
    }
    out[0] = lo[0];
    out[1] = lo[1];
}

// Copy x[0..cols) into LDS behind kLdsFront zero bytes and put kLdsBack zero bytes after it.
template <int BLOCK>
__device__ __forceinline__ void stage_x(unsigned char *lds, const uint16_t *__restrict__ x, int cols, int tid)
{
    uint16_t *dst = reinterpret_cast<uint16_t *>(lds + kLdsFront);
    if (tid < kLdsFront / 4) reinterpret_cast<u32 *>(lds)[tid] = 0;
    if (tid < kLdsBack / 2) dst[cols + tid] = 0;
    if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        const int nvec = cols >> 3;
        const u32x4 *src = reinterpret_cast<const u32x4 *>(x);
        u32x4 *d4 = reinterpret_cast<u32x4 *>(dst);
        for (int i = tid; i < nvec; i += BLOCK) d4[i] = src[i];
        for (int i = (nvec << 3) + tid; i < cols; i += BLOCK) dst[i] = x[i];
    } else {
        for (int i = tid; i < cols; i += BLOCK) dst[i] = x[i];
    }
}

// 128-bit mask helpers: keep halves [from, 8) / [0, upto) of a 4-dword vector.
__device__ __forceinline__ void mask_from(u32x4 &v, u32 &d, int from)
{
    unsigned long long lo = from < 4 ? (~0ull << (16 * from)) : 0ull;
    unsigned long long hi = from < 4 ? ~0ull : (~0ull << (16 * (from - 4)));
    v.x &= (u32)lo;
    v.y &= (u32)(lo >> 32);
    v.z &= (u32)hi;
    v.w &= (u32)(hi >> 32);
    d &= ~0u << (4 * from);
}

__device__ __forceinline__ void mask_upto(u32x4 &v, u32 &d, int upto)  // 1 <= upto <= 7
{
    unsigned long long lo = upto < 4 ? ((1ull << (16 * upto)) - 1) : ~0ull;
    unsigned long long hi = upto <= 4 ? 0ull : ((1ull << (16 * (upto - 4))) - 1);
    v.x &= (u32)lo;
    v.y &= (u32)(lo >> 32);
    v.z &= (u32)hi;
    v.w &= (u32)(hi >> 32);
    d &= (1u << (4 * upto)) - 1;
}

template <int BLOCK, int D, bool X_LDS, bool AXPBY>
__global__ void __launch_bounds__(BLOCK) spmv_rows_kernel(const SpmvArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    constexpr int WAVES = BLOCK / kWave;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = uniform(tid >> 6);
    const int n_waves = gridDim.x * WAVES;
    const int gw = blockIdx.x * WAVES + wave;

    // ---- which rows are mine -------------------------------------------------------------
    int range[2];
    {
        int target[2], guess[2];
        target[0] = (int)(((long long)gw * a.padded) / n_waves);
        target[1] = (int)(((long long)(gw + 1) * a.padded) / n_waves);
        guess[0] = (int)(((long long)gw * a.rows) / n_waves);
        guess[1] = (int)(((long long)(gw + 1) * a.rows) / n_waves);
        wave_lower_bound2(a.row_ptr, a.rows, lane, target, guess, range);
        if (gw == 0) range[0] = 0;
        if (gw == n_waves - 1) range[1] = a.rows;
    }
    const int row_first = uniform(range[0]);
    const int row_last = uniform(range[1]);

    if (X_LDS) {
        stage_x<BLOCK>(lds, a.x, a.cols, tid);
        __syncthreads();
    }

    const __amdgpu_buffer_rsrc_t rs_values =
        __builtin_amdgcn_make_buffer_rsrc((void *)a.values, 0, (int)(u32)(a.padded * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_deltas =
        __builtin_amdgcn_make_buffer_rsrc((void *)a.deltas, 0, (int)(a.padded / 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x =
        __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.cols * 2, 0x00020000);
    (void)rs_x;

    for (int r0 = row_first; r0 < row_last; r0 += kWave - 1) {
        const int batch = uniform(row_last - r0 < kWave - 1 ? row_last - r0 : kWave - 1);
        int idx = r0 + lane;
        idx = idx > a.rows ? a.rows : idx;
        const int rp = a.row_ptr[idx];  // lane i: start of row r0 + i
        for (int i = 0; i < batch; ++i) {
            const int e0 = __builtin_amdgcn_readlane(rp, i);
            const int e1 = __builtin_amdgcn_readlane(rp, i + 1);
            float acc0 = 0.f, acc1 = 0.f;
            if (e1 > e0) {
                const int cb = e0 >> 3;
                const int ce = (e1 + 7) >> 3;
                const int head = e0 & 7;
                const int tail = e1 & 7;
                int carry = 0;  // nibble sum of the row so far
                for (int c0 = cb; c0 < ce; c0 += kWave * D) {
                    u32x4 v[D];
                    u32 d[D];
#pragma unroll
                    for (int j = 0; j < D; ++j) {
                        const int t0 = c0 + kWave * j;
                        v[j] = (u32x4){0, 0, 0, 0};
                        d[j] = 0;
                        if (t0 + lane < ce) {
                            v[j] = __builtin_amdgcn_raw_buffer_load_b128(rs_values, lane * 16, (int)((u32)t0 * 16u), 0);
                            d[j] = __builtin_amdgcn_raw_buffer_load_b32(rs_deltas, lane * 4, t0 * 4, 0);
                        }
                    }
#pragma unroll
                    for (int j = 0; j < D; ++j) {
                        const int t0 = c0 + kWave * j;
                        if (t0 < ce) {
                            u32x4 vj = v[j];
                            u32 dj = d[j];
                            if (t0 == cb && head != 0) {
                                if (lane == 0) mask_from(vj, dj, head);
                            }
                            if (tail != 0 && ce - 1 - t0 < kWave) {
                                if (lane == ce - 1 - t0) mask_upto(vj, dj, tail);
                            }
                            const int s = (int)__builtin_amdgcn_udot8(dj, 0x11111111u, 0u, false);
                            const int incl = wave_scan_inclusive(s);
                            const int excl = incl - s + carry;
                            carry += __builtin_amdgcn_readlane(incl, kWave - 1);
                            if (t0 + lane < ce) {
                                // LDS byte address of x[col] for entry 0 of this chunk, before its own
                                // nibble is added; 8c - e0 >= -7, so this stays positive
                                const u32 base = (u32)(kLdsFront + 2 * (8 * (t0 + lane) - e0 + excl));
                                const u32 m[8] = {0x2u,      0x22u,      0x222u,      0x2222u,
                                                  0x22222u,  0x222222u,  0x2222222u,  0x22222222u};
#pragma unroll
                                for (int k = 0; k < 8; ++k) {
                                    const u32 addr = __builtin_amdgcn_udot8(dj, m[k], base, false);
                                    uint16_t xb;
                                    if (X_LDS) {
                                        xb = *reinterpret_cast<const uint16_t *>(lds + addr + 2 * k);
                                    } else {
                                        int o = (int)addr + 2 * k - kLdsFront;
                                        const int omax = 2 * a.cols - 2;
                                        o = o < 0 ? 0 : (o > omax ? omax : o);
                                        xb = __builtin_amdgcn_raw_buffer_load_b16(rs_x, o, 0, 0);
                                    }
                                    const u32 w = vj[k >> 1];
                                    const uint16_t mb = (k & 1) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu);
                                    if (k & 1)
                                        acc1 = __builtin_fmaf(half_bits_to_float(mb), half_bits_to_float(xb), acc1);
                                    else
                                        acc0 = __builtin_fmaf(half_bits_to_float(mb), half_bits_to_float(xb), acc0);
                                }
                            }
                        }
                    }
                }
            }
            const float total = wave_sum(acc0 + acc1);
            if (lane == 0) {
                float out = total;
                if (AXPBY) out = a.alpha * total + a.beta * half_bits_to_float(a.y[r0 + i]);
                a.y[r0 + i] = float_to_half_bits(out);
            }
        }
    }
}

// y[r] = 0 (or beta*y[r]) for matrices without stored entries.
template <bool AXPBY>
__global__ void spmv_empty_kernel(uint16_t *y, int rows, float beta)
{
    int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r < rows) y[r] = AXPBY ? float_to_half_bits(beta * half_bits_to_float(y[r])) : (uint16_t)0;
}

template <int BLOCK, int D, bool X_LDS, bool AXPBY>
int launch_rows(const SpmvArgs &a, int grid, size_t lds_bytes, hipStream_t stream)
{
    auto kernel = spmv_rows_kernel<BLOCK, D, X_LDS, AXPBY>;
    if (lds_bytes > 64 * 1024) {
        // one-time opt-in to more than 64 KiB of dynamic LDS, per device
        static bool done[64] = {};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return (int)e;
        if (dev < 0 || dev >= 64 || !done[dev]) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            if (dev >= 0 && dev < 64) done[dev] = true;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(BLOCK), lds_bytes, stream, a);
    return (int)hipGetLastError();
}

template <bool AXPBY>
int spmv_dispatch(const SpmvArgs &a, hipStream_t stream)
{
    if (a.rows == 0) return 0;
    if (a.padded == 0) {
        hipLaunchKernelGGL(spmv_empty_kernel<AXPBY>, dim3((a.rows + 255) / 256), dim3(256), 0, stream, a.y,
                           a.rows, a.beta);
        return (int)hipGetLastError();
    }
    DeviceInfo info;
    int rc = device_info(&info);
    if (rc != 0) return rc;

    constexpr int BLOCK = 1024;
    constexpr int WAVES = BLOCK / kWave;
    int grid = (a.rows + WAVES - 1) / WAVES;
    if (grid > info.compute_units) grid = info.compute_units;
    if (grid < 1) grid = 1;

    const size_t lds_need = (size_t)kLdsFront + 2 * (size_t)a.cols + kLdsBack;
    if (lds_need <= (size_t)info.max_lds_bytes)
        return launch_rows<BLOCK, 4, true, AXPBY>(a, grid, lds_need, stream);
    return launch_rows<BLOCK, 4, false, AXPBY>(a, grid, 0, stream);
}

int check_spmv_args(const void *values, const void *deltas, const int32_t *row_ptr, const void *x, void *y,
                    int32_t rows, int32_t cols, int64_t padded)
{
    if (rows < 0 || cols < 0 || padded < 0) return MACKO_E_INVALID_ARGUMENT;
    if (padded % kChunk != 0) return MACKO_E_INVALID_ARGUMENT;
    if (padded >= (1ll << 31)) return MACKO_E_INVALID_ARGUMENT;
    if (rows > 0 && (row_ptr == nullptr || y == nullptr)) return MACKO_E_INVALID_ARGUMENT;
    if (padded > 0 && (values == nullptr || deltas == nullptr || x == nullptr || cols == 0))
        return MACKO_E_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(values) & 15) || (reinterpret_cast<uintptr_t>(deltas) & 3) ||
        (reinterpret_cast<uintptr_t>(row_ptr) & 3) || (reinterpret_cast<uintptr_t>(x) & 1) ||
        (reinterpret_cast<uintptr_t>(y) & 1))
        return MACKO_E_INVALID_ARGUMENT;
    return 0;
}

}  // namespace
}  // namespace macko

extern "C" int macko_spmv_f16(const void *values, const void *deltas, const int32_t *row_ptr, const void *x,
                              void *y, int32_t rows, int32_t cols, int64_t padded_entries, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries);
    if (rc != 0) return rc;
    SpmvArgs a{(const u32 *)values, (const u32 *)deltas, row_ptr, (const uint16_t *)x, (uint16_t *)y,
               rows,                cols,                padded_entries, 1.0f,          0.0f};
    return spmv_dispatch<false>(a, as_stream(stream));
}

extern "C" int macko_spmv_f16_axpby(const void *values, const void *deltas, const int32_t *row_ptr,
                                    const void *x, void *y, int32_t rows, int32_t cols,
                                    int64_t padded_entries, float alpha, float beta, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries);
    if (rc != 0) return rc;
    SpmvArgs a{(const u32 *)values, (const u32 *)deltas, row_ptr, (const uint16_t *)x, (uint16_t *)y,
               rows,                cols,                padded_entries, alpha,         beta};
    return spmv_dispatch<true>(a, as_stream(stream));
}
