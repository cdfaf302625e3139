// MACKO compressors (fp16 and int8 values) and fp16 decompressor for gfx950 (wave64).
//
// The fp16 format is restated from src/macko_spmv/cuda/cpu_compressor.cuh:6-73 of the upstream
// package as a per-column rule that needs no sequential walk:
//   column x of a row stores an entry when its element is non-zero as a float (so -0.0 does
//   not count and NaN does), or when x - p is a positive multiple of 16, p being the column
//   of the previous non-zero (-1 before the first) -- a padding entry.  The nibble of a
//   non-zero is (x - p - 1) & 15, of a padding entry 15.  Entries after the row's last
//   non-zero are not stored.  A stored element keeps its bits (a padding entry keeps the sign
//   of its zero); a NaN is stored as 0x7fff, the result of CUDA's float->half conversion that
//   the upstream code routes every value through.
//
// The int8 format (compress_rows_int8_cpu, cpu_compressor.cuh:75-117) follows the same rule on
// int8 elements, except that the padding entries after a row's last non-zero ARE stored.
//
// Pass 1 (count_rows_kernel + scan_rows_kernel) produces row_ptr; pass 2 (fill_rows_kernel)
// writes values and nibbles.  One wave owns one row in both passes; lanes take 8 consecutive
// columns and learn the previous non-zero's column from a DPP running maximum.

#include "macko_common.h"

namespace macko {
namespace {

constexpr int kRowsPerBlock = 4;              // waves per workgroup, one row each
constexpr int kBlock = kRowsPerBlock * kWave;
constexpr int kNoColumn = (int)0x80000000;

// The two element formats.  A chunk is the 8 consecutive elements a lane handles per tile.
struct Fp16Format {
    typedef uint16_t Elem;
    typedef u32x4 Chunk;                          // 8 halves
    static constexpr bool kKeepTrailing = false;  // padding entries behind the last non-zero are dropped
    static __device__ __forceinline__ u32 at(const Chunk &v, int i) { return (v[i >> 1] >> (16 * (i & 1))) & 0xffffu; }
    static __device__ __forceinline__ void put(Chunk &v, int i, u32 bits) { v[i >> 1] |= bits << (16 * (i & 1)); }
    // non-zero as a float: -0.0 is a zero, NaN is not
    static __device__ __forceinline__ bool nonzero(u32 bits) { return (bits & 0x7fffu) != 0; }
    // what is stored: the element itself, a NaN as 0x7fff
    static __device__ __forceinline__ u32 stored(u32 bits) { return (bits & 0x7fffu) > 0x7c00u ? 0x7fffu : bits; }
};
struct Int8Format {
    typedef unsigned char Elem;
    typedef u32x2 Chunk;                         // 8 bytes
    static constexpr bool kKeepTrailing = true;  // cpu_compressor.cuh:75-117 has no withdrawal step
    static __device__ __forceinline__ u32 at(const Chunk &v, int i) { return (v[i >> 2] >> (8 * (i & 3))) & 0xffu; }
    static __device__ __forceinline__ void put(Chunk &v, int i, u32 bits) { v[i >> 2] |= bits << (8 * (i & 3)); }
    static __device__ __forceinline__ bool nonzero(u32 bits) { return bits != 0; }
    static __device__ __forceinline__ u32 stored(u32 bits) { return bits; }
};

// 8 consecutive elements of a row, zero beyond `cols`.  STREAM: the dense matrix will not be read
// again soon (non-temporal hint).
template <typename F, bool STREAM>
__device__ __forceinline__ typename F::Chunk load8(const typename F::Elem *__restrict__ row, int col, int cols,
                                                   bool vector_ok)
{
    typename F::Chunk v = {};
    if (col + 8 <= cols && vector_ok) {
        const typename F::Chunk *p = reinterpret_cast<const typename F::Chunk *>(row + col);
        v = STREAM ? __builtin_nontemporal_load(p) : *p;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const u32 h = (col + i < cols) ? (u32)row[col + i] : 0u;
            F::put(v, i, h);
        }
    }
    return v;
}

// bit i set when element i is non-zero
template <typename F>
__device__ __forceinline__ u32 nonzero_bits(const typename F::Chunk &v)
{
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) m |= (F::nonzero(F::at(v, i)) ? 1u : 0u) << i;
    return m;
}

// Column of the last non-zero strictly before this lane's chunk, given the lane's own last
// non-zero column (kNoColumn if none) and the carry from earlier passes.  Also returns the
// last non-zero column of the whole pass through `pass_last`.
__device__ __forceinline__ int previous_nonzero(int own_last, int carry, int lane, int &pass_last)
{
    const int incl = wave_scan_max_inclusive(own_last);
    pass_last = __builtin_amdgcn_readlane(incl, kWave - 1);
    int before = __shfl_up(incl, 1);
    before = lane == 0 ? kNoColumn : before;
    return before > carry ? before : carry;
}

__device__ __forceinline__ int wave_sum_int(int x)
{
    return __builtin_amdgcn_readlane(wave_scan_inclusive(x), kWave - 1);
}

template <typename F, bool STREAM>
__global__ void __launch_bounds__(kBlock) count_rows_kernel(const typename F::Elem *__restrict__ dense, int rows,
                                                            int cols, int *__restrict__ counts)
{
    typedef typename F::Elem Elem;
    typedef typename F::Chunk Chunk;
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + uniform(threadIdx.x >> 6);
    if (row >= rows) return;
    const Elem *src = dense + (size_t)row * (size_t)cols;
    const bool vector_ok = (reinterpret_cast<uintptr_t>(src) & (sizeof(Chunk) - 1)) == 0;
    int carry = -1;  // column of the last non-zero seen in earlier passes
    int mine = 0;
    for (int c0 = 0; c0 < cols; c0 += kTile) {
        const int col = c0 + lane * kChunk;
        const Chunk v = load8<F, STREAM>(src, col, cols, vector_ok && col < cols);
        const u32 nz = nonzero_bits<F>(v);
        const int own_last = nz ? col + 31 - __builtin_clz(nz) : kNoColumn;
        int pass_last;
        int p = previous_nonzero(own_last, carry, lane, pass_last);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (nz & (1u << i)) {
                mine += 1 + ((col + i - p - 1) >> 4);
                p = col + i;
            }
        }
        carry = pass_last > carry ? pass_last : carry;
    }
    int total = wave_sum_int(mine);
    if (F::kKeepTrailing) total += (cols - 1 - carry) >> 4;  // padding entries at carry+16, carry+32, ... < cols
    if (lane == 0) counts[row] = total;
}

// row_ptr[0] = 0, row_ptr[r+1] = counts[0] + ... + counts[r].  `counts` aliases row_ptr + 1.
// One workgroup; each thread owns a contiguous slice.
__global__ void __launch_bounds__(1024) scan_rows_kernel(int *__restrict__ row_ptr, int rows)
{
    __shared__ int wave_totals[16];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int per = (rows + 1023) / 1024;
    const int begin = tid * per < rows ? tid * per : rows;
    const int end = begin + per < rows ? begin + per : rows;
    int *counts = row_ptr + 1;
    int sum = 0;
    for (int i = begin; i < end; ++i) sum += counts[i];
    const int incl = wave_scan_inclusive(sum);
    if (lane == kWave - 1) wave_totals[wave] = incl;
    __syncthreads();
    int base = incl - sum;
    for (int w = 0; w < wave; ++w) base += wave_totals[w];
    for (int i = begin; i < end; ++i) {
        base += counts[i];
        counts[i] = base;
    }
    if (tid == 0) row_ptr[0] = 0;
}

// Packs the low nibbles of 8 staged entries (bits 16..19 of each word) into one delta word.
__device__ __forceinline__ u32 pack_nibbles(const u32 (&e)[8])
{
    u32 w = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) w |= ((e[i] >> 16) & 15u) << (4 * i);
    return w;
}

// Orders this wave's LDS writes before its later LDS reads (the staging area is private to
// the wave, so no workgroup barrier is involved).
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// Pass 2.  The wave stages the entries of its row in LDS at the offset they have inside their
// 8-entry group of the output, so that every complete group leaves as one 16-byte store of
// values and one 4-byte store of nibbles.  Groups cut by a row boundary are shared with the
// neighbouring row's wave: their values go out as 2-byte stores and their nibbles are OR-ed
// into the (zeroed) delta word.  `deltas` must be zero on entry; `values` need not be.
template <typename F, bool STREAM>
__global__ void __launch_bounds__(kBlock) fill_rows_kernel(const typename F::Elem *__restrict__ dense, int rows,
                                                           int cols, const int *__restrict__ row_ptr,
                                                           typename F::Elem *__restrict__ values,
                                                           u32 *__restrict__ delta_words, int padded)
{
    typedef typename F::Elem Elem;
    typedef typename F::Chunk Chunk;
    constexpr int kStage = kTile + 8;  // a tile's entries plus the carried part of a group
    __shared__ u32 stage_all[kRowsPerBlock][kStage];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = uniform(threadIdx.x >> 6);
    const int row = blockIdx.x * kRowsPerBlock + wave;
    if (row >= rows) return;
    const int e0 = row_ptr[row];
    const int e1 = row_ptr[row + 1];
    u32 *stage = stage_all[wave];
    Chunk *value_groups = reinterpret_cast<Chunk *>(values);

    if (row == rows - 1) {  // the unused tail of the last 8-entry group
        for (int i = e1 + lane; i < padded; i += kWave) values[i] = 0;
    }
    if (e0 == e1) return;

    const Elem *src = dense + (size_t)row * (size_t)cols;
    const bool vector_ok = (reinterpret_cast<uintptr_t>(src) & (sizeof(Chunk) - 1)) == 0;

    // stage[i] holds output entry base + i; [lo, hi) is staged and not yet written out
    int base = e0 & ~7;
    int lo = e0 - base;
    int hi = lo;
    int carry = -1;

    // writes out groups [0, n_groups) of the stage; group g holds entries [a, b) with
    // a = lo for group 0 and b = hi - 8g for a last, incomplete group
    auto flush = [&](int n_groups) {
        for (int g = lane; g < n_groups; g += kWave) {
            u32 e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = stage[8 * g + i];
            const int a = g == 0 ? lo : 0;
            const int b = hi - 8 * g < 8 ? hi - 8 * g : 8;
            const int out = (base >> 3) + g;
            if (a == 0 && b == 8) {
                Chunk v = {};
#pragma unroll
                for (int i = 0; i < 8; ++i) F::put(v, i, e[i] & 0xffffu);
                value_groups[out] = v;
                delta_words[out] = pack_nibbles(e);
            } else {
                u32 keep = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (i >= a && i < b) {
                        values[8 * (size_t)out + i] = (Elem)e[i];
                        keep |= 15u << (4 * i);
                    }
                }
                atomicOr(&delta_words[out], pack_nibbles(e) & keep);
            }
        }
    };

    Chunk next = load8<F, STREAM>(src, lane * kChunk, cols, vector_ok && lane * kChunk < cols);
    for (int c0 = 0; c0 < cols; c0 += kTile) {
        const int col = c0 + lane * kChunk;
        const Chunk v = next;
        if (c0 + kTile < cols) {
            const int ncol = col + kTile;
            next = load8<F, STREAM>(src, ncol, cols, vector_ok && ncol < cols);
        }
        const u32 nz = nonzero_bits<F>(v);
        const int own_last = nz ? col + 31 - __builtin_clz(nz) : kNoColumn;
        int pass_last;
        int p = previous_nonzero(own_last, carry, lane, pass_last);
        carry = pass_last > carry ? pass_last : carry;
        // which of my 8 columns store an entry, and with which nibble
        u32 entry_bits = 0;
        u32 nibbles = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int x = col + i;
            const int dist = x - p;
            const bool is_nz = (nz >> i) & 1u;
            const bool is_entry = x < cols && (is_nz || (dist & 15) == 0);
            const u32 nib = is_nz ? (u32)(dist - 1) & 15u : 15u;
            entry_bits |= (is_entry ? 1u : 0u) << i;
            nibbles |= nib << (4 * i);
            p = is_nz ? x : p;
        }
        const int mine = __builtin_popcount(entry_bits);
        const int incl = wave_scan_inclusive(mine);
        const int produced = __builtin_amdgcn_readlane(incl, kWave - 1);
        // entries past e1 are padding entries behind the row's last non-zero: not stored
        const int room = e1 - (base + hi);
        const int n_new = produced < room ? produced : room;
        int slot = incl - mine;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if ((entry_bits & (1u << i)) && slot < n_new) {
                stage[hi + slot] = F::stored(F::at(v, i)) | (((nibbles >> (4 * i)) & 15u) << 16);
                ++slot;
            }
        }
        hi += n_new;
        wave_lds_fence();
        const bool row_done = base + hi == e1;
        const int n_groups = row_done ? (hi + 7) >> 3 : hi >> 3;
        flush(n_groups);
        if (row_done) break;
        if (n_groups > 0) {  // carry the incomplete group to the front of the stage
            const int rest = hi & 7;
            const u32 moved = lane < rest ? stage[8 * n_groups + lane] : 0u;
            wave_lds_fence();
            if (lane < rest) stage[lane] = moved;
            base += 8 * n_groups;
            lo = 0;
            hi = rest;
        }
    }
}

// One wave per row, one entry per lane per pass.  `padded` bounds every read of values / deltas, so
// a row_ptr that points past the arrays cannot make the kernel read outside them.
__global__ void __launch_bounds__(kBlock) decode_rows_kernel(const uint16_t *__restrict__ values,
                                                             const unsigned char *__restrict__ deltas,
                                                             const int *__restrict__ row_ptr, int rows, int cols,
                                                             long long padded, uint16_t *__restrict__ dense)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + uniform(threadIdx.x >> 6);
    if (row >= rows) return;
    long long e0 = row_ptr[row];
    long long e1 = row_ptr[row + 1];
    e0 = e0 < 0 ? 0 : (e0 > padded ? padded : e0);
    e1 = e1 < e0 ? e0 : (e1 > padded ? padded : e1);
    uint16_t *dst = dense + (size_t)row * (size_t)cols;
    int column = -1;  // column of the last entry decoded so far
    for (long long j0 = e0; j0 < e1; j0 += kWave) {
        const long long j = j0 + lane;
        int step = 0;
        uint16_t val = 0;
        if (j < e1) {
            step = ((deltas[j >> 1] >> (4 * (j & 1))) & 15) + 1;
            val = values[j];
        }
        const int incl = wave_scan_inclusive(step);
        const int c = column + incl;
        if (j < e1 && c < cols) dst[c] = val;
        column += __builtin_amdgcn_readlane(incl, kWave - 1);
    }
}

// dst[0 .. n_vec) = 0, 16 bytes per thread and step (a fill kernel rather than a memset node, so
// the call can sit in a captured graph).
__global__ void __launch_bounds__(256) zero_fill_kernel(u32x4 *__restrict__ dst, size_t n_vec, uint16_t *__restrict__ tail,
                                                        int n_tail)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (size_t i = first; i < n_vec; i += stride) dst[i] = u32x4{0u, 0u, 0u, 0u};
    if (first < (size_t)n_tail) tail[first] = 0;
}

}  // namespace
}  // namespace macko

namespace macko {
namespace {

// The fill pass reads the matrix again after the count pass: up to about half the last-level
// cache (256 MB) both leave it there (measured: 5 % faster at 90 MB), beyond that they read it
// with the non-temporal hint (2 % faster at 470 MB and more).
template <typename Elem>
bool streams_past_cache(int32_t rows, int32_t cols)
{
    return (size_t)rows * (size_t)cols * sizeof(Elem) > ((size_t)128 << 20);
}

template <typename F>
int compress_count(const void *dense, int32_t rows, int32_t cols, int32_t *row_ptr, void *stream)
{
    typedef typename F::Elem Elem;
    if (rows < 0 || cols < 0 || row_ptr == nullptr) return MACKO_E_INVALID_ARGUMENT;
    if ((long long)rows * (long long)cols >= (1ll << 31)) return MACKO_E_INVALID_ARGUMENT;
    if (rows > 0 && cols > 0 && dense == nullptr) return MACKO_E_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(dense) & (sizeof(Elem) - 1)) || (reinterpret_cast<uintptr_t>(row_ptr) & 3))
        return MACKO_E_INVALID_ARGUMENT;
    hipStream_t s = as_stream(stream);
    if (rows > 0) {
        const bool stream_reads = streams_past_cache<Elem>(rows, cols);
        const dim3 grid((rows + kRowsPerBlock - 1) / kRowsPerBlock);
        if (stream_reads)
            hipLaunchKernelGGL((count_rows_kernel<F, true>), grid, dim3(kBlock), 0, s, (const Elem *)dense, rows, cols,
                               row_ptr + 1);
        else
            hipLaunchKernelGGL((count_rows_kernel<F, false>), grid, dim3(kBlock), 0, s, (const Elem *)dense, rows, cols,
                               row_ptr + 1);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(scan_rows_kernel, dim3(1), dim3(1024), 0, s, row_ptr, rows);
    return (int)hipGetLastError();
}

template <typename F>
int compress_fill(const void *dense, int32_t rows, int32_t cols, const int32_t *row_ptr, void *values,
                  void *deltas, int64_t padded_entries, void *stream)
{
    typedef typename F::Elem Elem;
    if (rows < 0 || cols < 0 || padded_entries < 0 || padded_entries % kChunk != 0)
        return MACKO_E_INVALID_ARGUMENT;
    if ((long long)rows * (long long)cols >= (1ll << 31)) return MACKO_E_INVALID_ARGUMENT;
    if (padded_entries == 0) return 0;
    if (dense == nullptr || row_ptr == nullptr || values == nullptr || deltas == nullptr)
        return MACKO_E_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(dense) & (sizeof(Elem) - 1)) ||
        (reinterpret_cast<uintptr_t>(values) & (sizeof(typename F::Chunk) - 1)) ||
        (reinterpret_cast<uintptr_t>(deltas) & 3))
        return MACKO_E_INVALID_ARGUMENT;
    hipStream_t s = as_stream(stream);
    // row-boundary nibbles are OR-ed in, so the nibble array starts from zero
    hipError_t e = hipMemsetAsync(deltas, 0, (size_t)padded_entries / 2, s);
    if (e != hipSuccess) return (int)e;
    if (rows == 0) return (int)hipMemsetAsync(values, 0, (size_t)padded_entries * sizeof(Elem), s);
    const dim3 grid((rows + kRowsPerBlock - 1) / kRowsPerBlock);
    if (streams_past_cache<Elem>(rows, cols))
        hipLaunchKernelGGL((fill_rows_kernel<F, true>), grid, dim3(kBlock), 0, s, (const Elem *)dense, rows, cols,
                           row_ptr, (Elem *)values, (u32 *)deltas, (int)padded_entries);
    else
        hipLaunchKernelGGL((fill_rows_kernel<F, false>), grid, dim3(kBlock), 0, s, (const Elem *)dense, rows, cols,
                           row_ptr, (Elem *)values, (u32 *)deltas, (int)padded_entries);
    return (int)hipGetLastError();
}

}  // namespace
}  // namespace macko

extern "C" int macko_compress_f16_count(const void *dense, int32_t rows, int32_t cols, int32_t *row_ptr,
                                        void *stream)
{
    return macko::compress_count<macko::Fp16Format>(dense, rows, cols, row_ptr, stream);
}

extern "C" int macko_compress_f16_fill(const void *dense, int32_t rows, int32_t cols, const int32_t *row_ptr,
                                       void *values, void *deltas, int64_t padded_entries, void *stream)
{
    return macko::compress_fill<macko::Fp16Format>(dense, rows, cols, row_ptr, values, deltas, padded_entries,
                                                   stream);
}

extern "C" int macko_compress_i8_count(const void *dense, int32_t rows, int32_t cols, int32_t *row_ptr,
                                       void *stream)
{
    return macko::compress_count<macko::Int8Format>(dense, rows, cols, row_ptr, stream);
}

extern "C" int macko_compress_i8_fill(const void *dense, int32_t rows, int32_t cols, const int32_t *row_ptr,
                                      void *values, void *deltas, int64_t padded_entries, void *stream)
{
    return macko::compress_fill<macko::Int8Format>(dense, rows, cols, row_ptr, values, deltas, padded_entries,
                                                   stream);
}

extern "C" int macko_decompress_f16(const void *values, const void *deltas, const int32_t *row_ptr, int32_t rows,
                                    int32_t cols, int64_t padded_entries, void *dense, void *stream)
{
    using namespace macko;
    if (rows < 0 || cols < 0 || padded_entries < 0) return MACKO_E_INVALID_ARGUMENT;
    if ((long long)rows * (long long)cols >= (1ll << 31)) return MACKO_E_INVALID_ARGUMENT;
    if (rows == 0 || cols == 0) return 0;
    if (dense == nullptr || row_ptr == nullptr) return MACKO_E_INVALID_ARGUMENT;
    if (padded_entries > 0 && (values == nullptr || deltas == nullptr)) return MACKO_E_INVALID_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(dense) & 1) return MACKO_E_INVALID_ARGUMENT;
    hipStream_t s = as_stream(stream);
    {   // zeros first: whole 16-byte pieces from the first aligned address on, the few elements around them singly
        const size_t n = (size_t)rows * (size_t)cols;
        uint16_t *d = (uint16_t *)dense;
        size_t head = ((16 - (reinterpret_cast<uintptr_t>(d) & 15)) & 15) / 2;
        if (head > n) head = n;
        const size_t n_vec = (n - head) / 8;
        const size_t rest = n - head - 8 * n_vec;
        if (head > 0)
            hipLaunchKernelGGL(zero_fill_kernel, dim3(1), dim3(256), 0, s, (u32x4 *)nullptr, (size_t)0, d, (int)head);
        size_t blocks = (n_vec + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        if (blocks < 1) blocks = 1;
        hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (u32x4 *)(d + head), n_vec,
                           d + head + 8 * n_vec, (int)rest);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(decode_rows_kernel, dim3((rows + kRowsPerBlock - 1) / kRowsPerBlock), dim3(kBlock), 0, s,
                       (const uint16_t *)values, (const unsigned char *)deltas, row_ptr, rows, cols,
                       (long long)padded_entries, (uint16_t *)dense);
    return (int)hipGetLastError();
}
