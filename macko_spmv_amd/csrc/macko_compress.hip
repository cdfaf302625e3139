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
constexpr int kAhead = 4;                     // tiles of its row a wave keeps in flight

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
    // the 8 values of a full group from their stage words (value in the low half of each)
    static __device__ __forceinline__ Chunk pack(const u32 (&e)[8])
    {
        Chunk v;
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = __builtin_amdgcn_perm(e[2 * k + 1], e[2 * k], 0x05040100u);
        return v;
    }
    // a half is a NaN when its low 15 bits exceed 0x7c00: adding 0x03ff then carries into bit 15
    static __device__ __forceinline__ bool any_nan(const Chunk &v)
    {
        u32 hit = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) hit |= ((v[w] & 0x7fff7fffu) + 0x03ff03ffu) & 0x80008000u;
        return hit != 0;
    }
};
struct Int8Format {
    typedef unsigned char Elem;
    typedef u32x2 Chunk;                         // 8 bytes
    static constexpr bool kKeepTrailing = true;  // cpu_compressor.cuh:75-117 has no withdrawal step
    static __device__ __forceinline__ u32 at(const Chunk &v, int i) { return (v[i >> 2] >> (8 * (i & 3))) & 0xffu; }
    static __device__ __forceinline__ void put(Chunk &v, int i, u32 bits) { v[i >> 2] |= bits << (8 * (i & 3)); }
    static __device__ __forceinline__ bool nonzero(u32 bits) { return bits != 0; }
    static __device__ __forceinline__ u32 stored(u32 bits) { return bits; }
    static __device__ __forceinline__ bool any_nan(const Chunk &) { return false; }
    static __device__ __forceinline__ Chunk pack(const u32 (&e)[8])
    {
        Chunk v;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const u32 lo = __builtin_amdgcn_perm(e[4 * k + 1], e[4 * k], 0x0c0c0400u);
            const u32 hi = __builtin_amdgcn_perm(e[4 * k + 3], e[4 * k + 2], 0x0c0c0400u);
            v[k] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        }
        return v;
    }
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
    // kAhead tiles of the row are in flight at any time: a wave walks its row alone, so what hides
    // the memory latency is the depth of its own queue
    Chunk ahead[kAhead];
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
        const int col = k * kTile + lane * kChunk;
        ahead[k] = load8<F, STREAM>(src, col, cols, vector_ok && col < cols);
    }
    for (int c0 = 0; c0 < cols; c0 += kAhead * kTile) {
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            const int col = c0 + k * kTile + lane * kChunk;
            if (c0 + k * kTile >= cols) break;  // wave-uniform
            const Chunk v = ahead[k];
            const int ncol = col + kAhead * kTile;
            if (c0 + (k + kAhead) * kTile < cols) ahead[k] = load8<F, STREAM>(src, ncol, cols, vector_ok && ncol < cols);
            const u32 nz = nonzero_bits<F>(v);
            const int own_last = nz ? col + 31 - __builtin_clz(nz) : kNoColumn;
            int pass_last;
            const int p = previous_nonzero(own_last, carry, lane, pass_last);
            // every non-zero is an entry; padding entries can only stand in front of the first
            // non-zero of my 8 columns (the others follow their predecessor within 8 columns)
            if (nz) mine += __builtin_popcount(nz) + ((col + __builtin_ctz(nz) - p - 1) >> 4);
            carry = pass_last > carry ? pass_last : carry;
        }
    }
    int total = wave_sum_int(mine);
    if (F::kKeepTrailing) total += (cols - 1 - carry) >> 4;  // padding entries at carry+16, carry+32, ... < cols
    if (lane == 0) counts[row] = total;
}

// row_ptr[0] = 0, row_ptr[r+1] = counts[0] + ... + counts[r].  `counts` aliases row_ptr + 1.
// One workgroup walks the rows in slices of kScanSlice: the slice comes into LDS through
// coalesced loads that are all in flight together, each thread sums and scans the kScanPer
// consecutive rows it owns there, and the slice goes back out coalesced.
constexpr int kScanPer = 8;
constexpr int kScanSlice = 1024 * kScanPer;
__global__ void __launch_bounds__(1024) scan_rows_kernel(int *__restrict__ row_ptr, int rows, int *total_out)
{
    __shared__ int slice[kScanSlice + kScanSlice / 32];  // one word of padding per 32: consecutive owners, different banks
    __shared__ int wave_totals[16];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    int *counts = row_ptr + 1;
    int running = 0;  // sum of all earlier slices
    auto at = [](int i) { return i + (i >> 5); };
    for (int s0 = 0; s0 < rows; s0 += kScanSlice) {
        int v[kScanPer];
#pragma unroll
        for (int j = 0; j < kScanPer; ++j) {
            const int i = s0 + j * 1024 + tid;
            v[j] = i < rows ? counts[i] : 0;
        }
#pragma unroll
        for (int j = 0; j < kScanPer; ++j) slice[at(j * 1024 + tid)] = v[j];
        __syncthreads();
        int sum = 0;
#pragma unroll
        for (int j = 0; j < kScanPer; ++j) {
            sum += slice[at(tid * kScanPer + j)];
            v[j] = sum;
        }
        const int incl = wave_scan_inclusive(sum);
        if (lane == kWave - 1) wave_totals[wave] = incl;
        __syncthreads();
        int base = running + incl - sum;
        int slice_total = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) {
            const int t = wave_totals[w];
            base += w < wave ? t : 0;
            slice_total += t;
        }
#pragma unroll
        for (int j = 0; j < kScanPer; ++j) slice[at(tid * kScanPer + j)] = base + v[j];
        running += slice_total;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kScanPer; ++j) {
            const int i = s0 + j * 1024 + tid;
            if (i < rows) counts[i] = slice[at(j * 1024 + tid)];
        }
        __syncthreads();  // the slice and the wave totals are reused
    }
    if (tid == 0) {
        row_ptr[0] = 0;
        // for a host thread that waits for this word to change rather than for the stream
        if (total_out != nullptr) __hip_atomic_store(total_out, running, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// Packs the nibbles of 8 staged entries (bits 16..19 of each word, bits 20..23 zero) into one delta
// word: byte 2 of four words at a time into one register, neighbouring bytes folded into one byte.
__device__ __forceinline__ u32 pack_nibbles(const u32 (&e)[8])
{
    u32 folded[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const u32 a = __builtin_amdgcn_perm(e[4 * h + 1], e[4 * h], 0x0c0c0602u);      // n0 | n1 << 8
        const u32 b = __builtin_amdgcn_perm(e[4 * h + 3], e[4 * h + 2], 0x0c0c0602u);  // n2 | n3 << 8
        const u32 four = __builtin_amdgcn_perm(b, a, 0x05040100u);                     // n0, n1, n2, n3 in bytes
        folded[h] = four | (four >> 4);  // byte 0 = n0 | n1 << 4, byte 2 = n2 | n3 << 4
    }
    return __builtin_amdgcn_perm(folded[1], folded[0], 0x06040200u);
}

// Orders this wave's LDS writes before its later LDS reads by other lanes.  The staging area is
// private to the wave and a wave's LDS operations are carried out in the order issued, so this is
// a matter of instruction order only: fences of wavefront scope, which wait for nothing (a wider
// scope would also wait for the row's loads in flight and the stores on their way out).
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Pass 2.  The wave stages the entries of its row in LDS at the offset they have inside their
// 8-entry group of the output, so that every complete group leaves as one 16-byte store of
// values and one 4-byte store of nibbles.  Groups cut by a row boundary are shared with the
// neighbouring row's wave: their values go out as 2-byte stores and their nibbles as bytes.  A
// byte holds two nibbles; where a row ends on an odd entry its last nibble shares a byte with the
// first nibble of the next non-empty row.  That byte is written by the earlier row's wave, which
// works the later row's first nibble out for itself from that row's first 16 columns (the column
// of its first non-zero, or 15 for a padding entry); the later row's wave leaves the byte alone.
// So every byte of `deltas` and every element of `values` has exactly one writer, and neither
// array needs to be cleared beforehand.
template <typename F, bool STREAM>
__global__ void __launch_bounds__(kBlock) fill_rows_kernel(const typename F::Elem *__restrict__ dense, int rows,
                                                           int cols, const int *__restrict__ row_ptr,
                                                           typename F::Elem *__restrict__ values,
                                                           u32 *__restrict__ delta_words, int padded)
{
    typedef typename F::Elem Elem;
    typedef typename F::Chunk Chunk;
    constexpr int kStage = kTile + 8;  // a tile's entries plus the carried part of a group
    __shared__ __attribute__((aligned(16))) u32 stage_all[kRowsPerBlock][kStage + kWave];  // + a spare word per lane
    // gap_table[m]: the 8 nibbles of a lane whose non-zero columns are the set bits of m, as far as
    // they can be told from m alone: 15 where there is no non-zero, the distance to the previous
    // set bit less one for a non-zero, and 0 for the first non-zero, whose distance reaches back
    // into earlier lanes and is put in by the lane itself
    __shared__ u32 gap_table[256];
    static_assert(kBlock == 256, "one table entry per thread");
    {
        const u32 m = threadIdx.x;
        u32 word = 0;
        int previous = -1;
        for (int i = 0; i < 8; ++i) {
            u32 nib = 15u;
            if ((m >> i) & 1u) {
                nib = previous < 0 ? 0u : (u32)(i - previous - 1);
                previous = i;
            }
            word |= nib << (4 * i);
        }
        gap_table[m] = word;
    }
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = uniform(threadIdx.x >> 6);
    const int row = blockIdx.x * kRowsPerBlock + wave;
    if (row >= rows) return;
    const int e0 = row_ptr[row];
    const int e1 = row_ptr[row + 1];
    u32 *stage = stage_all[wave];
    Chunk *value_groups = reinterpret_cast<Chunk *>(values);
    unsigned char *delta_bytes = reinterpret_cast<unsigned char *>(delta_words);

    if (row == rows - 1) {  // the unused tail of the last 8-entry group (an odd e1's byte has its owner)
        for (int i = e1 + lane; i < padded; i += kWave) values[i] = 0;
        for (int i = ((e1 + 1) >> 1) + lane; i < (padded >> 1); i += kWave) delta_bytes[i] = 0;
    }
    if (e0 == e1) return;

    // The first nibble behind my row, wanted if my last entry is the low half of a byte: asked for
    // now, on the guess that the next row is not empty, and looked at when my row is done.
    const bool shares_last_byte = (e1 & 1) != 0;
    const bool probe_lane = lane < 16 && lane < cols;
    int next_end = e1;
    u32 next_probe = 0;
    if (shares_last_byte && row + 1 < rows) {
        next_end = row_ptr[row + 2];
        if (probe_lane) next_probe = dense[(size_t)(row + 1) * (size_t)cols + lane];
    }
    auto first_nibble_behind = [&]() -> u32 {
        int r2 = row + 1;
        if (r2 >= rows) return 0u;  // my row holds the last entry: the rest of the byte is padding
        if (next_end == e1) {       // empty rows behind mine: walk on to the next one that is not
            do {
                ++r2;
            } while (r2 < rows && row_ptr[r2 + 1] == e1);
            if (r2 >= rows) return 0u;
            next_probe = probe_lane ? (u32)dense[(size_t)r2 * (size_t)cols + lane] : 0u;
        }
        // a row with entries whose first 16 columns are zero starts with the padding entry of column 15
        const unsigned long long m = __ballot(probe_lane && F::nonzero(next_probe));
        return m ? (u32)__builtin_ctzll(m) : 15u;
    };

    const Elem *src = dense + (size_t)row * (size_t)cols;
    const bool vector_ok = (reinterpret_cast<uintptr_t>(src) & (sizeof(Chunk) - 1)) == 0;

    // stage[i] holds output entry base + i; [lo, hi) is staged and not yet written out
    int base = e0 & ~7;
    int lo = e0 - base;
    int hi = lo;
    int carry = -1;

    // writes out groups [0, n_groups) of the stage; group g holds entries [a, b) with
    // a = lo for group 0 and b = hi - 8g for a last, incomplete group (which ends the row)
    auto flush = [&](int n_groups, u32 nibble_behind) {
        for (int g = lane; g < n_groups; g += kWave) {
            u32 e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = stage[8 * g + i];
            const int a = g == 0 ? lo : 0;
            const int b = hi - 8 * g < 8 ? hi - 8 * g : 8;
            const int out = (base >> 3) + g;
            if (a == 0 && b == 8) {
                value_groups[out] = F::pack(e);
                delta_words[out] = pack_nibbles(e);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (i >= a && i < b) values[8 * (size_t)out + i] = (Elem)e[i];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool low_mine = 2 * j >= a && 2 * j < b;
                    const bool high_mine = 2 * j + 1 >= a && 2 * j + 1 < b;
                    // low nibble mine: my byte, whoever the high nibble belongs to
                    if (low_mine) {
                        const u32 low = (e[2 * j] >> 16) & 15u;
                        const u32 high = high_mine ? (e[2 * j + 1] >> 16) & 15u : nibble_behind;
                        delta_bytes[4 * (size_t)out + j] = (unsigned char)(low | (high << 4));
                    }
                }
            }
        }
    };

    // kAhead tiles of the row in flight, as in pass 1
    Chunk ahead[kAhead];
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
        const int col = k * kTile + lane * kChunk;
        ahead[k] = load8<F, STREAM>(src, col, cols, vector_ok && col < cols);
    }
    bool row_done = false;
    for (int c0 = 0; c0 < cols && !row_done; c0 += kAhead * kTile) {
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            if (row_done || c0 + k * kTile >= cols) break;  // wave-uniform
            const int col = c0 + k * kTile + lane * kChunk;
            const Chunk v = ahead[k];
            const int ncol = col + kAhead * kTile;
            if (c0 + (k + kAhead) * kTile < cols) ahead[k] = load8<F, STREAM>(src, ncol, cols, vector_ok && ncol < cols);
            const u32 nz = nonzero_bits<F>(v);
            const int own_last = nz ? col + 31 - __builtin_clz(nz) : kNoColumn;
            int pass_last;
            int p = previous_nonzero(own_last, carry, lane, pass_last);
            carry = pass_last > carry ? pass_last : carry;
            // Non-zeros are entries.  A padding entry stands at p + 16, p + 32, ...: among my 8
            // columns at most one, and only in front of my first non-zero (behind it the previous
            // non-zero is less than 8 columns away).
            const int pad_at = p + (((col - p + 15) >> 4) << 4) - col;  // >= 0, my column index of it
            const int first_nz = nz ? __builtin_ctz(nz) : 8;
            const bool has_pad = pad_at < first_nz && col + pad_at < cols;
            const u32 entry_bits = nz | (has_pad ? 1u << pad_at : 0u);
            u32 nibbles = gap_table[nz];
            if (nz) nibbles |= ((u32)(col + first_nz - p - 1) & 15u) << (4 * first_nz);
            const int mine = __builtin_popcount(entry_bits);
            const int incl = wave_scan_inclusive(mine);
            const int produced = __builtin_amdgcn_readlane(incl, kWave - 1);
            // entries past e1 are padding entries behind the row's last non-zero: not stored
            const int room = e1 - (base + hi);
            const int n_new = produced < room ? produced : room;
            // Those dropped entries are whole lanes: behind the row's last non-zero a lane holds at
            // most its one padding entry, and the lane of the last non-zero has its padding entry
            // in front of it.  So a lane keeps all of its entries or none.
            const int slot = incl - mine;
            const u32 kept = slot < n_new ? entry_bits : 0u;
            Chunk vs = v;
            if (__builtin_expect(__ballot(F::any_nan(v)) != 0ull, 0)) {  // NaNs are stored in one form
                vs = Chunk{};
#pragma unroll
                for (int i = 0; i < 8; ++i) F::put(vs, i, F::stored(F::at(v, i)));
            }
            // every lane writes all 8 of its columns, no branches: what is not kept goes to a word
            // of the lane's own behind the stage
            const int first_index = hi + slot;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool take = ((kept >> i) & 1u) != 0;
                const int rank = __builtin_popcount(kept & ((1u << i) - 1u));
                const u32 word = F::at(vs, i) | (((nibbles >> (4 * i)) & 15u) << 16);
                stage[take ? first_index + rank : kStage + lane] = word;
            }
            hi += n_new;
            wave_lds_fence();
            row_done = base + hi == e1;
            const int n_groups = row_done ? (hi + 7) >> 3 : hi >> 3;
            flush(n_groups, row_done && shares_last_byte ? first_nibble_behind() : 0u);
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
int compress_count(const void *dense, int32_t rows, int32_t cols, int32_t *row_ptr, int32_t *total, void *stream)
{
    typedef typename F::Elem Elem;
    if (rows < 0 || cols < 0 || row_ptr == nullptr) return MACKO_E_INVALID_ARGUMENT;
    if ((long long)rows * (long long)cols >= (1ll << 31)) return MACKO_E_INVALID_ARGUMENT;
    if (rows > 0 && cols > 0 && dense == nullptr) return MACKO_E_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(dense) & (sizeof(Elem) - 1)) || (reinterpret_cast<uintptr_t>(row_ptr) & 3) ||
        (reinterpret_cast<uintptr_t>(total) & 3))
        return MACKO_E_INVALID_ARGUMENT;  // before anything is launched
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
    hipLaunchKernelGGL(scan_rows_kernel, dim3(1), dim3(1024), 0, s, row_ptr, rows, total);
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
    if (rows == 0) return MACKO_E_INVALID_ARGUMENT;  // entries without rows
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
    return macko::compress_count<macko::Fp16Format>(dense, rows, cols, row_ptr, nullptr, stream);
}

extern "C" int macko_compress_f16_fill(const void *dense, int32_t rows, int32_t cols, const int32_t *row_ptr,
                                       void *values, void *deltas, int64_t padded_entries, void *stream)
{
    return macko::compress_fill<macko::Fp16Format>(dense, rows, cols, row_ptr, values, deltas, padded_entries,
                                                   stream);
}

extern "C" int macko_compress_f16_count_total(const void *dense, int32_t rows, int32_t cols, int32_t *row_ptr,
                                              int32_t *total, void *stream)
{
    return macko::compress_count<macko::Fp16Format>(dense, rows, cols, row_ptr, total, stream);
}

extern "C" int macko_compress_i8_count_total(const void *dense, int32_t rows, int32_t cols, int32_t *row_ptr,
                                             int32_t *total, void *stream)
{
    return macko::compress_count<macko::Int8Format>(dense, rows, cols, row_ptr, total, stream);
}

extern "C" int macko_compress_i8_count(const void *dense, int32_t rows, int32_t cols, int32_t *row_ptr,
                                       void *stream)
{
    return macko::compress_count<macko::Int8Format>(dense, rows, cols, row_ptr, nullptr, stream);
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
