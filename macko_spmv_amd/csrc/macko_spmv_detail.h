// Pieces shared by the two SpMV kernels of libmacko_hip.so (internal; the public ABI is
// include/macko_hip.h): launch arguments, the row_ptr searches, masks, buffer descriptors.
#pragma once

#include "macko_common.h"

namespace macko {
namespace spmv_detail {


constexpr int kLdsFront = 16;   // zero bytes in front of x in LDS
constexpr int kLdsBack = 64;    // zero bytes behind x
constexpr int kTileShift = 9;   // log2(kTile)
constexpr int kXRegs = 2;       // 16-byte pieces of x a thread fetches with tracked loads
constexpr int kLookBack = 2048; // entries covered by one 16-byte-per-lane load of deltas

struct SpmvArgs {
    const u32 *values;      // fp16 pairs (or int8 quads for the int8 variant)
    const u32 *deltas;      // 8 nibbles per word
    const int *row_ptr;
    const uint16_t *x;
    uint16_t *y;
    int rows;
    int cols;
    long long padded;       // P
    float alpha;
    float beta;
    // Precomputed on the host so the kernel does no 64-bit division.  Rows are owned whole by N
    // owners (the launch's waves, or its workgroups in the split kernel).  The P stored entries
    // are dealt to them as evenly as possible: owner k starts at k*q + min(k, rem).  Where its
    // first row should be if all rows were equally long, floor(k*rows/N), is
    // k*rows_q + ((k*rows_frac) >> 32) with rows_frac = floor((rows % N) * 2^32 / N).
    u32 entries_q, entries_rem;
    u32 rows_q, rows_frac;
    // 1 when there are no more rows than owners: owner k then simply owns rows
    // [floor(k*rows/N), floor((k+1)*rows/N)), at most one row each.  No split of whole rows can do
    // better than the longest row, and cutting by entries could hand one owner two rows.
    u32 row_even;
    // batched product (NB > 1 vectors per launch): elements between consecutive vectors of x / y
    int ldx, ldy;
    // fused x staging (XF != 0): the second operand of the function that produces x, and its epsilon
    const uint16_t *x2;
    float eps;
    // Split kernel only.  log2 of the number of waves per workgroup that stream tiles (the others
    // only help to stage x).
    u32 active_shift;
    // Split kernel only.  How many entries in front of a wave's first entry are requested ahead of time (they tell a
    // wave that starts inside a row at which column it continues): 512, or 2048 * k, k = 1..4.
    // Chosen from the mean row length; rows that began further back cost an extra round trip.
    u32 look_entries;
    // Whole-row kernel only.  What a row weighs, in stored entries, when the rows are dealt to the
    // waves: the cuts balance entries + row_cost * rows (a row's end costs a reduction, a store and
    // masked passes, whatever its length).  entries_q / entries_rem then split that sum.
    u32 row_cost;
    // Whole-row kernel, variant for short rows only.  What is left of a tile when at least
    // rows_pass_min more rows end in it is worked in one pass over all those rows; that pass keeps
    // 2 KB per wave in LDS, rows_pass_lds bytes into the dynamic LDS.
    u32 rows_pass_min;
    u32 rows_pass_lds;
    // Whole-row kernel with prepared cuts only: {first row, its first entry} per wave of the launch
    // and one more pair for the end (rows, stored entries), as macko_spmv_plan_build writes them.
    const int *plan;
    int plan_entries;  // host side only: int32 elements behind `plan`, 2 * (waves of the launch + 1)
#ifdef MACKO_DEV_HOOKS
    long long *trace;  // 8 timestamps per wave (development builds only)
#endif
};

#ifdef MACKO_DEV_HOOKS
#define MACKO_STAMP(slot) \
    do { if (a.trace && lane == 0) a.trace[(size_t)stamp_wave * 8 + (slot)] = (long long)__builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define MACKO_STAMP(slot) do { } while (0)
#endif

// First item of part k when n items are dealt to the parts as evenly as possible.
__device__ __forceinline__ u32 even_split(u32 k, u32 q, u32 rem) { return k * q + (k < rem ? k : rem); }

__device__ __forceinline__ float half_bits_to_float(uint16_t h)
{
    return (float)__builtin_bit_cast(_Float16, h);
}

__device__ __forceinline__ uint16_t float_to_half_bits(float f)
{
    return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// Where the first probe of the row search looks: 64 consecutive row_ptr values starting a few
// rows before `guess`.
__device__ __forceinline__ int probe_base(int guess, int rows)
{
    int w0 = guess - 8;
    const int wmax = rows - 63;
    w0 = w0 > wmax ? wmax : w0;
    return w0 < 0 ? 0 : w0;
}

// Lane i of the returned value holds row_ptr[base + i] (row_ptr[rows] beyond the end).
__device__ __forceinline__ int load_row_window(const int *__restrict__ row_ptr, int rows, int base, int lane)
{
    const int idx = base + lane;
    return row_ptr[idx <= rows ? idx : rows];
}

// Smallest r in [0, rows] with row_ptr[r] >= target (rows if there is none), for two targets at
// once.  All 64 lanes probe together.  window[k] is an already loaded probe (see
// load_row_window) at base[k]; it resolves the search when rows carry similar entry counts.
// Otherwise one more window is probed where the target should be if rows elsewhere are as long as
// the ones just seen (which usually lands within a few rows even for very uneven matrices; that
// window then replaces window[k] / base[k] so the caller finds its row starts in it), and 64-ary
// rounds over what is still undecided follow.  Every value here is wave-uniform.
// With row_cost != 0 the search runs on row_ptr[r] + row_cost * r instead of row_ptr[r] (a row then
// weighs row_cost entries on top of its own); the windows keep plain row_ptr values.
__device__ __forceinline__ void wave_lower_bound2(const int *__restrict__ row_ptr, int rows, int lane,
                                                  const int target[2], int (&window)[2], int (&base)[2],
                                                  int out[2], int row_cost = 0)
{
    int lo[2], hi[2];
    // narrows [lo, hi] with a window of row_ptr values: probed[i] >= target puts the answer at or
    // before base + i, probed[i] < target puts it after
    auto narrow = [&](int k, int probed, int at) {
        const bool beyond = at + lane > rows;
        const unsigned long long m = __ballot(beyond || probed + row_cost * (at + lane) >= target[k]);
        if (m == 0) {
            const int after = at + 64 > rows ? rows : at + 64;
            lo[k] = lo[k] > after ? lo[k] : after;
        } else {
            const int f = __builtin_ctzll(m);
            const int le = at + f > rows ? rows : at + f;
            hi[k] = hi[k] < le ? hi[k] : le;
            if (f > 0) lo[k] = lo[k] > le ? lo[k] : le;
        }
        if (lo[k] > hi[k]) lo[k] = hi[k];
    };
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        lo[k] = 0;
        hi[k] = rows;
        narrow(k, window[k], base[k]);
    }
    if (__builtin_expect(lo[0] < hi[0] || lo[1] < hi[1], 0)) {
        // second window, from the local row length: rows per entry around the first window
        int probe[2], at[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            at[k] = base[k];
            if (lo[k] < hi[k]) {
                const int last = base[k] + 63 <= rows ? 63 : rows - base[k];
                const int v0 = __builtin_amdgcn_readlane(window[k], 0) + row_cost * base[k];
                const int v1 = __builtin_amdgcn_readlane(window[k], last) + row_cost * (base[k] + last);
                const float per_entry = (float)(last > 0 ? last : 1) / (float)(v1 > v0 ? v1 - v0 : 1);
                float jump = (float)(target[k] - v0) * per_entry;
                jump = jump > 2.0e9f ? 2.0e9f : (jump < -2.0e9f ? -2.0e9f : jump);
                long long g = (long long)base[k] + (long long)jump - 32;
                const int gmax = rows - 63 > 0 ? rows - 63 : 0;
                g = g < lo[k] - 1 ? lo[k] - 1 : g;  // stay inside what is still undecided
                g = g > hi[k] - 32 ? hi[k] - 32 : g;
                g = g < 0 ? 0 : (g > gmax ? gmax : g);
                at[k] = (int)g;
            }
            probe[k] = load_row_window(row_ptr, rows, at[k], lane);  // both loads in flight together
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            if (lo[k] < hi[k]) {
                narrow(k, probe[k], at[k]);
                window[k] = probe[k];
                base[k] = at[k];
            }
        }
    }
    while (__builtin_expect(lo[0] < hi[0] || lo[1] < hi[1], 0)) {
        int step[2], probe[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            step[k] = (hi[k] - lo[k] + 63) >> 6;
            const int idx = lo[k] + lane * step[k];
            probe[k] = (lo[k] < hi[k] && idx < hi[k]) ? row_ptr[idx] + row_cost * idx : 0x7fffffff;
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            if (lo[k] < hi[k]) {
                const unsigned long long m = __ballot(probe[k] >= target[k]);
                if (m == 0) {
                    lo[k] = lo[k] + 63 * step[k] + 1;
                } else {
                    const int f = __builtin_ctzll(m);
                    const int at = lo[k] + f * step[k];
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

// Smallest r in [lo, hi] with row_ptr[r] >= target, given that row_ptr[hi] >= target: 64-ary
// rounds, all lanes probing together.  Wave-uniform.
__device__ __forceinline__ int wave_lower_bound_in(const int *__restrict__ row_ptr, int lane, int lo, int hi,
                                                   int target)
{
    while (lo < hi) {
        const int step = (hi - lo + 63) >> 6;
        const int idx = lo + lane * step;
        const int probe = idx < hi ? row_ptr[idx] : 0x7fffffff;
        const unsigned long long m = __ballot(probe >= target);
        if (m == 0) {
            lo = lo + 63 * step + 1;
        } else {
            const int f = __builtin_ctzll(m);
            const int at = lo + f * step;
            if (f > 0) lo = lo + (f - 1) * step + 1;
            if (at < hi) hi = at;
        }
        if (lo > hi) lo = hi;
    }
    return lo;
}

// Mask helpers: keep values [from, 8) / [0, upto) of a lane's 8 values (VB bytes each) and the
// matching nibbles.  `from` / `upto` are wave-uniform, so the masks are built on the scalar unit.
template <int VB>
__device__ __forceinline__ void mask_from(u32x4 &v, u32 &d, int from)  // 1 <= from <= 7
{
    if (VB == 1) {  // 8 one-byte values in v.x, v.y
        const unsigned long long m = ~0ull << (8 * from);
        v.x &= (u32)m;
        v.y &= (u32)(m >> 32);
        d &= ~0u << (4 * from);
        return;
    }
    const unsigned long long lo = from < 4 ? (~0ull << (16 * from)) : 0ull;
    const unsigned long long hi = from < 4 ? ~0ull : (~0ull << (16 * (from - 4)));
    v.x &= (u32)lo;
    v.y &= (u32)(lo >> 32);
    v.z &= (u32)hi;
    v.w &= (u32)(hi >> 32);
    d &= ~0u << (4 * from);
}

template <int VB>
__device__ __forceinline__ void mask_upto(u32x4 &v, u32 &d, int upto)  // 1 <= upto <= 7
{
    if (VB == 1) {
        const unsigned long long m = (1ull << (8 * upto)) - 1;
        v.x &= (u32)m;
        v.y &= (u32)(m >> 32);
        d &= (1u << (4 * upto)) - 1;
        return;
    }
    const unsigned long long lo = upto < 4 ? ((1ull << (16 * upto)) - 1) : ~0ull;
    const unsigned long long hi = upto <= 4 ? 0ull : ((1ull << (16 * (upto - 4))) - 1);
    v.x &= (u32)lo;
    v.y &= (u32)(lo >> 32);
    v.z &= (u32)hi;
    v.w &= (u32)(hi >> 32);
    d &= (1u << (4 * upto)) - 1;
}

constexpr u32 kNoTileValues = 0xfffff000u;  // beyond any values array (2P < 2^32 - 8192)
constexpr u32 kNoTileDeltas = 0x7ffff000u;  // beyond any deltas array (P/2 < 2^30)

// Buffer descriptor (V#) over `bytes` bytes at `base`: raw buffer, bounds-checked on the offset.
__device__ __forceinline__ u32x4 make_buffer(const void *base, u32 bytes)
{
    const unsigned long long addr = reinterpret_cast<unsigned long long>(base);
    u32x4 r;
    r.x = uniform((int)(u32)addr);
    r.y = uniform((int)((u32)(addr >> 32) & 0xffffu));
    r.z = uniform((int)bytes);
    r.w = 0x00020000u;
    return r;
}

// The multiplier 2 in nibble positions 0..k: v_dot8_u32_u4 with it gives twice the sum of a word's
// first k+1 nibbles.
__device__ __forceinline__ constexpr u32 twos_upto(int k)
{
    return (k >= 7 ? 0xffffffffu : ((1u << (4 * (k + 1))) - 1u)) & 0x22222222u;
}

// Lane L's copy of element idx of an array of eight per-lane values; idx and L are wave-uniform.
__device__ __forceinline__ float pick_lane(const float (&c)[8], int idx, int L)
{
    int bits;
    switch (idx) {
    case 0: bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[0]), L); break;
    case 1: bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[1]), L); break;
    case 2: bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[2]), L); break;
    case 3: bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[3]), L); break;
    case 4: bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[4]), L); break;
    case 5: bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[5]), L); break;
    case 6: bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[6]), L); break;
    default: bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[7]), L); break;
    }
    return __builtin_bit_cast(float, bits);
}

}  // namespace spmv_detail

// The kernel for matrices with few, long rows (macko_spmv_split.hip): workgroups own whole rows and
// their waves share the workgroup's tiles evenly.  Variant selectors: axpby (y = alpha*Mx + beta*y),
// value_bytes 2 (fp16) or 1 (int8), n_vectors 1/2/4/8, fused 0/1/2 (see SpmvArgs::x2), x_in_lds.
// lds_x = bytes of LDS that x takes (0 when x is gathered from memory).  Returns an ABI error code.
int spmv_split_launch(const spmv_detail::SpmvArgs &a, bool axpby, int value_bytes, int n_vectors, int fused,
                      bool x_in_lds, int grid, size_t lds_x, hipStream_t stream);

}  // namespace macko
