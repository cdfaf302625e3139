// Shared host/device helpers of libmacko_hip.so (internal; the public ABI is include/macko_hip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "macko_hip.h"

namespace macko {

typedef uint32_t u32;
typedef __attribute__((ext_vector_type(4))) u32 u32x4;
typedef __attribute__((ext_vector_type(2))) u32 u32x2;

constexpr int kWave = 64;          // gfx950 wavefront
constexpr int kChunk = 8;          // entries per 128-bit value load / 32-bit delta load
constexpr int kTile = kWave * kChunk;  // entries one wave handles per pass

// Static facts about the current device, fetched once per device and cached.
struct DeviceInfo {
    int compute_units;
    int max_lds_bytes;   // per workgroup
};
int device_info(DeviceInfo *out);  // 0 or an error code of the public ABI

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// ---- wave64 cross-lane primitives (DPP; row = 16 lanes) ---------------------------------

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ int wave_scan_inclusive(int x)
{
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, true);   // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, true);   // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, true);   // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, true);   // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);  // row_bcast:15 -> rows 1,3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);  // row_bcast:31 -> rows 2,3
    return x;
}

template <int CTRL, int ROW_MASK, bool BOUND_ZERO>
__device__ __forceinline__ float dpp_f32(float x)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROW_MASK, 0xF, BOUND_ZERO));
}

// Sum over the 64 lanes; the result is wave-uniform.
__device__ __forceinline__ float wave_sum(float x)
{
    x += dpp_f32<0x111, 0xF, true>(x);
    x += dpp_f32<0x112, 0xF, true>(x);
    x += dpp_f32<0x114, 0xF, true>(x);
    x += dpp_f32<0x118, 0xF, true>(x);
    x += dpp_f32<0x142, 0xA, false>(x);
    x += dpp_f32<0x143, 0xC, false>(x);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

// Segmented inclusive prefix sums over the 64 lanes of a wave.  A lane whose flag is set starts a
// new segment: it keeps its own value, the lanes behind it sum from there.  The flags travel as
// wave masks, which the scalar unit shifts alongside the vector adds; one set of masks serves any
// number of scans over the same segments.
struct SegmentMasks {
    unsigned long long step[6];  // lanes that take nothing in step s (a segment starts within reach)
};

__device__ __forceinline__ SegmentMasks segment_masks(unsigned long long starts)
{
    SegmentMasks m;
    unsigned long long f = starts;
    m.step[0] = f;
    f |= (f << 1) & ~0x0001000100010001ull;  // row_shr stops at the 16-lane rows
    m.step[1] = f;
    f |= (f << 2) & ~0x0003000300030003ull;
    m.step[2] = f;
    f |= (f << 4) & ~0x000f000f000f000full;
    m.step[3] = f;
    f |= (f << 8) & ~0x00ff00ff00ff00ffull;
    m.step[4] = f;
    // row_bcast:15 hands lane 15 to row 1 and lane 47 to row 3
    f |= ((f >> 15) & 1 ? 0x00000000ffff0000ull : 0ull) | ((f >> 47) & 1 ? 0xffff000000000000ull : 0ull);
    m.step[5] = f;
    return m;
}

template <typename T> __device__ __forceinline__ T wave_segmented_scan(T x, const SegmentMasks &m)
{
    auto step = [&](auto tag, unsigned long long keep) {
        constexpr int S = decltype(tag)::value;
        constexpr int ctrl = S == 0 ? 0x111 : S == 1 ? 0x112 : S == 2 ? 0x114 : S == 3 ? 0x118 : S == 4 ? 0x142 : 0x143;
        constexpr int rows = S == 4 ? 0xA : S == 5 ? 0xC : 0xF;
        const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, rows, 0xF, S < 4);
        const T sum = x + __builtin_bit_cast(T, moved);
        x = __builtin_amdgcn_inverse_ballot_w64(keep) ? x : sum;
    };
    step(std::integral_constant<int, 0>{}, m.step[0]);
    step(std::integral_constant<int, 1>{}, m.step[1]);
    step(std::integral_constant<int, 2>{}, m.step[2]);
    step(std::integral_constant<int, 3>{}, m.step[3]);
    step(std::integral_constant<int, 4>{}, m.step[4]);
    step(std::integral_constant<int, 5>{}, m.step[5]);
    return x;
}

// The value of the lane below (0 in lane 0) / of the lane above (0 in lane 63).
__device__ __forceinline__ int wave_from_lane_below(int x) { return __builtin_amdgcn_update_dpp(0, x, 0x138, 0xF, 0xF, true); }
__device__ __forceinline__ int wave_from_lane_above(int x) { return __builtin_amdgcn_update_dpp(0, x, 0x130, 0xF, 0xF, true); }

// Inclusive running maximum over the 64 lanes.
__device__ __forceinline__ int wave_scan_max_inclusive(int x)
{
    const int lowest = (int)0x80000000;
    int t;
    t = __builtin_amdgcn_update_dpp(lowest, x, 0x111, 0xF, 0xF, false); x = t > x ? t : x;
    t = __builtin_amdgcn_update_dpp(lowest, x, 0x112, 0xF, 0xF, false); x = t > x ? t : x;
    t = __builtin_amdgcn_update_dpp(lowest, x, 0x114, 0xF, 0xF, false); x = t > x ? t : x;
    t = __builtin_amdgcn_update_dpp(lowest, x, 0x118, 0xF, 0xF, false); x = t > x ? t : x;
    t = __builtin_amdgcn_update_dpp(lowest, x, 0x142, 0xA, 0xF, false); x = t > x ? t : x;
    t = __builtin_amdgcn_update_dpp(lowest, x, 0x143, 0xC, 0xF, false); x = t > x ? t : x;
    return x;
}

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// Compile-time loop: calls f(std::integral_constant<int, 0>{}) ... f(<N-1>{}) in order.
template <int I>
struct index_constant {
    static constexpr int value = I;
};
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(index_constant<I>{});
        static_for<N, I + 1>(f);
    }
}

}  // namespace macko
