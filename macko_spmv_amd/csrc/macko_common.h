// Shared host/device helpers of libmacko_hip.so (internal; the public ABI is include/macko_hip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

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
