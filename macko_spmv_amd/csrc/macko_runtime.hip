// Host-side odds and ends of libmacko_hip.so: device facts, error text, ABI version.

#include <string.h>

#include <atomic>

#include "macko_common.h"

namespace macko {

int device_info(DeviceInfo *out)
{
    constexpr int kMaxDevices = 64;
    // per device: 0 = unknown, 1 = being written, 2 = known.  Concurrent first calls may both query
    // the device; only one of them writes the cache entry, readers wait for state 2.
    static DeviceInfo cache[kMaxDevices];
    static std::atomic<int> state[kMaxDevices];
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e == hipErrorNoDevice ? MACKO_E_NO_DEVICE : (int)e;
    const bool cached = dev >= 0 && dev < kMaxDevices;
    if (cached && state[dev].load(std::memory_order_acquire) == 2) {
        *out = cache[dev];
        return 0;
    }
    DeviceInfo info;
    e = hipDeviceGetAttribute(&info.compute_units, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return (int)e;
    // gfx950 gives a workgroup up to 160 KiB of LDS; anything else is treated as 64 KiB
    info.max_lds_bytes = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 160 * 1024 : 64 * 1024;
    if (cached) {
        int expected = 0;
        if (state[dev].compare_exchange_strong(expected, 1, std::memory_order_acq_rel)) {
            cache[dev] = info;
            state[dev].store(2, std::memory_order_release);
        }
    }
    *out = info;
    return 0;
}

}  // namespace macko

extern "C" int macko_hip_abi_version(void) { return 2; }

extern "C" const char *macko_hip_error_string(int code)
{
    switch (code) {
    case 0: return "success";
    case MACKO_E_INVALID_ARGUMENT: return "macko: invalid argument (null/misaligned pointer, negative or oversized dimension)";
    case MACKO_E_NO_DEVICE: return "macko: no usable HIP device";
    default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "macko: unknown error code";
}
