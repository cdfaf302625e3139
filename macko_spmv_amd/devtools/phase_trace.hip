// phase_trace: per-wave phase timestamps of the SpMV kernels.
//
// Loads the tracing build of the library (libmacko_hip_trace.so: the product sources compiled with
// -DMACKO_DEV_HOOKS, which adds s_memrealtime stamps at the kernels' phase boundaries and two
// extra entry points, macko_spmv_set_trace and macko_spmv_tune), compresses a synthetic matrix,
// runs the product repeatedly over rotating copies and prints, for the last launch, when the
// waves reached each phase: as percentiles over all waves, by XCD, by wave slot within the
// workgroup, and as the spread within workgroups.  The shipped library has none of this.
//
// usage (from the repository root, or with MACKO_TRACE_LIBRARY naming the tracing library):
//   phase_trace ROWS COLS DENSITY [ring-depth workgroups unused split(1|-1)]
//   (a negative DENSITY gives rows of power-law length with mean -DENSITY)
// build: python -m macko_spmv_amd._build --devtools
#include <hip/hip_runtime.h>
#include <dlfcn.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>
#include <algorithm>
#include <cmath>
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); exit(1);} } while (0)
typedef int (*spmv_fn)(const void*, const void*, const int32_t*, const void*, void*, int32_t, int32_t, int64_t, void*);
typedef int (*count_fn)(const void*, int32_t, int32_t, int32_t*, void*);
typedef int (*fill_fn)(const void*, int32_t, int32_t, const int32_t*, void*, void*, int64_t, void*);
typedef void (*tune_fn)(int, int, int, int);
typedef void (*trace_fn)(long long*);
__device__ inline uint32_t hash32(uint32_t x) { x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16; return x; }
// row_density == nullptr: every element is kept with probability `density`; else row r with row_density[r]
__global__ void k_gen_dense(uint16_t* M, int rows, int cols, float density, const float* row_density, uint32_t seed)
{
    size_t n = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t h = hash32(hash32((uint32_t)i) ^ (seed * 0x9e3779b9u + 77u));
        float u = (h >> 8) * (1.0f / 16777216.0f);
        if (row_density) density = row_density[i / cols];
        uint16_t v = 0;
        if (u < density) { v = (uint16_t)(0x2000 + (hash32(h) & 0x0fff)); if (h & 1) v |= 0x8000; }
        M[i] = v;
    }
}
int main(int argc, char** argv)
{
    void* hn = dlopen(getenv("MACKO_TRACE_LIBRARY") ? getenv("MACKO_TRACE_LIBRARY") : "macko_spmv_amd/devtools/libmacko_hip_trace.so", RTLD_NOW | RTLD_LOCAL);
    if (!hn) { printf("dlopen: %s\n", dlerror()); return 1; }
    spmv_fn spmv = (spmv_fn)dlsym(hn, "macko_spmv_f16");
    count_fn cnt = (count_fn)dlsym(hn, "macko_compress_f16_count"); fill_fn fil = (fill_fn)dlsym(hn, "macko_compress_f16_fill");
    tune_fn tune = (tune_fn)dlsym(hn, "macko_spmv_tune"); trace_fn set_trace = (trace_fn)dlsym(hn, "macko_spmv_set_trace");
    if (!tune || !set_trace) { printf("library has no development hooks\n"); return 1; }
    int R = atoi(argv[1]), C = atoi(argv[2]); float d = atof(argv[3]);
    tune(argc > 4 ? atoi(argv[4]) : 0, argc > 5 ? atoi(argv[5]) : 0, argc > 6 ? atoi(argv[6]) : 0, argc > 7 ? atoi(argv[7]) : 0);
    hipStream_t s; CK(hipStreamCreate(&s));
    uint16_t* M; CK(hipMalloc(&M, (size_t)R * C * 2));
    float* row_density = nullptr;
    if (d < 0) {  // skewed rows: density ~ 0.01 * Pareto(1.5), clipped to [0.01, 0.95], rescaled to mean -d
        std::vector<double> rd(R);
        for (int r = 0; r < R; r++) {
            uint32_t h = 0x9e3779b9u * (uint32_t)(r + 1); h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
            double u = ((h >> 8) + 0.5) / 16777216.0;
            rd[r] = std::min(0.95, std::max(0.01, 0.01 * pow(1.0 - u, -1.0 / 1.5)));
        }
        for (int it = 0; it < 20; it++) {
            double m = 0; for (double v : rd) m += v; m /= R;
            for (double& v : rd) v = std::min(0.95, std::max(0.01, v * (-d / m)));
        }
        std::vector<float> rf(rd.begin(), rd.end());
        CK(hipMalloc(&row_density, R * sizeof(float)));
        CK(hipMemcpy(row_density, rf.data(), R * sizeof(float), hipMemcpyHostToDevice));
    }
    hipLaunchKernelGGL(k_gen_dense, dim3(2048), dim3(256), 0, s, M, R, C, d, row_density, 12345u);
    int ncopy = (int)std::max<size_t>(3, std::min<size_t>(24, (size_t)1500000000 / ((size_t)((double)R * C * fabs(d) * 3) + 1)));
    std::vector<int*> rp(ncopy); std::vector<uint8_t*> v(ncopy), dl(ncopy);
    CK(hipMalloc(&rp[0], (R + 1) * 4));
    cnt(M, R, C, rp[0], s);
    int n; CK(hipMemcpyAsync(&n, rp[0] + R, 4, hipMemcpyDeviceToHost, s)); CK(hipStreamSynchronize(s));
    long long P = ((long long)n + 7) / 8 * 8;
    CK(hipMalloc(&v[0], P * 2)); CK(hipMalloc(&dl[0], P / 2));
    fil(M, R, C, rp[0], v[0], dl[0], P, s);
    for (int k = 1; k < ncopy; k++) {
        CK(hipMalloc(&rp[k], (R + 1) * 4)); CK(hipMalloc(&v[k], P * 2)); CK(hipMalloc(&dl[k], P / 2));
        CK(hipMemcpyAsync(rp[k], rp[0], (R + 1) * 4, hipMemcpyDeviceToDevice, s));
        CK(hipMemcpyAsync(v[k], v[0], P * 2, hipMemcpyDeviceToDevice, s));
        CK(hipMemcpyAsync(dl[k], dl[0], P / 2, hipMemcpyDeviceToDevice, s));
    }
    uint16_t* x; CK(hipMalloc(&x, C * 2)); CK(hipMemset(x, 0x3c, C * 2));
    uint16_t* y; CK(hipMalloc(&y, R * 2));
    const int max_waves = 256 * 16;
    long long* trace; CK(hipMalloc(&trace, (size_t)max_waves * 8 * 8));
    CK(hipMemsetAsync(trace, 0, (size_t)max_waves * 8 * 8, s));
    const int last_it = 40;
    for (int it = 0; it <= last_it; it++) {
        set_trace(it == last_it ? trace : nullptr);
        hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
        if (it >= last_it - 3) CK(hipStreamSynchronize(s));
        CK(hipEventRecord(a, s));
        int rc = spmv(v[it % ncopy], dl[it % ncopy], rp[it % ncopy], x, y, R, C, P, s);
        CK(hipEventRecord(b, s)); CK(hipEventSynchronize(b));
        float ms; CK(hipEventElapsedTime(&ms, a, b));
        if (it >= last_it - 2) printf("launch %d rc=%d event time %.2f us\n", it, rc, ms * 1e3);
    }
    std::vector<long long> h((size_t)max_waves * 8);
    CK(hipMemcpy(h.data(), trace, h.size() * 8, hipMemcpyDeviceToHost));
    long long t0 = -1; int nw = 0;
    for (int w = 0; w < max_waves; w++) if (h[w * 8]) { nw++; if (t0 < 0 || h[w * 8] < t0) t0 = h[w * 8]; }
    printf("shape %dx%d d=%.2f P=%lld (%.1f MB) waves traced %d\n", R, C, d, P, P * 2.5 / 1e6, nw);
    const char* names[8] = {"start", "x staged", "cuts (fast)", "x in lds", "after barrier", "loop start", "loop end", "kernel end"};
    for (int sl = 0; sl < 8; sl++) {
        std::vector<double> ts;
        for (int w = 0; w < max_waves; w++) if (h[w * 8] && h[w * 8 + sl]) ts.push_back((h[w * 8 + sl] - t0) * 0.01);
        if (ts.empty()) continue;
        std::sort(ts.begin(), ts.end());
        printf("  %-14s n=%5zu  min %6.2f  p10 %6.2f  med %6.2f  p90 %6.2f  max %6.2f us\n", names[sl], ts.size(), ts.front(), ts[ts.size() / 10], ts[ts.size() / 2], ts[ts.size() * 9 / 10], ts.back());
    }
    std::vector<double> dur;
    for (int w = 0; w < max_waves; w++) if (h[w * 8] && h[w * 8 + 6] && h[w * 8 + 5]) dur.push_back((h[w * 8 + 6] - h[w * 8 + 5]) * 0.01);
    std::sort(dur.begin(), dur.end());
    if (!dur.empty()) printf("  loop duration per wave: min %.2f p10 %.2f med %.2f p90 %.2f p99 %.2f max %.2f us\n", dur.front(), dur[dur.size() / 10], dur[dur.size() / 2], dur[dur.size() * 9 / 10], dur[dur.size() * 99 / 100], dur.back());
    {
        // breakdowns of loop end and duration: by XCD (32 consecutive logical workgroups), by wave slot, and within workgroups
        auto stat = [&](const char* what, int groups, auto group_of) {
            printf("  by %s (loop end med/max | duration med/max):\n", what);
            for (int g = 0; g < groups; g++) {
                std::vector<double> e, du;
                for (int w = 0; w < max_waves; w++) if (h[w * 8] && h[w * 8 + 6] && group_of(w) == g) { e.push_back((h[w * 8 + 6] - t0) * 0.01); du.push_back((h[w * 8 + 6] - h[w * 8 + 5]) * 0.01); }
                if (e.empty()) continue;
                std::sort(e.begin(), e.end()); std::sort(du.begin(), du.end());
                printf("    %2d: %6.2f %6.2f | %6.2f %6.2f\n", g, e[e.size() / 2], e.back(), du[du.size() / 2], du.back());
            }
        };
        stat("xcd", 8, [](int w) { return (w / 16) / 32; });
        stat("wave slot", 16, [](int w) { return w % 16; });
        std::vector<double> spread, wgend;
        for (int g = 0; g < max_waves / 16; g++) {
            double lo = 1e9, hi = -1; 
            for (int w = g * 16; w < g * 16 + 16; w++) if (h[w * 8] && h[w * 8 + 6]) { double e = (h[w * 8 + 6] - t0) * 0.01; lo = std::min(lo, e); hi = std::max(hi, e); }
            if (hi >= 0) { spread.push_back(hi - lo); wgend.push_back(hi); }
        }
        std::sort(spread.begin(), spread.end()); std::sort(wgend.begin(), wgend.end());
        if (!spread.empty()) printf("  within workgroup: spread of loop end med %.2f max %.2f; workgroup end min %.2f med %.2f max %.2f\n", spread[spread.size() / 2], spread.back(), wgend.front(), wgend[wgend.size() / 2], wgend.back());
    }
    return 0;
}