// Loads whose completion is tracked by hand, shared by the SpMV kernels of libmacko_hip.so (internal;
// the public ABI is include/macko_hip.h).
//
// The tile ring, the row_ptr probes and the first pieces of x are fetched with inline-asm buffer
// loads into FIXED physical VGPRs and awaited with explicit s_waitcnt vmcnt(N).  Vector-memory
// loads complete in issue order, so "at most N loads outstanding" proves that every load older
// than the N youngest has landed; N is always the number of tracked loads issued after the one
// being awaited (loads or stores the compiler issues on its own can only make such a wait
// longer, never too short).  A kernel that uses these loads is compiled with
// amdgpu_num_vgpr(BASE), which keeps the register allocator below the fixed registers, so nothing
// else ever lives in them, and names every fixed register once in the clobber list of an empty asm
// statement (MACKO_RESERVE_FIXED_REGISTERS), which makes them part of the kernel's register count.
// A `take` copies a landed slot into ordinary registers after its wait.  The byte offset goes into
// the VGPR operand because only that operand takes part in the buffer's bounds check:
// past-the-end addresses read as zero without touching memory, which is also how "no tile" is
// encoded (kNoTile*).
//
// Register map, BASE = first fixed VGPR:  BASE, BASE+1 row_ptr probes;  BASE+2 .. BASE+9 two
// 16-byte pieces of x;  from BASE+10 the ring of depth D: slot j keeps its values in
// v[BASE+10+4j : BASE+13+4j] and its delta word in v(BASE+10+4D+j).  What lies behind the ring is
// the kernel's own.
#pragma once

#include "macko_spmv_detail.h"

namespace macko {
namespace spmv_detail {

#define MACKO_RESERVE_FIXED_REGISTERS(...) asm volatile("" ::: __VA_ARGS__)

template <int BASE>
struct TrackedLoads {
    // row_ptr probe k (k = 0, 1) -> v(BASE + k)
    template <int K>
    static __device__ __forceinline__ void probe_issue(u32 byte_offset, const u32x4 &buffer)
    {
        asm volatile("buffer_load_dword v%c2, %0, %1, 0 offen" ::"v"(byte_offset), "s"(buffer), "n"(BASE + K) : "memory");
    }
    template <int K, int N>
    static __device__ __forceinline__ int probe_take()
    {
        int w;
        asm volatile("s_waitcnt vmcnt(%1)\n\tv_mov_b32 %0, v%c2" : "=v"(w) : "n"(N), "n"(BASE + K) : "memory");
        return w;
    }

    // piece j of x (j = 0, 1) -> v[BASE+2+4j : BASE+5+4j]
    template <int J>
    static __device__ __forceinline__ void xpiece_issue(u32 byte_offset, const u32x4 &buffer)
    {
        asm volatile("buffer_load_dwordx4 v[%c2:%c3], %0, %1, 0 offen" ::"v"(byte_offset), "s"(buffer),
                     "n"(BASE + 2 + 4 * J), "n"(BASE + 5 + 4 * J)
                     : "memory");
    }
    // waits for piece j and writes it to LDS straight from its registers
    template <int J, int N>
    static __device__ __forceinline__ void xpiece_to_lds(u32 lds_byte_address)
    {
        asm volatile("s_waitcnt vmcnt(%1)\n\tds_write_b128 %0, v[%c2:%c3]" ::"v"(lds_byte_address), "n"(N),
                     "n"(BASE + 2 + 4 * J), "n"(BASE + 5 + 4 * J)
                     : "memory");
    }

    // Ring slot J of a D-deep ring: issue both loads.  VB = bytes per stored value: 2 (fp16, 16 bytes
    // per lane and tile) or 1 (int8, 8 bytes per lane and tile, which land in the first two registers
    // of the slot).  `stream` (wave-uniform) adds the non-temporal hint: the matrix is read once per
    // product, and a streaming read of that kind measures 11% faster with it at a few hundred MB.
    // Tiles shared with a neighbour go without it, so the second reader still finds them in L2.
    template <int D, int J, int VB>
    static __device__ __forceinline__ void ring_issue(u32 values_offset, u32 deltas_offset, const u32x4 &buf_values,
                                                      const u32x4 &buf_deltas, bool stream)
    {
        static_assert(J >= 0 && J < D && (VB == 1 || VB == 2), "ring slot");
        constexpr int V0 = BASE + 10 + 4 * J, DREG = BASE + 10 + 4 * D + J;
        if (VB == 2) {
            if (stream)
                asm volatile("buffer_load_dwordx4 v[%c4:%c5], %0, %2, 0 offen nt\n\tbuffer_load_dword v%c6, %1, %3, 0 offen nt"
                             ::"v"(values_offset), "v"(deltas_offset), "s"(buf_values), "s"(buf_deltas), "n"(V0),
                             "n"(V0 + 3), "n"(DREG) : "memory");
            else
                asm volatile("buffer_load_dwordx4 v[%c4:%c5], %0, %2, 0 offen\n\tbuffer_load_dword v%c6, %1, %3, 0 offen"
                             ::"v"(values_offset), "v"(deltas_offset), "s"(buf_values), "s"(buf_deltas), "n"(V0),
                             "n"(V0 + 3), "n"(DREG) : "memory");
        } else {
            if (stream)
                asm volatile("buffer_load_dwordx2 v[%c4:%c5], %0, %2, 0 offen nt\n\tbuffer_load_dword v%c6, %1, %3, 0 offen nt"
                             ::"v"(values_offset), "v"(deltas_offset), "s"(buf_values), "s"(buf_deltas), "n"(V0),
                             "n"(V0 + 1), "n"(DREG) : "memory");
            else
                asm volatile("buffer_load_dwordx2 v[%c4:%c5], %0, %2, 0 offen\n\tbuffer_load_dword v%c6, %1, %3, 0 offen"
                             ::"v"(values_offset), "v"(deltas_offset), "s"(buf_values), "s"(buf_deltas), "n"(V0),
                             "n"(V0 + 1), "n"(DREG) : "memory");
        }
    }

    // waits until at most N tracked loads issued after slot J's are outstanding and copies the slot out
    template <int D, int J, int N>
    static __device__ __forceinline__ void ring_take(u32x4 &v, u32 &d)
    {
        static_assert(J >= 0 && J < D, "ring slot");
        constexpr int V0 = BASE + 10 + 4 * J, DREG = BASE + 10 + 4 * D + J;
        asm volatile("s_waitcnt vmcnt(%5)\n\tv_mov_b32 %0, v%c6\n\tv_mov_b32 %1, v%c7\n\tv_mov_b32 %2, v%c8\n\tv_mov_b32 %3, v%c9"
                     "\n\tv_mov_b32 %4, v%c10"
                     : "=v"(v.x), "=v"(v.y), "=v"(v.z), "=v"(v.w), "=v"(d)
                     : "n"(N), "n"(V0), "n"(V0 + 1), "n"(V0 + 2), "n"(V0 + 3), "n"(DREG)
                     : "memory");
    }
};

// What of x does not travel through the two tracked pieces per thread goes to LDS through ordinary
// loads: everything with NB > 1 vectors (interleaved: element c of vector b at half-word c * NB + b)
// or a function applied while staging (XF: 1 = RMS norm, 2 = SiLU gate; SpmvArgs::x2), else the
// pieces beyond 2 * BLOCK (more than 16 * BLOCK columns) and an x that is not 16-byte aligned or of
// odd length.  Also zeroes the bytes in front of and behind x.  The caller provides the barrier.
template <int BLOCK, bool X_LDS, int NB, int XF>
__device__ __forceinline__ void stage_x_untracked(unsigned char *lds, const SpmvArgs &a, int tid, int lane, int wave,
                                                  bool x_vec, int x_nvec)
{
    constexpr int WAVES = BLOCK / kWave;
    if (NB > 1) {
        // every vector through ordinary loads, interleaved: element c of vector b at dst[c * NB + b]
        uint16_t *dst = reinterpret_cast<uint16_t *>(lds + kLdsFront * NB);
        const bool vec_ok = x_vec && (a.ldx & 7) == 0;
        const int nvec = vec_ok ? a.cols >> 3 : 0;
        // 8 columns of every vector per thread and step: NB 16-byte loads, interleaved in registers,
        // written back as NB 16-byte stores (16 * NB contiguous bytes of LDS)
        for (int i = tid; i < nvec; i += BLOCK) {
            u32x4 v[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b)
                v[b] = reinterpret_cast<const u32x4 *>(a.x + (size_t)b * (size_t)a.ldx)[i];
            u32 out[4 * NB];  // half-word (c * NB + b) = element c of vector b
#pragma unroll
            for (int c = 0; c < 8; ++c) {
#pragma unroll
                for (int b = 0; b < NB; b += 2) {
                    const u32 lo = (v[b][c >> 1] >> (16 * (c & 1))) & 0xffffu;
                    const u32 hi = (v[b + 1][c >> 1] >> (16 * (c & 1))) & 0xffffu;
                    out[(c * NB + b) >> 1] = lo | (hi << 16);
                }
            }
            u32x4 *d4 = reinterpret_cast<u32x4 *>(dst + (size_t)8 * i * NB);
#pragma unroll
            for (int q = 0; q < NB; ++q) d4[q] = u32x4{out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]};
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint16_t *xb = a.x + (size_t)b * (size_t)a.ldx;
            for (int i = (nvec << 3) + tid; i < a.cols; i += BLOCK) dst[i * NB + b] = xb[i];
        }
        if (tid < kLdsFront * NB / 4) reinterpret_cast<u32 *>(lds)[tid] = 0;
        if (tid < kLdsBack * NB / 2) dst[a.cols * NB + tid] = 0;
    } else if (XF != 0) {
        uint16_t *dst = reinterpret_cast<uint16_t *>(lds + kLdsFront);
        u32x4 *d4 = reinterpret_cast<u32x4 *>(dst);
        const int nvec = a.cols >> 3;
        auto lo = [](u32 w) { return half_bits_to_float((uint16_t)(w & 0xffffu)); };
        auto hi = [](u32 w) { return half_bits_to_float((uint16_t)(w >> 16)); };
        auto pack = [](float l, float h) { return (u32)float_to_half_bits(l) | ((u32)float_to_half_bits(h) << 16); };
        if (XF == 1) {
            // pass 1: raw x into LDS and the sum of squares; pass 2: each thread scales the pieces
            // it wrote itself, so only the sum needs a barrier
            float ss = 0.f;
            for (int i = tid; i < nvec; i += BLOCK) {
                const u32x4 v = reinterpret_cast<const u32x4 *>(a.x)[i];
                d4[i] = v;
#pragma unroll
                for (int e = 0; e < 4; ++e) ss += lo(v[e]) * lo(v[e]) + hi(v[e]) * hi(v[e]);
            }
            float *red = reinterpret_cast<float *>(lds + kLdsFront + 2 * (size_t)a.cols + kLdsBack);
            const float ws = wave_sum(ss);
            if (lane == 0) red[wave] = ws;
            __syncthreads();
            float total = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) total += red[w];
            const float inv = rsqrtf(total / (float)a.cols + a.eps);
            for (int i = tid; i < nvec; i += BLOCK) {
                const u32x4 v = d4[i];
                const u32x4 g = reinterpret_cast<const u32x4 *>(a.x2)[i];
                u32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = pack(lo(v[e]) * inv * lo(g[e]), hi(v[e]) * inv * hi(g[e]));
                d4[i] = o;
            }
        } else {
            auto gate = [](float g, float u) { return g / (1.0f + __expf(-g)) * u; };
            for (int i = tid; i < nvec; i += BLOCK) {
                const u32x4 g = reinterpret_cast<const u32x4 *>(a.x)[i];
                const u32x4 u = reinterpret_cast<const u32x4 *>(a.x2)[i];
                u32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = pack(gate(lo(g[e]), lo(u[e])), gate(hi(g[e]), hi(u[e])));
                d4[i] = o;
            }
        }
        if (tid < kLdsFront / 4) reinterpret_cast<u32 *>(lds)[tid] = 0;
        if (tid < kLdsBack / 2) dst[a.cols + tid] = 0;
    } else if (X_LDS) {
        uint16_t *dst = reinterpret_cast<uint16_t *>(lds + kLdsFront);
        u32x4 *d4 = reinterpret_cast<u32x4 *>(dst);
        if (__builtin_expect(x_nvec > kXRegs * BLOCK, 0))
            for (int i = tid + kXRegs * BLOCK; i < x_nvec; i += BLOCK) d4[i] = reinterpret_cast<const u32x4 *>(a.x)[i];
        if (__builtin_expect((x_nvec << 3) < a.cols, 0))
            for (int i = (x_nvec << 3) + tid; i < a.cols; i += BLOCK) dst[i] = a.x[i];
        if (tid < kLdsFront / 4) reinterpret_cast<u32 *>(lds)[tid] = 0;
        if (tid < kLdsBack / 2) dst[a.cols + tid] = 0;
    }
}

}  // namespace spmv_detail
}  // namespace macko
