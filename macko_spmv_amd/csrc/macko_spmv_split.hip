// MACKO sparse matrix-vector product for gfx950, the kernel for matrices with few, long rows.
//
// macko_spmv.hip gives every wave whole rows.  With fewer rows than waves that leaves waves
// idle, and a row longer than a wave's fair share cannot be balanced at all.  Here the WORKGROUP
// owns whole rows (the ones that start nearest to its even share of the stored entries), and the
// tiles that hold them are dealt evenly to its waves, so a wave's share does not depend on where
// rows begin or end: rows are split between waves wherever a share ends.  A wave that starts
// inside a row first sums the nibbles of the row's earlier entries ("look-back": the deltas
// only, a fifth of the bytes, requested ahead of time as far back as rows usually reach) to
// know at which column it continues; the pieces of a row that spans several waves meet in LDS
// at the end of the kernel.  Nothing is shared between workgroups: no atomics, no second pass,
// no scratch memory.  With fewer rows than compute units the launch has one workgroup per row.
//
// Per tile: one pass, whatever rows begin inside it (see starts_tile); the streaming machinery
// (x in LDS, hand-tracked ring of tile loads, v_dot8_u32_u4 column decode) is that of macko_spmv.hip.
//
// Behaviour restated from src/macko_spmv/cuda/kernels.cuh:34-124 of the upstream package.

#include <atomic>

#include "macko_spmv_tracked.h"

namespace macko {
namespace {

using namespace spmv_detail;

// The hand-tracked loads (macko_spmv_tracked.h) with this kernel's register map: the compiler keeps
// below v84; v84,v85 row_ptr probes; v86..v93 two 16-byte pieces of x; v94..v103 the ring (D <= 2);
// v104..v119 four 16-byte pieces of the deltas in front of a wave's first entry ("look-back").
constexpr int kCompilerVgprs = 84;
#define MACKO_SPLIT_FIXED_REGISTERS "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119"
typedef TrackedLoads<kCompilerVgprs> Tracked;
template <int K> __device__ __forceinline__ void probe_issue(u32 o, const u32x4 &b) { Tracked::probe_issue<K>(o, b); }
template <int K, int N> __device__ __forceinline__ int probe_take() { return Tracked::probe_take<K, N>(); }
template <int J> __device__ __forceinline__ void xpiece_issue(u32 o, const u32x4 &b) { Tracked::xpiece_issue<J>(o, b); }
template <int J, int N> __device__ __forceinline__ void xpiece_to_lds(u32 a) { Tracked::xpiece_to_lds<J, N>(a); }
template <int D, int J, int VB>
__device__ __forceinline__ void ring_issue(u32 vo, u32 dof, const u32x4 &bv, const u32x4 &bd, bool stream)
{
    static_assert(D == 1 || D == 2, "ring depth");
    Tracked::ring_issue<D, J, VB>(vo, dof, bv, bd, stream);
}
template <int D, int J, int N> __device__ __forceinline__ void ring_take(u32x4 &v, u32 &d) { Tracked::ring_take<D, J, N>(v, d); }

// look-back piece j (j = 0..3) -> v[104+4j : 107+4j]
template <int J>
__device__ __forceinline__ void look_issue(u32 byte_offset, const u32x4 &buffer)
{
    if (J == 0) asm volatile("buffer_load_dwordx4 v[104:107], %0, %1, 0 offen" ::"v"(byte_offset), "s"(buffer) : "memory", "v104", "v105", "v106", "v107");
    if (J == 1) asm volatile("buffer_load_dwordx4 v[108:111], %0, %1, 0 offen" ::"v"(byte_offset), "s"(buffer) : "memory", "v108", "v109", "v110", "v111");
    if (J == 2) asm volatile("buffer_load_dwordx4 v[112:115], %0, %1, 0 offen" ::"v"(byte_offset), "s"(buffer) : "memory", "v112", "v113", "v114", "v115");
    if (J == 3) asm volatile("buffer_load_dwordx4 v[116:119], %0, %1, 0 offen" ::"v"(byte_offset), "s"(buffer) : "memory", "v116", "v117", "v118", "v119");
}
#define MACKO_LOOK_TAKE(A, B, C, E)                                                                                 \
    asm volatile("s_waitcnt vmcnt(%4)\n\tv_mov_b32 %0, " A "\n\tv_mov_b32 %1, " B "\n\tv_mov_b32 %2, " C           \
                 "\n\tv_mov_b32 %3, " E                                                                              \
                 : "=v"(v.x), "=v"(v.y), "=v"(v.z), "=v"(v.w) : "n"(N) : "memory")
template <int J, int N>
__device__ __forceinline__ u32x4 look_take()
{
    u32x4 v;
    if (J == 0) MACKO_LOOK_TAKE("v104", "v105", "v106", "v107");
    if (J == 1) MACKO_LOOK_TAKE("v108", "v109", "v110", "v111");
    if (J == 2) MACKO_LOOK_TAKE("v112", "v113", "v114", "v115");
    if (J == 3) MACKO_LOOK_TAKE("v116", "v117", "v118", "v119");
    return v;
}


// NB = vectors multiplied per launch (1, 2, 4 or 8).  With NB > 1 the NB copies of x are interleaved in
// LDS (element c of vector b at half-word c * NB + b), so one LDS read per stored entry fetches the
// operand of every vector, and a row ends with NB sums.  NB > 1 exists for fp16 values, x in LDS,
// plain product only.
// XF = function applied to the input while it is staged into LDS, so the producer of x needs no
// launch of its own: 0 = none (x as given), 1 = RMS norm (x * rsqrt(mean(x^2) + eps) * x2, x2 the
// norm weight), 2 = SiLU gate (silu(x) * x2).  The staged vector is rounded to fp16 exactly as a
// separate kernel writing it to memory would.  XF != 0 needs cols % 8 == 0 and 16-byte aligned x, x2.
template <int BLOCK, int D, bool X_LDS, bool AXPBY, int VB, int NB, int XF>
__global__ void __launch_bounds__(BLOCK) __attribute__((amdgpu_num_vgpr(kCompilerVgprs)))
spmv_split_kernel(const SpmvArgs a)
{
    static_assert(NB == 1 || (NB <= 8 && X_LDS && !AXPBY && VB == 2), "batched variant: fp16, x in LDS, plain product");
    static_assert(XF == 0 || (NB == 1 && X_LDS && VB == 2), "fused staging: fp16, one vector, x in LDS");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    MACKO_RESERVE_FIXED_REGISTERS(MACKO_SPLIT_FIXED_REGISTERS);
    constexpr int WAVES = BLOCK / kWave;
    constexpr int kBatchShift = NB == 8 ? 3 : (NB == 4 ? 2 : (NB == 2 ? 1 : 0));
    constexpr int kTileLoads = 2 * D;  // tracked loads per full ring
    constexpr int kPre = 1;  // ring slots filled before the workgroup's barrier
    constexpr int kNone = 0x7fffffff;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = uniform(tid >> 6);
    const u32 n_wg = gridDim.x;
    // Workgroups are dealt round-robin to the 8 XCDs (workgroup i runs on XCD i % 8).  Giving XCD k
    // the k-th contiguous eighth of the matrix keeps neighbouring workgroups, which share boundary
    // tiles, behind one L2.
    u32 wg = blockIdx.x;
    if ((gridDim.x & 7) == 0) wg = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
#ifdef MACKO_DEV_HOOKS
    const u32 stamp_wave = wg * WAVES + (u32)wave;
#endif
    MACKO_STAMP(0);

    const u32x4 buf_values = make_buffer(a.values, (u32)(a.padded * VB));
    const u32x4 buf_deltas = make_buffer(a.deltas, (u32)(a.padded / 2));
    const u32x4 buf_rows = make_buffer(a.row_ptr, ((u32)a.rows + 1) * 4);
    const __amdgpu_buffer_rsrc_t rs_x =
        __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.cols * 2, 0x00020000);
    (void)rs_x;
    const __amdgpu_buffer_rsrc_t rs_deltas =
        __builtin_amdgcn_make_buffer_rsrc((void *)a.deltas, 0, (int)(a.padded / 2), 0x00020000);
    const u32 lane_values = (u32)lane * (kChunk * VB), lane4 = (u32)lane * 4;

    const bool x_vec = (reinterpret_cast<uintptr_t>(a.x) & 15) == 0;
    const int x_nvec = x_vec ? a.cols >> 3 : 0;

    // ---- 1. tracked loads, oldest first: row_ptr probes, x pieces ------------------------------------
    // probes: 64 consecutive row_ptr values around where my workgroup's first row and the next
    // workgroup's first row should be
    const int n_active = 1 << a.active_shift;
    const bool active = wave < n_active;  // wave-uniform
    const u32 unit = wg, n_units = n_wg;  // the workgroup owns whole rows
    int target[2] = {0, 0}, base[2] = {0, 0}, guess[2] = {0, 0};
    if (active) {
        target[0] = (int)even_split(unit, a.entries_q, a.entries_rem);  // < P < 2^31
        target[1] = (int)even_split(unit + 1, a.entries_q, a.entries_rem);
        guess[0] = (int)(unit * a.rows_q + __umulhi(unit, a.rows_frac));
        guess[1] = unit == n_units - 1 ? a.rows : (int)((unit + 1) * a.rows_q + __umulhi(unit + 1, a.rows_frac));
        base[0] = probe_base(guess[0], a.rows);
        base[1] = probe_base(guess[1], a.rows);
        int i0 = base[0] + lane, i1 = base[1] + lane;
        i0 = i0 <= a.rows ? i0 : a.rows;
        i1 = i1 <= a.rows ? i1 : a.rows;
        probe_issue<0>((u32)i0 * 4, buf_rows);
        probe_issue<1>((u32)i1 * 4, buf_rows);
    }
    const u32x4 buf_x = make_buffer(a.x, (u32)x_nvec * 16);  // past the end reads as zero
    if (X_LDS && NB == 1 && XF == 0) {
        xpiece_issue<0>((u32)tid * 16, buf_x);
        xpiece_issue<1>((u32)(tid + BLOCK) * 16, buf_x);
    }
    auto issue_slot = [&](auto slot, u32 tile, bool fetch, bool stream) {
        constexpr int J = decltype(slot)::value;
        ring_issue<D, J, VB>(lane_values + (fetch ? tile * (u32)(kTile * VB) : kNoTileValues),
                         lane4 + (fetch ? tile << (kTileShift - 1) : kNoTileDeltas), buf_values, buf_deltas, stream);
    };
    // ---- 2. x: everything beyond the two register pieces per thread, and unaligned or odd-length
    //         x, goes to LDS through ordinary loads (rare: more than 16384 columns, or an x that is
    //         not 16-byte aligned) ------------------------------------------------------------------
    stage_x_untracked<BLOCK, X_LDS, NB, XF>(lds, a, tid, lane, wave, x_vec, x_nvec);
    MACKO_STAMP(1);

    constexpr int kXLoads = X_LDS && NB == 1 && XF == 0 ? kXRegs : 0;
    constexpr size_t kXBytesFixed = (size_t)NB * (kLdsFront + kLdsBack) + (XF == 1 ? 64 : 0);
    // behind x in LDS: one piece of a row sum per wave and vector, one flag per wave (section 8)
    size_t lead_off = X_LDS ? kXBytesFixed + (size_t)NB * 2 * (size_t)a.cols : 0;
    lead_off = (lead_off + 3) & ~(size_t)3;
    float *lead_lds = reinterpret_cast<float *>(lds + lead_off);
    int *flag_lds = reinterpret_cast<int *>(lds + lead_off + (size_t)NB * WAVES * 4);

    if (!active) {
        // a wave that streams no tiles: its share of x, then the workgroup's two barriers
        if (kXLoads != 0) {
            const u32 lds_x = (u32)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds + kLdsFront;
            const u32 dst0 = lds_x + (u32)tid * 16, dst1 = dst0 + BLOCK * 16;
            if (tid < x_nvec) xpiece_to_lds<0, 1>(dst0);
            if (tid + BLOCK < x_nvec) xpiece_to_lds<1, 0>(dst1);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        if (X_LDS) __syncthreads();
        __syncthreads();
        return;
    }

    // ---- 3. which rows are my workgroup's: rows [rho0, rho1), stored entries [cut0, cut1) ---------------
    int window[2];
    window[0] = probe_take<0, kXLoads + 1>();
    window[1] = probe_take<1, kXLoads>();
    int rho0 = 0, rho1 = 0, cut0 = 0, cut1 = 0;
    {
        // Cut k is the first row start at or after target k, or the one before it if that is
        // nearer; the first workgroup starts at row 0, the last one ends at the last row.
        bool ok[2] = {true, true};
        int rho[2] = {0, 0}, cut[2] = {0, 0};
        if (a.row_even) {  // the cuts are the guesses themselves; both lie inside their windows
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                rho[k] = guess[k];
                cut[k] = __builtin_amdgcn_readlane(window[k], guess[k] - base[k]);
            }
        } else {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const u32 edge = unit + (u32)k;
                if (edge == 0) {
                    rho[k] = 0;
                    cut[k] = 0;
                } else if (edge == n_units) {
                    rho[k] = a.rows;
                    cut[k] = __builtin_amdgcn_readlane(window[k], a.rows - base[k]);
                } else {
                    const unsigned long long m = __ballot(window[k] >= target[k]);
                    const int f = m ? __builtin_ctzll(m) : 0;
                    if (__builtin_expect(f >= 1, 1)) {
                        const int at = __builtin_amdgcn_readlane(window[k], f);
                        const int before = __builtin_amdgcn_readlane(window[k], f - 1);
                        const int back = target[k] - before < at - target[k] ? 1 : 0;
                        rho[k] = base[k] + f - back;
                        cut[k] = back ? before : at;
                    } else {
                        ok[k] = false;
                    }
                }
            }
        }
        MACKO_STAMP(2);
        if (__builtin_expect(!(ok[0] && ok[1]), 0)) {
            // General case: search rounds where a window missed.
            int range[2];
            wave_lower_bound2(a.row_ptr, a.rows, lane, target, window, base, range);
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                if (ok[k]) continue;
                int rr = range[k];
                int at;
                if (rr >= base[k] && rr <= base[k] + 63)
                    at = __builtin_amdgcn_readlane(window[k], rr - base[k]);
                else
                    at = uniform(a.row_ptr[rr]);
                if (rr > 0) {
                    int before;
                    if (rr - 1 >= base[k] && rr - 1 <= base[k] + 63)
                        before = __builtin_amdgcn_readlane(window[k], rr - 1 - base[k]);
                    else
                        before = uniform(a.row_ptr[rr - 1]);
                    if (target[k] - before < at - target[k]) {
                        rr -= 1;
                        at = before;
                    }
                }
                rho[k] = rr;
                cut[k] = at;
            }
            // nothing the compiler loaded on this path may still count as outstanding later on
            __builtin_amdgcn_s_waitcnt(0x0f70);
        }
        rho0 = uniform(rho[0]);
        rho1 = uniform(rho[1]);
        cut0 = uniform(cut[0]);
        cut1 = uniform(cut[1]);
        if (rho1 < rho0) rho1 = rho0;
        if (cut1 < cut0) cut1 = cut0;
    }

    // ---- 4. my tiles: the workgroup's tiles dealt evenly to its waves -------------------------------------
    const u32 tile_first = (u32)cut0 >> kTileShift;
    const u32 tile_end = rho0 < rho1 ? ((u32)cut1 + kTile - 1) >> kTileShift : tile_first;
    const u32 n_tiles = tile_end > tile_first ? tile_end - tile_first : 0u;
    const u32 T0 = tile_first + (((u32)wave * n_tiles) >> a.active_shift);
    const u32 T1 = tile_first + (((u32)(wave + 1) * n_tiles) >> a.active_shift);
    const int g0 = (int)(T0 << kTileShift);
    const bool first_wave = wave == 0;           // my first tile may be shared with another workgroup
    const bool last_wave = wave == n_active - 1;  // so may my last one

    // ---- 5. the ring: my first tiles are requested before x is even in LDS; they fly while the
    //         workgroup finishes the copy and meets at the barrier.  Only kPre slots are filled
    //         here: what the early waves of a compute unit request queues in front of the late
    //         waves' probes and pieces of x, and the barrier waits for the latest wave. --------------
    constexpr int kLookLoads = 4;
    {
        // look-back: pieces of 2048 entries going back from my first entry; a lane asks for its 32
        // entries only if they lie within look_entries of it (nothing is in progress at the
        // workgroup's first entry)
        const bool fetch = T0 != tile_first && T0 < T1;
        static_for<4>([&](auto piece) {
            constexpr int J = decltype(piece)::value;
            const int lo = g0 - (J + 1) * kLookBack + 32 * lane;  // my first entry of this piece
            const bool mine = fetch && g0 - lo <= (int)a.look_entries;
            look_issue<J>(mine ? (u32)(lo >> 1) : kNoTileDeltas, buf_deltas);
        });
    }
    static_for<kPre>([&](auto slot) {
        constexpr int J = decltype(slot)::value;
        const u32 t = T0 + J;
        issue_slot(slot, t, t < T1, !((first_wave && J == 0) || (last_wave && t + 1 == T1)));
    });
    __builtin_amdgcn_sched_barrier(0);

    // ---- 6. x pieces into LDS (older than the ring loads just issued) -----------------------------------
    if (NB > 1 || XF != 0) {
        __syncthreads();
    } else if (X_LDS) {
        const u32 lds_x = (u32)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds + kLdsFront;
        const u32 dst0 = lds_x + (u32)tid * 16, dst1 = dst0 + BLOCK * 16;
        if (tid < x_nvec) xpiece_to_lds<0, 2 * kPre + kLookLoads + 1>(dst0);
        if (tid + BLOCK < x_nvec) xpiece_to_lds<1, 2 * kPre + kLookLoads>(dst1);
        // the copies above are asm the compiler's wait tracking does not see
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        MACKO_STAMP(3);
        __syncthreads();
    }
    MACKO_STAMP(4);


    // the rest of the ring
    static_for<D>([&](auto slot) {
        constexpr int J = decltype(slot)::value;
        if constexpr (J >= kPre) {
            const u32 t = T0 + J;
            issue_slot(slot, t, t < T1, !(last_wave && t + 1 == T1));
        }
    });
    __builtin_amdgcn_sched_barrier(0);

    // ---- 6b. which rows my tiles hold (the loads are in flight) -----------------------------------------
    // window of row_ptr values the row walk reads row starts from: lane i holds row_ptr[win_base + i]
    int win_base = base[0];
    int win = window[0];
    auto row_start = [&](int r) -> int {  // r in [win_base, win_base + 63]
        return __builtin_amdgcn_readlane(win, r - win_base);
    };
    auto reload_window = [&](int r) {  // rows r .. r + 63 become addressable
        win_base = r;
        win = load_row_window(a.row_ptr, a.rows, win_base, lane);
        // Awaited on the spot: a load the compiler still counts as outstanding at the loop's
        // back edge makes it protect the register with a vmcnt(0) at the top of every
        // iteration, which would also wait for the ring loads just issued.
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), expcnt and lgkmcnt untouched
    };
    auto need_row = [&](int r) {  // make row r addressable
        if (__builtin_expect(r < win_base || r > win_base + 63, 0)) reload_window(r);
    };

    // first row that starts at or behind my first entry (rho1 at most); the row before it, if it is
    // one of my workgroup's, is in progress at my first entry
    int r_first = rho0;
    if (T0 != tile_first) {
        if (rho0 >= base[0] && rho1 <= base[0] + 63) {
            const int idx = base[0] + lane;
            const unsigned long long m = __ballot(idx >= rho0 && (window[0] >= g0 || idx >= rho1));
            r_first = base[0] + (m ? __builtin_ctzll(m) : 63);
        } else {
            r_first = wave_lower_bound_in(a.row_ptr, lane, rho0, rho1, g0);
            __builtin_amdgcn_s_waitcnt(0x0f70);
        }
        r_first = uniform(r_first);
    }
    const int r_lim = rho1;  // the row start that ends my workgroup's last row
    int open_row = r_first > rho0 ? r_first - 1 : -1;  // -1: entries that are not my workgroup's
    {
        const int lowest = open_row >= 0 ? open_row : r_first;
        if (lowest < win_base || r_first > win_base + 63) reload_window(lowest);
    }
    const int s0 = open_row >= 0 ? row_start(open_row) : g0;
    int r_next = r_first;
    int b_next = row_start(r_next);

    // The row in progress at my first entry began at entry s0 < g0: the nibbles of its entries
    // [s0, g0) tell at which column it continues.  Deltas only, a fifth of the bytes of those
    // entries, and usually in L2 (the wave in front of me streams them).
    int look_sum = 0;
    const bool look_back = open_row >= 0 && s0 < g0 && T0 < T1;
    // nibble sum of the lane's 32 entries of the piece starting at entry `lo` that belong to the row
    auto look_chunk = [&](const u32x4 &dl, int lo, int acc) -> int {
        const int first = s0 - (lo + 32 * lane);  // how many of my 32 entries lie in front of the row start
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int nf = first - 8 * j;
            const u32 keep = nf <= 0 ? 0xffffffffu : (nf >= 8 ? 0u : 0xffffffffu << (4 * nf));
            acc = (int)__builtin_amdgcn_udot8(dl[j] & keep, 0x11111111u, (u32)acc, false);
        }
        return acc;
    };
    if (look_back) {
        const int covered = (int)a.look_entries;  // what the pieces requested ahead of time hold
        if (__builtin_expect(g0 - s0 > covered, 0)) {
            // The row began further back: those entries through ordinary loads, eight pieces in
            // flight together, more in a loop.  (The same lanes as above skip what they hold.)
            auto look_load = [&](int lo) -> u32x4 {
                const int mine = lo + 32 * lane;
                const bool want = mine + 32 > s0 && g0 - mine > covered;
                return __builtin_amdgcn_raw_buffer_load_b128(rs_deltas, want ? mine >> 1 : 0x7ffffff0, 0, 0);
            };
            u32x4 far[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) far[c] = look_load(g0 - (c + 1) * kLookBack);
#pragma unroll
            for (int c = 0; c < 8; ++c) look_sum = look_chunk(far[c], g0 - (c + 1) * kLookBack, look_sum);
            for (int hi = g0 - 8 * kLookBack; hi > s0; hi -= 2 * kLookBack) {
                const u32x4 d0 = look_load(hi - kLookBack);
                const u32x4 d1 = look_load(hi - 2 * kLookBack);
                look_sum = look_chunk(d0, hi - kLookBack, look_sum);
                look_sum = look_chunk(d1, hi - 2 * kLookBack, look_sum);
            }
            // nothing the compiler loaded here may still count as outstanding later on
            __builtin_amdgcn_s_waitcnt(0x0f70);
        }
    }
    // ---- 7. stream ----------------------------------------------------------------------------------
    float acc0 = 0.f, acc1 = 0.f;
    float accb[NB > 1 ? NB : 1] = {};  // batched variant: one accumulator per vector
    typedef __attribute__((address_space(3))) const uint16_t *lds_u16_ptr;
    typedef __attribute__((address_space(3))) const u32 *lds_u32_ptr;
    typedef __attribute__((address_space(3))) const u32x2 *lds_u32x2_ptr;
    typedef __attribute__((address_space(3))) const u32x4 *lds_u32x4_ptr;
    // LDS byte address of x[0] (x sits kLdsFront bytes, times NB, into this kernel's dynamic LDS)
    const u32 x_addr = (u32)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds + kLdsFront * NB;
    // row_addr: LDS byte address the next entry of the current row would read if its nibble were 0,
    // i.e. row_origin + 2 * (entries of the row consumed so far + their nibble sum).  Wave-uniform.
    // With NB > 1 it stays relative to x (row_origin = 0) and is scaled by NB when an entry is read.
    const u32 row_origin = NB == 1 ? x_addr : 0u;
    u32 row_addr = row_origin;
    __builtin_amdgcn_sched_barrier(0);
    if (look_back) {
        // pieces requested ahead of time; younger tracked loads: the later pieces and the ring
        look_sum = look_chunk(look_take<0, kTileLoads + 3>(), g0 - kLookBack, look_sum);
        if (g0 - kLookBack > s0 && a.look_entries > kLookBack) {
            look_sum = look_chunk(look_take<1, kTileLoads + 2>(), g0 - 2 * kLookBack, look_sum);
            if (g0 - 2 * kLookBack > s0 && a.look_entries > 2 * kLookBack) {
                look_sum = look_chunk(look_take<2, kTileLoads + 1>(), g0 - 3 * kLookBack, look_sum);
                look_sum = look_chunk(look_take<3, kTileLoads>(), g0 - 4 * kLookBack, look_sum);
            }
        }
        const int n = __builtin_amdgcn_readlane(wave_scan_inclusive(look_sum), kWave - 1);
        row_addr += 2u * (u32)(n + (g0 - s0));
    }
    // What is being summed.  `open_row` is the row the current entries belong to (-1: not one of my
    // workgroup's rows, summed and dropped).  `lead_open`: that row began in front of my first
    // entry, so its sum up to its end is a piece ("lead") that an earlier wave of the workgroup
    // collects.  `row_pend`: part of the current row's sum kept on the scalar side.
    bool lead_open = open_row >= 0;
    bool has_boundary = false;
    float lead_sum[NB] = {};
    float row_pend = 0.f;
    MACKO_STAMP(5);

    auto store_row = [&](int r, float total, int b = 0) {
        if (lane == 0) {
            float out = total;
            uint16_t *y = NB == 1 ? a.y : a.y + (size_t)b * (size_t)a.ldy;
            if (AXPBY) out = a.alpha * total + a.beta * half_bits_to_float(y[r]);
            y[r] = float_to_half_bits(out);
        }
    };
    // the current row ends with sum tot
    auto close_row = [&](const float (&tot)[NB]) {
        if (lead_open) {
#pragma unroll
            for (int b = 0; b < NB; ++b) lead_sum[b] = tot[b];
            lead_open = false;
        } else if (open_row >= 0) {
#pragma unroll
            for (int b = 0; b < NB; ++b) store_row(open_row, tot[b], b);
        }
        has_boundary = true;
    };
    // row r_next begins; the row start behind it becomes the next boundary
    auto open_next = [&]() {
        open_row = r_next < r_lim ? r_next : -1;
        ++r_next;
        if (r_next <= r_lim) {
            need_row(r_next);
            b_next = row_start(r_next);
        } else {
            b_next = kNone;
        }
    };
    auto wave_totals = [&](float (&tot)[NB]) {
        if (NB == 1) {
            tot[0] = wave_sum(acc0 + acc1) + row_pend;
        } else {
#pragma unroll
            for (int b = 0; b < NB; ++b) tot[b] = wave_sum(accb[b]);
        }
    };
    // a row start where no tile is being processed: the current row ends with what has been summed
    auto boundary_event = [&]() {
        float tot[NB];
        wave_totals(tot);
        close_row(tot);
        acc0 = acc1 = 0.f;
#pragma unroll
        for (int b = 0; b < NB; ++b) accb[b] = 0.f;
        row_pend = 0.f;
        row_addr = row_origin;
        open_next();
    };

    auto value_of = [&](const u32x4 &vv, int k) -> float {
        if (VB == 2) {
            const u32 w = vv[k >> 1];
            return half_bits_to_float((k & 1) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu));
        }
        return (float)((int)(vv[k >> 2] << (24 - 8 * (k & 3))) >> 24);  // sign-extended byte k
    };
    // x at LDS byte address `addr` + 2k (or the same element straight from memory)
    auto x_at = [&](u32 addr, int k) -> uint16_t {
        if (X_LDS) return *reinterpret_cast<lds_u16_ptr>((u32)(addr + 2 * k));  // ds_read_u16 with offset 2k
        int o = (int)(addr - x_addr) + 2 * k;
        const int omax = 2 * a.cols - 2;
        o = o < 0 ? 0 : (o > omax ? omax : o);
        return __builtin_amdgcn_raw_buffer_load_b16(rs_x, o, 0, 0);
    };

    // The eight multiply-adds of a lane: entry k reads x at base + 2k + 2 * (nibbles 0..k), which is
    // one v_dot8_u32_u4 with the multiplier 2 in the first k+1 nibble positions.  CHECKED: entries
    // outside [kmin, kmax) of the lane are not part of the row; their operand is replaced by zero.
    auto lane_fma = [&](const u32x4 &vv, u32 dd, u32 base, auto checked, int kmin, int kmax) {
        constexpr bool CHECKED = decltype(checked)::value != 0;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const u32 addr = __builtin_amdgcn_udot8(dd, twos_upto(k), base, false);
            if constexpr (NB > 1) {
                const float mv = value_of(vv, k);
                const u32 at = x_addr + (addr << kBatchShift) + ((2 * k) << kBatchShift);
                u32 xs[NB / 2 > 0 ? NB / 2 : 1];  // the NB operands, two per word
                if (NB == 2) {
                    xs[0] = *reinterpret_cast<lds_u32_ptr>(at);
                } else if (NB == 4) {
                    const u32x2 t = *reinterpret_cast<lds_u32x2_ptr>(at);
                    xs[0] = t.x;
                    xs[1 % (NB / 2)] = t.y;
                } else {
                    const u32x4 t = *reinterpret_cast<lds_u32x4_ptr>(at);
#pragma unroll
                    for (int q = 0; q < 4; ++q) xs[q % (NB / 2)] = t[q];
                }
                const bool valid = !CHECKED || (k >= kmin && k < kmax);
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    uint16_t h = (b & 1) ? (uint16_t)(xs[b >> 1] >> 16) : (uint16_t)(xs[b >> 1] & 0xffffu);
                    if (CHECKED) h = valid ? h : (uint16_t)0;
                    accb[b] = __builtin_fmaf(mv, half_bits_to_float(h), accb[b]);
                }
            } else {
                uint16_t xb = x_at(addr, k);
                if (CHECKED) xb = (k >= kmin && k < kmax) ? xb : (uint16_t)0;
                const float m = value_of(vv, k);
                if (k & 1)
                    acc1 = __builtin_fmaf(m, half_bits_to_float(xb), acc1);
                else
                    acc0 = __builtin_fmaf(m, half_bits_to_float(xb), acc0);
            }
        }
    };

    // A tile in which no row begins: every lane advances the row address by 16 bytes (its 8 entries)
    // plus twice its nibble sum; the DPP scan of that quantity gives every lane its starting address.
    auto full_tile_pass = [&](const u32x4 &vj, u32 dj) {
        const u32 step = __builtin_amdgcn_udot8(dj, 0x22222222u, 16u, false);
        const u32 incl = (u32)wave_scan_inclusive((int)step);
        const u32 base = (incl - step) + row_addr;
        row_addr += (u32)__builtin_amdgcn_readlane((int)incl, kWave - 1);
        lane_fma(vj, dj, base, index_constant<0>{}, 0, 8);
    };

    // Entries [pos, seg_end) of the tile starting at entry `tb`, all in the current row: lanes
    // outside the segment are switched off, the first and last lane of the segment are masked.
    // A row that starts `q0` entries into its first lane shifts every address by -2*q0.
    auto segment_pass = [&](const u32x4 &vj, u32 dj, int tb, int pos, int seg_end) {
        const int rel0 = pos - tb;
        const int rel1 = seg_end - tb;
        const int l0 = rel0 >> 3, q0 = rel0 & 7;
        const int l1 = (rel1 - 1) >> 3, q1 = rel1 & 7;
        u32x4 vv = vj;
        u32 dd = dj;
        const bool active = lane >= l0 && lane <= l1;
        if (q0 != 0 && lane == l0) mask_from<VB>(vv, dd, q0);
        if (q1 != 0 && lane == l1) mask_upto<VB>(vv, dd, q1);
        u32 step = __builtin_amdgcn_udot8(dd, 0x22222222u, 16u, false);
        step = active ? step : 0u;
        const u32 incl = (u32)wave_scan_inclusive((int)step);
        const u32 origin = row_addr - 2u * (u32)q0;
        const u32 base = (incl - step) + origin;
        row_addr = origin + (u32)__builtin_amdgcn_readlane((int)incl, kWave - 1);
        const int kmin = lane == l0 ? q0 : 0;
        const int kmax = (lane == l1 && q1 != 0) ? q1 : 8;
        if (active) lane_fma(vv, dd, base, index_constant<1>{}, kmin, kmax);
    };

    // Any tile, one pass per piece of a row (the way out for tiles the one-pass code below does not
    // take: two row starts inside one lane, batched products).
    auto pieces_tile = [&](const u32x4 &vj, u32 dj, int tb) {
        const int te = tb + kTile;
        int pos = tb;
        for (;;) {
            while (b_next == pos) boundary_event();
            const int seg_end = b_next < te ? b_next : te;
            if (open_row >= 0) segment_pass(vj, dj, tb, pos, seg_end);
            pos = seg_end;
            if (pos >= te) break;
        }
    };

    // A tile in which rows begin, in one pass (NB == 1).  Entries of the row in progress at the
    // tile's start read x from row_addr on, as in full_tile_pass; the entries of a row that starts
    // at tile entry b read from x_addr - (what the tile's entries in front of b advance).  Every
    // lane gets the origin of the row its first entry belongs to, and a lane in which a row begins
    // at entry q > 0 a second origin for its entries q..7.  Afterwards the per-lane sums are folded
    // row by row: whole lanes through a masked DPP sum, the two parts of a lane with a row start
    // through prefix sums (entries 0..q-1) and suffix sums (entries q..7) kept per entry.
    auto starts_tile = [&](const u32x4 &vj, u32 dj, int tb) {
        const int te = tb + kTile;
        const u32 step = __builtin_amdgcn_udot8(dj, 0x22222222u, 16u, false);
        const u32 incl = (u32)wave_scan_inclusive((int)step);
        const u32 excl = incl - step;
        // pass A: origins.  rb1: origin for a lane's entries in front of its row start (all eight if
        // it has none); rb2 / qlane: origin and first entry behind a row start inside the lane.
        u32 rb1 = row_addr, rb2 = 0u;
        int qlane = 8;
        u32 last_origin = row_addr;
        bool one_pass = true;
        {
            int r = r_next, b = b_next, prev_b = -1, prev_l = -1;
            while (b < te) {
                if (b != prev_b) {
                    const int rel = b - tb, L = rel >> 3, q = rel & 7;
                    if (L == prev_l) {  // a second row start in one lane
                        one_pass = false;
                        break;
                    }
                    u32 before = (u32)__builtin_amdgcn_readlane((int)excl, L);
                    if (q != 0) {
                        const u32 mq = ((1u << (4 * q)) - 1u) & 0x22222222u;
                        before += (u32)__builtin_amdgcn_readlane(
                            (int)__builtin_amdgcn_udot8(dj, mq, 2u * (u32)q, false), L);
                    }
                    const u32 origin = x_addr - before;
                    rb1 = lane >= L + (q != 0 ? 1 : 0) ? origin : rb1;
                    if (q != 0) {
                        rb2 = lane == L ? origin : rb2;
                        qlane = lane == L ? q : qlane;
                    }
                    last_origin = origin;
                    prev_l = L;
                    prev_b = b;
                }
                ++r;
                if (r > r_lim) break;
                if (r > win_base + 63) {  // more row starts in this tile than the window holds
                    one_pass = false;
                    break;
                }
                b = row_start(r);
            }
        }
        if (!one_pass) {
            pieces_tile(vj, dj, tb);
            return;
        }
        // pass B: the eight products of every lane, as running sums from the front (c) and from the
        // back (s)
        const u32 b1 = rb1 + excl, b2 = rb2 + excl;
        float xf[8], vf[8], c[8], s[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const u32 addr = __builtin_amdgcn_udot8(dj, twos_upto(k), k >= qlane ? b2 : b1, false);
            xf[k] = half_bits_to_float(x_at(addr, k));
            vf[k] = value_of(vj, k);
        }
        c[0] = vf[0] * xf[0];
#pragma unroll
        for (int k = 1; k < 8; ++k) c[k] = __builtin_fmaf(vf[k], xf[k], c[k - 1]);
        s[7] = vf[7] * xf[7];
#pragma unroll
        for (int k = 6; k >= 0; --k) s[k] = __builtin_fmaf(vf[k], xf[k], s[k + 1]);
        // pass C: fold
        float carry = acc0 + acc1;  // per lane: what earlier tiles added to the row in progress
        float pend = row_pend;
        int first_whole = 0;  // first lane all of whose entries belong to the current row
        int prev_b = -1;
        while (b_next < te) {
            const int b = b_next;
            float tot[NB] = {};
            if (b != prev_b) {
                const int rel = b - tb, L = rel >> 3, q = rel & 7;
                const float head = q != 0 ? pick_lane(c, q - 1, L) : 0.f;
                const float v = carry + ((lane >= first_whole && lane < L) ? c[7] : 0.f);
                tot[0] = wave_sum(v) + pend + head;
                carry = 0.f;
                pend = q != 0 ? pick_lane(s, q, L) : 0.f;
                first_whole = L + (q != 0 ? 1 : 0);
            }
            close_row(tot);
            prev_b = b;
            open_next();
        }
        acc0 = lane >= first_whole ? c[7] : 0.f;
        acc1 = 0.f;
        row_pend = pend;
        row_addr = last_origin + (u32)__builtin_amdgcn_readlane((int)incl, kWave - 1);
    };

    // The ring holds my first D tiles; now: take a slot, refill it, process.  Every step issues
    // exactly two loads (a "no tile" address once the range is exhausted), so a slot's loads are
    // always followed by those of the D - 1 other slots when it is awaited.  Only the take and the
    // refill exist once per slot; the code that processes a tile exists once.
    int slot_now = 0;
    for (u32 tile = T0; tile < T1; ++tile) {
        u32x4 vj;
        u32 dj;
        static_for<D>([&](auto slot) {
            constexpr int J = decltype(slot)::value;
            if (slot_now == J) {  // wave-uniform
                ring_take<D, J, kTileLoads - 2>(vj, dj);
                // refill at once: the copy is out
                issue_slot(slot, tile + D, tile + D < T1, !(last_wave && tile + D + 1 == T1));
            }
        });
        slot_now = slot_now + 1 == D ? 0 : slot_now + 1;
        const int tb = (int)(tile << kTileShift);
        while (b_next == tb) boundary_event();
        if (b_next >= tb + kTile)
            full_tile_pass(vj, dj);
        else if (NB == 1)
            starts_tile(vj, dj, tb);
        else
            pieces_tile(vj, dj, tb);
    }
    // row starts at the very end of the workgroup's range (its last row ends with its last tile, or
    // it has rows without entries there) are the last wave's
    if (last_wave)
        while (r_next <= r_lim) boundary_event();
    MACKO_STAMP(6);

    // ---- 8. the pieces of rows that span waves meet in LDS ------------------------------------------------
    // A wave whose share holds a row start publishes the sum in front of its first one (its "lead")
    // and keeps the sum behind its last one (its "tail", the beginning of row open_row); a wave
    // without a row start publishes its whole sum.  The tail's row ends in the first later wave
    // that has a row start, so the wave adds the leads up to that one and stores the row.
    {
        float tail[NB];
        wave_totals(tail);
        if (!has_boundary && lead_open) {
#pragma unroll
            for (int b = 0; b < NB; ++b) lead_sum[b] = tail[b];
        }
        const int tail_row = has_boundary ? open_row : -1;
        if (lane == 0) {
#pragma unroll
            for (int b = 0; b < NB; ++b) lead_lds[b * WAVES + wave] = lead_sum[b];
            flag_lds[wave] = has_boundary ? 1 : 0;
        }
        __syncthreads();
        if (tail_row >= 0) {
            const int fl = lane < n_active ? flag_lds[lane] : 1;
            const unsigned long long m = __ballot(lane > wave && fl != 0);
            const int stop = m ? __builtin_ctzll(m) : n_active;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const float v = (lane > wave && lane <= stop && lane < n_active) ? lead_lds[b * WAVES + lane] : 0.f;
                store_row(tail_row, tail[b] + wave_sum(v), b);
            }
        }
    }
    MACKO_STAMP(7);
}


template <int D, bool X_LDS, bool AXPBY, int VB, int NB, int XF>
int launch_split(SpmvArgs a, int grid, size_t lds_x, hipStream_t stream)
{
    constexpr int BLOCK = 1024;
    auto kernel = spmv_split_kernel<BLOCK, D, X_LDS, AXPBY, VB, NB, XF>;
    const u32 n_wg = (u32)grid;  // the owners of whole rows
    a.entries_q = (u32)(a.padded / n_wg);
    a.entries_rem = (u32)(a.padded % n_wg);
    a.rows_q = (u32)a.rows / n_wg;
    a.rows_frac = (u32)(((unsigned long long)((u32)a.rows % n_wg) << 32) / n_wg);
    a.row_even = (u32)a.rows <= n_wg ? 1u : 0u;
    a.active_shift = 4;
    {   // look-back hint from the mean row length (entries per row, a quarter more)
        const long long mean = a.padded / (a.rows > 0 ? a.rows : 1);
        const long long want = mean + mean / 4;
        a.look_entries = want <= kTile ? (u32)kTile : (u32)(want <= kLookBack ? 1 : want <= 2 * kLookBack ? 2 : 4) * kLookBack;
    }
    // behind x: one piece of a row sum per wave and vector, and one flag per wave
    const size_t lds_bytes = ((lds_x + 3) & ~(size_t)3) + (size_t)(BLOCK / kWave) * 4 * (NB + 1);
    if (lds_bytes > 64 * 1024) {
        // one-time opt-in to more than 64 KiB of dynamic LDS, per device and kernel
        static std::atomic<bool> done[64];
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return (int)e;
        if (dev < 0 || dev >= 64 || !done[dev].load(std::memory_order_acquire)) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            if (dev >= 0 && dev < 64) done[dev].store(true, std::memory_order_release);
        }
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(BLOCK), lds_bytes, stream, a);
    return (int)hipGetLastError();
}

}  // namespace

int spmv_split_launch(const spmv_detail::SpmvArgs &a, bool axpby, int value_bytes, int n_vectors, int fused,
                      bool x_in_lds, int grid, size_t lds_x, hipStream_t stream)
{
    if (fused == 1 && !axpby && x_in_lds) return launch_split<2, true, false, 2, 1, 1>(a, grid, lds_x, stream);
    if (fused == 2 && x_in_lds) {
        if (axpby) return launch_split<2, true, true, 2, 1, 2>(a, grid, lds_x, stream);
        return launch_split<2, true, false, 2, 1, 2>(a, grid, lds_x, stream);
    }
    if (fused != 0) return MACKO_E_INVALID_ARGUMENT;
    if (n_vectors > 1) {
        if (axpby || value_bytes != 2 || !x_in_lds) return MACKO_E_INVALID_ARGUMENT;
        if (n_vectors == 8) return launch_split<2, true, false, 2, 8, 0>(a, grid, lds_x, stream);
        if (n_vectors == 4) return launch_split<2, true, false, 2, 4, 0>(a, grid, lds_x, stream);
        if (n_vectors == 2) return launch_split<2, true, false, 2, 2, 0>(a, grid, lds_x, stream);
        return MACKO_E_INVALID_ARGUMENT;
    }
    if (value_bytes == 1) {
        if (!x_in_lds) return axpby ? launch_split<2, false, true, 1, 1, 0>(a, grid, 0, stream)
                                    : launch_split<2, false, false, 1, 1, 0>(a, grid, 0, stream);
        return axpby ? launch_split<2, true, true, 1, 1, 0>(a, grid, lds_x, stream)
                     : launch_split<2, true, false, 1, 1, 0>(a, grid, lds_x, stream);
    }
    if (!x_in_lds) return axpby ? launch_split<2, false, true, 2, 1, 0>(a, grid, 0, stream)
                                : launch_split<2, false, false, 2, 1, 0>(a, grid, 0, stream);
    return axpby ? launch_split<2, true, true, 2, 1, 0>(a, grid, lds_x, stream)
                 : launch_split<2, true, false, 2, 1, 0>(a, grid, lds_x, stream);
}

}  // namespace macko
