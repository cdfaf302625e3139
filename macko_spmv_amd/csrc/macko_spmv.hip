// MACKO fp16 sparse matrix-vector product for gfx950 (wave64).
//
// Row ownership.  The value and delta arrays are cut into fixed tiles of 512 entries (one
// 128-bit value load and one 32-bit delta load per lane).  The launch has W waves; wave w owns
// the rows whose first entry index lies inside the tile range [w*NT/W, (w+1)*NT/W): contiguous
// whole rows, balanced by stored entries.  It finds them with a 64-wide probe of row_ptr placed
// by an arithmetic guess (one memory round trip when rows carry similar entry counts, 64-ary
// search rounds otherwise).  No row is shared between waves, so there is no cross-wave
// reduction, no atomics and no scratch memory.
//
// Data movement.  While the probe is in flight the workgroup copies x into LDS.  Each wave then
// streams the tiles that hold its rows through a ring of D register slots (hand-tracked loads,
// see below): take a slot, refill it with the tile D ahead, process.
//
// Per tile, the entries of one row form a segment [first lane/entry, last lane/entry]; each
// segment takes one pass: mask, DPP prefix sum of per-lane nibble sums, v_dot8_u32_u4 for the
// running sum inside a lane, gather of x from LDS, fp32 FMA.  A row ends with one DPP
// reduction and an fp16 store.
//
// Behaviour restated from src/macko_spmv/cuda/kernels.cuh:34-124 of the upstream package.

#include <atomic>

#include "macko_spmv_tracked.h"

namespace macko {
namespace {

using namespace spmv_detail;

// The hand-tracked loads (macko_spmv_tracked.h) with this kernel's register map: the compiler keeps
// below v78; v78,v79 row_ptr probes; v80..v87 two 16-byte pieces of x; v88.. the ring (up to four
// slots: v88..v103 values, v104..v107 delta words at depth 4).
constexpr int kCompilerVgprs = 78;
#define MACKO_STREAM_FIXED_REGISTERS "v78", "v79", "v80", "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107"
typedef TrackedLoads<kCompilerVgprs> Tracked;
template <int K> __device__ __forceinline__ void probe_issue(u32 o, const u32x4 &b) { Tracked::probe_issue<K>(o, b); }
template <int K, int N> __device__ __forceinline__ int probe_take() { return Tracked::probe_take<K, N>(); }
template <int J> __device__ __forceinline__ void xpiece_issue(u32 o, const u32x4 &b) { Tracked::xpiece_issue<J>(o, b); }
template <int J, int N> __device__ __forceinline__ void xpiece_to_lds(u32 a) { Tracked::xpiece_to_lds<J, N>(a); }
template <int D, int J, int VB>
__device__ __forceinline__ void ring_issue(u32 vo, u32 dof, const u32x4 &bv, const u32x4 &bd, bool stream)
{
    static_assert(D == 1 || D == 2 || (D == 4 && VB == 2), "ring depth");
    Tracked::ring_issue<D, J, VB>(vo, dof, bv, bd, stream);
}
template <int D, int J, int N> __device__ __forceinline__ void ring_take(u32x4 &v, u32 &d) { Tracked::ring_take<D, J, N>(v, d); }

// NB = vectors multiplied per launch (1, 2, 4 or 8).  With NB > 1 the NB copies of x are interleaved in
// LDS (element c of vector b at half-word c * NB + b), so one LDS read per stored entry fetches the
// operand of every vector, and a row ends with NB sums.  NB > 1 exists for fp16 values, x in LDS,
// plain product only.
// XF = function applied to the input while it is staged into LDS, so the producer of x needs no
// launch of its own: 0 = none (x as given), 1 = RMS norm (x * rsqrt(mean(x^2) + eps) * x2, x2 the
// norm weight), 2 = SiLU gate (silu(x) * x2).  The staged vector is rounded to fp16 exactly as a
// separate kernel writing it to memory would.  XF != 0 needs cols % 8 == 0 and 16-byte aligned x, x2.
// ROWS = with the pass that works all the rows of a tile at once (rows_pass below), for matrices of
// short rows.  A variant of its own: compiled into the kernel, that pass costs the row loop of
// every matrix 0.3 to 0.7 us per launch (measured on 4096 x 4096 and 11008 x 4096 at density 0.1),
// used or not.
// PLAN = every wave reads where its rows start from a table the caller had built for this matrix
// (a.plan, see macko_spmv_plan_build) instead of searching row_ptr for its cuts: the search costs
// nothing where the rows are about equally long (its first probe hits), and one or two more round
// trips to memory for whole workgroups where they are not.
template <int BLOCK, int D, bool X_LDS, bool AXPBY, int VB, int NB, int XF, bool ROWS, bool PLAN>
__global__ void __launch_bounds__(BLOCK) __attribute__((amdgpu_num_vgpr(kCompilerVgprs)))
spmv_stream_kernel(const SpmvArgs a)
{
    static_assert(NB == 1 || (NB <= 8 && X_LDS && !AXPBY && VB == 2), "batched variant: fp16, x in LDS, plain product");
    static_assert(XF == 0 || (NB == 1 && X_LDS && VB == 2), "fused staging: fp16, one vector, x in LDS");
    static_assert(!ROWS || (X_LDS && NB == 1 && XF == 0), "all rows of a tile in one pass: one vector, x in LDS");
    static_assert(!PLAN || (X_LDS && NB == 1 && XF == 0), "prepared cuts: one vector, x in LDS");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    MACKO_RESERVE_FIXED_REGISTERS(MACKO_STREAM_FIXED_REGISTERS);
    constexpr int WAVES = BLOCK / kWave;
    constexpr int kBatchShift = NB == 8 ? 3 : (NB == 4 ? 2 : (NB == 2 ? 1 : 0));
    constexpr int kTileLoads = 2 * D;  // tracked loads per full ring
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = uniform(tid >> 6);
    const u32 n_waves = gridDim.x * WAVES;
    // Workgroups are dealt round-robin to the 8 XCDs (workgroup i runs on XCD i % 8).  Giving XCD k
    // the k-th contiguous eighth of the matrix keeps neighbouring workgroups, which share boundary
    // tiles, behind one L2.
    u32 wg = blockIdx.x;
    if ((gridDim.x & 7) == 0) wg = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const u32 gw = wg * WAVES + wave;
#ifdef MACKO_DEV_HOOKS
    const u32 stamp_wave = gw;
#endif
    MACKO_STAMP(0);


    const u32x4 buf_values = make_buffer(a.values, (u32)(a.padded * VB));
    const u32x4 buf_deltas = make_buffer(a.deltas, (u32)(a.padded / 2));
    const u32x4 buf_rows = make_buffer(a.row_ptr, ((u32)a.rows + 1) * 4);
    const __amdgpu_buffer_rsrc_t rs_x =
        __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.cols * 2, 0x00020000);
    (void)rs_x;
    const u32 lane_values = (u32)lane * (kChunk * VB), lane4 = (u32)lane * 4;

    const bool x_vec = (reinterpret_cast<uintptr_t>(a.x) & 15) == 0;
    const int x_nvec = x_vec ? a.cols >> 3 : 0;

    // ---- 1. tracked loads, oldest first: row_ptr probes, x pieces ------------------------------------
    // probes: 64 consecutive row_ptr values around where my first / last row should be
    int target[2], base[2], guess[2];
    int cut_row[2] = {0, 0}, cut_entry[2] = {0, 0};
    if constexpr (PLAN) {
        // {first row, its first entry} of wave gw and of wave gw + 1: one scalar load
        const int4 cut = *reinterpret_cast<const int4 *>(a.plan + 2 * (size_t)gw);
        cut_row[0] = cut.x;
        cut_entry[0] = cut.y;
        cut_row[1] = cut.z;
        cut_entry[1] = cut.w;
        target[0] = target[1] = guess[0] = guess[1] = base[1] = 0;
    } else {
        target[0] = (int)even_split(gw, a.entries_q, a.entries_rem);  // < P < 2^31
        target[1] = (int)even_split(gw + 1, a.entries_q, a.entries_rem);
        guess[0] = (int)(gw * a.rows_q + __umulhi(gw, a.rows_frac));
        guess[1] = gw == n_waves - 1 ? a.rows : (int)((gw + 1) * a.rows_q + __umulhi(gw + 1, a.rows_frac));
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
    if constexpr (PLAN) {  // the window of row starts from my first row on, behind the x pieces
        base[0] = (int)((u32)cut_row[0] < (u32)a.rows ? (u32)cut_row[0] : (u32)a.rows);
        int i0 = base[0] + lane;
        i0 = i0 <= a.rows ? i0 : a.rows;
        probe_issue<0>((u32)i0 * 4, buf_rows);
    }
    // Tile t of mine holds entries [tile_origin + 512 t, tile_origin + 512 (t + 1)).  My tiles are
    // counted from my own first entry, not on a grid of the whole array's: there nearly every wave
    // would start in the middle of a tile and have one more tile to load and one more pass to make
    // for the same entries.  Where a wave has few tiles (D == 1) the origin is rounded down to a
    // lane's 8 entries only (rows of 500 entries, one to three per wave: 5 % per launch).  Long
    // streams (D == 2) round it down to 256 entries, so that every load still starts on a cache
    // line (128 bytes of nibbles): loads that do not cost them more than the tile they save (3 to
    // 7 % per launch at density 0.5 with an origin rounded to 8; 1 to 3 % gained with 256).
    constexpr u32 kOriginAlign = D == 1 ? kChunk : 256;
    u32 tile_origin = 0;
    auto issue_slot = [&](auto slot, u32 tile, bool fetch, bool stream) {
        constexpr int J = decltype(slot)::value;
        const u32 first = tile_origin + (tile << kTileShift);
        ring_issue<D, J, VB>(lane_values + (fetch ? first * (u32)VB : kNoTileValues),
                         lane4 + (fetch ? first >> 1 : kNoTileDeltas), buf_values, buf_deltas, stream);
    };
    // ---- 2. x: everything beyond the two register pieces per thread, and unaligned or odd-length
    //         x, goes to LDS through ordinary loads (rare: more than 16384 columns, or an x that is
    //         not 16-byte aligned) ------------------------------------------------------------------
    stage_x_untracked<BLOCK, X_LDS, NB, XF>(lds, a, tid, lane, wave, x_vec, x_nvec);
    MACKO_STAMP(1);

    // ---- 3. which rows are mine -----------------------------------------------------------------------
    constexpr int kXLoads = X_LDS && NB == 1 && XF == 0 ? kXRegs : 0;
    int window[2] = {0, 0};
    if constexpr (!PLAN) {
        window[0] = probe_take<0, kXLoads + 1>();
        window[1] = probe_take<1, kXLoads>();
    }
    // window of row_ptr values the row loop reads row starts from: lane i holds row_ptr[win_base + i]
    int win_base = base[0];
    int win = window[0];
    auto row_start = [&](int r) -> int {  // r in [win_base, win_base + 63]
        return __builtin_amdgcn_readlane(win, r - win_base);
    };
    auto slide_window = [&](int r) {  // make rows r and r + 1 addressable
        if (__builtin_expect(r < win_base || r + 1 > win_base + 63, 0)) {
            win_base = r;
            win = load_row_window(a.row_ptr, a.rows, win_base, lane);
            // Awaited on the spot: a load the compiler still counts as outstanding at the loop's
            // back edge makes it protect the register with a vmcnt(0) at the top of every
            // iteration, which would also wait for the ring loads just issued.
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), expcnt and lgkmcnt untouched
        }
    };
    auto store_row = [&](int r, float total, int b = 0) {
        if (lane == 0) {
            float out = total;
            uint16_t *y = NB == 1 ? a.y : a.y + (size_t)b * (size_t)a.ldy;
            if (AXPBY) out = a.alpha * total + a.beta * half_bits_to_float(y[r]);
            y[r] = float_to_half_bits(out);
        }
    };
    auto store_empty_row = [&](int r) {
#pragma unroll
        for (int b = 0; b < NB; ++b) store_row(r, 0.f, b);
    };

    int row_last = 0;
    bool have_work = false;
    int r = 0;  // current row
    int e0 = 0, e1 = 0, s_end = 0;
    bool resolved = false;
    constexpr u32 first_tile = 0;
    u32 last_tile = 0;
    auto fill_ring = [&]() __attribute__((always_inline)) {
        tile_origin = (u32)e0 & ~(kOriginAlign - 1);
        // (exclusive; none if my rows end in front of where they start, and none beyond the arrays:
        // a row_ptr that runs backwards or points outside cannot make the walk longer than the matrix)
        const int end = s_end < (int)a.padded ? s_end : (int)a.padded;
        last_tile = end > e0 ? ((u32)end - tile_origin + kTile - 1) >> kTileShift : 0u;
        static_for<D>([&](auto slot) {
            constexpr int J = decltype(slot)::value;
            // my first and last tile may be shared with a neighbouring wave: no streaming hint there
            issue_slot(slot, first_tile + J, first_tile + J < last_tile, J > 0 && first_tile + J + 1 < last_tile);
        });
    };
    if constexpr (PLAN) {
        // (clamped, so that a plan that does not belong to this matrix can make the result wrong
        // but no access leave the arrays and no loop run longer than the matrix is)
        // (unsigned minimum: a negative value counts as too large)
        auto at_most = [](int v, int most) { return (int)((u32)v < (u32)most ? (u32)v : (u32)most); };
        r = at_most(uniform(cut_row[0]), a.rows);
        row_last = at_most(uniform(cut_row[1]), a.rows);
        row_last = row_last < r ? r : row_last;
        e0 = at_most(uniform(cut_entry[0]), (int)a.padded);
        s_end = at_most(uniform(cut_entry[1]), (int)a.padded);
        s_end = s_end < e0 ? e0 : s_end;
        have_work = r < row_last && e0 < s_end;
        // nothing else stands between a wave and its tiles; the window of row starts is taken behind
        // the barrier (it was requested last, and x must not wait for it)
        if (__builtin_expect(have_work, 1)) fill_ring();
        resolved = true;
    }
    if constexpr (!PLAN) {
        // Straight-line case: both cuts fall inside their probe windows and my first row is not
        // empty.  Cut k is the first row start at or after target k, or the one before it if that
        // is nearer (with rows of similar length every wave then gets the same number of rows).
        // (cuts are taken on row_ptr[r] + row_cost * r: see SpmvArgs::row_cost)
        const int row_cost = (int)a.row_cost;
        const unsigned long long m0 = __ballot(window[0] + row_cost * (base[0] + lane) >= target[0]);
        const unsigned long long m1 = __ballot(window[1] + row_cost * (base[1] + lane) >= target[1]);
        const int f0 = m0 ? __builtin_ctzll(m0) : 0;
        const int f1 = m1 ? __builtin_ctzll(m1) : 0;
        if (a.row_even) {  // the cuts are the guesses themselves; both lie inside their windows
            r = guess[0];
            row_last = guess[1];
            have_work = r < row_last;
            if (have_work) {  // then r <= rows - 1 and r + 1 - base[0] <= 63
                e0 = __builtin_amdgcn_readlane(window[0], r - base[0]);
                e1 = __builtin_amdgcn_readlane(window[0], r + 1 - base[0]);
                s_end = __builtin_amdgcn_readlane(window[1], row_last - base[1]);
            }
            resolved = have_work && e1 != e0;
        } else if (__builtin_expect(f0 >= 1 && f0 <= 62 && f1 >= 1 && gw != n_waves - 1, 1)) {
            const int at0 = __builtin_amdgcn_readlane(window[0], f0);
            const int before0 = __builtin_amdgcn_readlane(window[0], f0 - 1);
            const int at1 = __builtin_amdgcn_readlane(window[1], f1);
            const int before1 = __builtin_amdgcn_readlane(window[1], f1 - 1);
            const int weight0 = row_cost * (base[0] + f0), weight1 = row_cost * (base[1] + f1);
            const int back0 = target[0] - (before0 + weight0 - row_cost) < at0 + weight0 - target[0] ? 1 : 0;
            const int back1 = target[1] - (before1 + weight1 - row_cost) < at1 + weight1 - target[1] ? 1 : 0;
            r = base[0] + f0 - back0;
            row_last = base[1] + f1 - back1;
            e0 = back0 ? before0 : at0;
            e1 = __builtin_amdgcn_readlane(window[0], f0 - back0 + 1);
            s_end = back1 ? before1 : at1;
            have_work = r < row_last;
            resolved = have_work && e1 != e0;
        }
    }
    MACKO_STAMP(2);
    if (__builtin_expect(!resolved, 0)) {
        // General case: search rounds where a window missed, first / last wave, leading empty rows.
        int range[2] = {guess[0], guess[1]};
        const int row_cost = (int)a.row_cost;
        if (!a.row_even) wave_lower_bound2(a.row_ptr, a.rows, lane, target, window, base, range, row_cost);
#pragma unroll
        for (int k = 0; k < 2 && !a.row_even; ++k) {
            const int rr = range[k];
            if (rr > 0 && rr <= a.rows) {
                int after, before;
                if (rr - 1 >= base[k] && rr <= base[k] + 63) {
                    after = __builtin_amdgcn_readlane(window[k], rr - base[k]);
                    before = __builtin_amdgcn_readlane(window[k], rr - 1 - base[k]);
                } else {
                    after = uniform(a.row_ptr[rr]);
                    before = uniform(a.row_ptr[rr - 1]);
                }
                if (target[k] - (before + row_cost * (rr - 1)) < after + row_cost * rr - target[k]) range[k] = rr - 1;
            }
        }
        if (gw == 0) range[0] = 0;
        if (gw == n_waves - 1) range[1] = a.rows;
        r = uniform(range[0]);
        row_last = uniform(range[1]);
        have_work = r < row_last;
        win_base = base[0];  // the search may have moved the windows
        win = window[0];
        if (have_work) {  // first non-empty owned row; empty ones are written on the way
            slide_window(r);
            e0 = row_start(r);
            e1 = row_start(r + 1);
            while (e1 == e0) {
                store_empty_row(r);
                ++r;
                if (r >= row_last) {
                    have_work = false;
                    break;
                }
                slide_window(r);
                e0 = row_start(r);
                e1 = row_start(r + 1);
            }
        }
        if (have_work) {  // end of my last owned row
            if (row_last >= base[1] && row_last <= base[1] + 63)
                s_end = __builtin_amdgcn_readlane(window[1], row_last - base[1]);
            else
                s_end = row_last >= win_base && row_last <= win_base + 63 ? row_start(row_last)
                                                                            : uniform(a.row_ptr[row_last]);
        }
        // nothing the compiler loaded on this path may still count as outstanding when the tile
        // loop is entered (see slide_window)
        __builtin_amdgcn_s_waitcnt(0x0f70);
    }

    // ---- 4. my tile range; the ring is filled with my first D tiles before x is even in LDS: they
    //         fly while the workgroup finishes the copy and meets at the barrier -------------------------
    if constexpr (!PLAN) {
        if (__builtin_expect(have_work, 1)) fill_ring();
    }

    // ---- 5. x pieces into LDS (older than the ring loads just issued, if any) ---------------------------
    if (NB > 1 || XF != 0) {
        __syncthreads();
    } else if (X_LDS) {
        const u32 lds_x = (u32)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds + kLdsFront;
        const u32 dst0 = lds_x + (u32)tid * 16, dst1 = dst0 + BLOCK * 16;
        // (with PLAN the window's load stands between the x pieces and the ring)
        constexpr int kBehindX = PLAN ? 1 : 0;
        if (__builtin_expect(have_work, 1)) {
            if (tid < x_nvec) xpiece_to_lds<0, kTileLoads + kBehindX + 1>(dst0);
            if (tid + BLOCK < x_nvec) xpiece_to_lds<1, kTileLoads + kBehindX>(dst1);
        } else {
            if (tid < x_nvec) xpiece_to_lds<0, kBehindX + 1>(dst0);
            if (tid + BLOCK < x_nvec) xpiece_to_lds<1, kBehindX>(dst1);
        }
        // the copies above are asm the compiler's wait tracking does not see
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        MACKO_STAMP(3);
        __syncthreads();
    }
    MACKO_STAMP(4);
    if constexpr (PLAN) {
        if (__builtin_expect(have_work, 1)) {
            win = probe_take<0, kTileLoads>();
            e1 = row_start(r + 1);
            while (e1 == e0 && r + 1 < row_last) {  // first non-empty row; empty ones are written on the way
                store_empty_row(r);
                ++r;
                slide_window(r);
                e1 = row_start(r + 1);
            }
        } else {
            win = probe_take<0, 0>();
            // rows without a single entry: a zero each
            for (int rr = r + lane; rr < row_last; rr += kWave) {
                float out = 0.f;
                if (AXPBY) out = a.beta * half_bits_to_float(a.y[rr]);
                a.y[rr] = float_to_half_bits(out);
            }
        }
    }

    if (__builtin_expect(!have_work, 0)) return;

    // ---- 6. stream ----------------------------------------------------------------------------------
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
    MACKO_STAMP(5);

    // The eight multiply-adds of a lane: entry k reads x at base + 2k + 2 * (nibbles 0..k), which is
    // one v_dot8_u32_u4 with the multiplier 2 in the first k+1 nibble positions.  CHECKED (a piece
    // of a row that ends inside the lane): entries kmax..7 of the lane are not part of the row;
    // their value is masked to zero, but what they would read lies behind the row's last column
    // and may be Inf or NaN, so they read the zero bytes in front of x instead.  (Entries in front
    // of kmin, masked at a row's start, read those zero bytes by construction when x is in LDS.)
    auto lane_fma = [&](const u32x4 &vv, u32 dd, u32 base, auto checked, int kmin, int kmax) __attribute__((always_inline)) {
        constexpr bool CHECKED = decltype(checked)::value != 0;
        const u32 zeros = row_origin - 16u;  // 16 zero bytes (times NB) in front of x
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            u32 addr = __builtin_amdgcn_udot8(dd, twos_upto(k), base, false);
            if constexpr (NB > 1) {
                if (CHECKED) addr = k < kmax ? addr : zeros;
                const u32 w = vv[k >> 1];
                const float mv = half_bits_to_float((k & 1) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu));
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
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    const uint16_t h = (b & 1) ? (uint16_t)(xs[b >> 1] >> 16) : (uint16_t)(xs[b >> 1] & 0xffffu);
                    accb[b] = __builtin_fmaf(mv, half_bits_to_float(h), accb[b]);
                }
            } else {
                uint16_t xb;
                if (X_LDS) {
                    if (CHECKED) addr = k < kmax ? addr : zeros;
                    xb = *reinterpret_cast<lds_u16_ptr>((u32)(addr + 2 * k));  // ds_read_u16 with offset 2k
                } else {
                    int o = (int)(addr - x_addr) + 2 * k;
                    const int omax = 2 * a.cols - 2;
                    o = o < 0 ? 0 : (o > omax ? omax : o);
                    if (CHECKED) o = (k >= kmin && k < kmax) ? o : 0x7ffffff0;  // past the end: reads as zero
                    xb = __builtin_amdgcn_raw_buffer_load_b16(rs_x, o, 0, 0);
                }
                float m;
                if (VB == 2) {
                    const u32 w = vv[k >> 1];
                    m = half_bits_to_float((k & 1) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu));
                } else {
                    m = (float)((int)(vv[k >> 2] << (24 - 8 * (k & 3))) >> 24);  // sign-extended byte k
                }
                if (k & 1)
                    acc1 = __builtin_fmaf(m, half_bits_to_float(xb), acc1);
                else
                    acc0 = __builtin_fmaf(m, half_bits_to_float(xb), acc0);
            }
        }
    };

    // A tile that lies wholly inside the current row: no masks, every lane active.  Each lane
    // advances the row address by 16 bytes (its 8 entries) plus twice its nibble sum; the DPP scan
    // of that quantity gives every lane its starting address.
    auto full_tile_pass = [&](const u32x4 &vj, u32 dj) __attribute__((always_inline)) {
        const u32 step = __builtin_amdgcn_udot8(dj, 0x22222222u, 16u, false);
        const u32 incl = (u32)wave_scan_inclusive((int)step);
        const u32 base = (incl - step) + row_addr;
        row_addr += (u32)__builtin_amdgcn_readlane((int)incl, kWave - 1);
        lane_fma(vj, dj, base, index_constant<0>{}, 0, 8);
    };

    // Entries [pos, seg_end) of the tile starting at entry `tb`, all in the current row: lanes
    // outside the segment are switched off, the first and last lane of the segment are masked.
    // A row that starts `q0` entries into its first lane shifts every address by -2*q0.
    auto segment_pass = [&](const u32x4 &vj, u32 dj, int tb, int pos, int seg_end, auto checked) __attribute__((always_inline)) {
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
        if (active) lane_fma(vv, dd, base, checked, kmin, kmax);
    };

    auto finish_row = [&](float total) __attribute__((always_inline)) {  // total: the row's sum where there is one vector
        if (NB == 1) {
            store_row(r, total);
            acc0 = acc1 = 0.f;
        } else {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                store_row(r, wave_sum(accb[b]), b);
                accb[b] = 0.f;
            }
        }
        row_addr = row_origin;
        do {  // next non-empty owned row; empty ones get their zero on the way
            ++r;
            if (r >= row_last) {
                // The row just finished ended at s_end and all loops end.  With a row_ptr that runs
                // backwards, or cuts that are not this matrix's, entries may seem to be left: no
                // row claims them (every later step then sees a row that starts at infinity, which
                // writes nothing and moves on), so the walk ends whatever the arrays hold.
                e0 = e1 = 0x7fffffff;
                last_tile = 0;
                break;
            }
            slide_window(r);
            e0 = row_start(r);
            e1 = row_start(r + 1);
            if (e1 == e0) store_empty_row(r);
        } while (e1 == e0);
    };

    // Entries [pos, stop) of the tile starting at entry `tb`, over all the rows they belong to at
    // once: for tiles in which several rows end, where a pass per row (segment_pass) would cost a
    // scan, eight multiply-adds, a reduction and a store per row, however short.  Here the column
    // addresses and the sums are segmented prefix scans that restart where a row starts:
    //   1. the rows of the window mark their first entry in a per-lane bit mask (through LDS);
    //   2. every lane walks its 8 entries from the address the scan hands it, back to x[0] at a mark;
    //   3. the products are summed the same way; every entry's running row sum goes to LDS;
    //   4. the window's lanes, one per row, fetch the sum at their row's last entry and store y.
    // `stop` is the tile's end, the end of my rows, or the start of the window's last row,
    // whichever comes first; the current row r may have begun in an earlier tile (its partial sums
    // are in acc0 / acc1, its address in row_addr).  Leaves r, e0, e1, acc0, acc1, row_addr as the
    // row loop expects them at entry `stop`.  No entry is masked: every entry in [pos, stop) is
    // read at its own column, and what lies outside never reaches a stored sum.
    auto rows_pass = [&](const u32x4 &vj, u32 dj, int tb, int pos, int stop) __attribute__((always_inline)) {
        typedef __attribute__((address_space(3))) u32 *lds_w32;
        typedef __attribute__((address_space(3))) float *lds_f32;
        typedef __attribute__((address_space(3))) u32x4 *lds_w32x4;
        auto bits = [](float f) { return __builtin_bit_cast(u32, f); };
        const u32 area = (u32)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds + a.rows_pass_lds +
                         (u32)wave * (kTile * 4);
        const int rw_end = row_last < win_base + 63 ? row_last : win_base + 63;  // last row whose start I know
        const int row_j = win_base + lane;
        const int e_j = win;
        const int e_next = wave_from_lane_above(win);
        const bool continuing = e0 < tb;
        const float carry_sum = continuing ? wave_sum(acc0 + acc1) : 0.f;
        const u32 carry_addr = row_addr - row_origin;

        // 1. marks
        *(lds_w32)(uintptr_t)(area + lane4) = 0u;
        __builtin_amdgcn_wave_barrier();
        if (row_j >= r && row_j <= rw_end && e_j >= pos && e_j > tb && e_j <= stop && e_j < tb + kTile) {
            const u32 rel = (u32)(e_j - tb);
            __hip_atomic_fetch_or((lds_w32)(uintptr_t)(area + (rel >> 3) * 4), 1u << (rel & 7), __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_WAVEFRONT);
        }
        __builtin_amdgcn_wave_barrier();
        const u32 marks = *(lds_w32)(uintptr_t)(area + lane4);
        const bool marked = marks != 0;
        const SegmentMasks seg = segment_masks(__ballot(marked));

        // 2. addresses: what a lane passes on is its walk from its last mark (all 8 entries if none)
        const int last_mark = marked ? 31 - __builtin_clz(marks) : 0;
        u32 walk = __builtin_amdgcn_udot8(dj & (~0u << (4 * last_mark)), 0x22222222u, 2u * (u32)(8 - last_mark), false);
        if (lane == 0 && !marked) walk += carry_addr;
        const u32 walk_incl = wave_segmented_scan<u32>(walk, seg);
        u32 run = (u32)wave_from_lane_below((int)walk_incl);
        if (lane == 0) run = carry_addr;
        run += row_origin;
        const int rel0 = pos - tb, rel1 = stop - tb;
        const bool active = lane >= (rel0 >> 3) && lane <= ((rel1 - 1) >> 3);

        // 3. products and running row sums
        float t[8];
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const bool mark = (marks >> k) & 1u;
            run = mark ? row_origin : run;
            const u32 addr = run + 2u * ((dj >> (4 * k)) & 15u);
            run = addr + 2u;
            uint16_t xb = 0;
            if (active) xb = *(lds_u16_ptr)(uintptr_t)addr;
            float m;
            if (VB == 2) {
                const u32 w = vj[k >> 1];
                m = half_bits_to_float((k & 1) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu));
            } else {
                m = (float)((int)(vj[k >> 2] << (24 - 8 * (k & 3))) >> 24);
            }
            sum = mark ? 0.f : sum;
            sum = __builtin_fmaf(m, half_bits_to_float(xb), sum);
            t[k] = sum;
        }
        const float sum_incl = wave_segmented_scan<float>(sum, seg);
        const float before = __builtin_bit_cast(float, wave_from_lane_below(__builtin_bit_cast(int, sum_incl)));
        *(lds_w32x4)(uintptr_t)(area + (u32)lane * 32) = u32x4{bits(t[0]), bits(t[1]), bits(t[2]), bits(t[3])};
        *(lds_w32x4)(uintptr_t)(area + (u32)lane * 32 + 16) = u32x4{bits(t[4]), bits(t[5]), bits(t[6]), bits(t[7])};
        __builtin_amdgcn_wave_barrier();
        // the entries in front of a lane's first mark continue the row of the lanes before: only the
        // last of them can end a row, so only its sum needs what those lanes add
        if ((marks & 1u) == 0) {
            const int fix = marked ? __builtin_ctz(marks) - 1 : 7;
            __hip_atomic_fetch_add((lds_f32)(uintptr_t)(area + (u32)lane * 32 + (u32)fix * 4), before, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WAVEFRONT);
        }
        __builtin_amdgcn_wave_barrier();

        // 4. one lane per row that ends in [pos, stop]
        if (row_j >= r && row_j < rw_end && e_next <= stop) {
            float total = 0.f;
            if (e_next != e_j) {
                total = *(lds_f32)(uintptr_t)(area + (u32)(e_next - 1 - tb) * 4);
                if (row_j == r) total += carry_sum;
            }
            float out = total;
            if (AXPBY) out = a.alpha * total + a.beta * half_bits_to_float(a.y[row_j]);
            a.y[row_j] = float_to_half_bits(out);
        }

        // the row that holds entry `stop`
        const unsigned long long begun = __ballot(row_j >= r && row_j <= rw_end && e_j <= stop);
        const int open_row = r + __builtin_popcountll(begun) - 1;
        float open_sum = 0.f;
        u32 open_addr = row_origin;
        if (stop == tb + kTile) {
            open_sum = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sum_incl), kWave - 1));
            if (open_row == r) open_sum += carry_sum;
            open_addr = row_origin + (u32)__builtin_amdgcn_readlane((int)walk_incl, kWave - 1);
        }
        r = open_row - 1;
        do {
            ++r;
            if (r >= row_last) {  // as in finish_row
                e0 = e1 = 0x7fffffff;
                last_tile = 0;
                break;
            }
            slide_window(r);
            e0 = row_start(r);
            e1 = row_start(r + 1);
            if (e1 == e0) store_empty_row(r);
        } while (e1 == e0);
        const bool open = r < row_last && e0 < stop;
        acc0 = (open && lane == 0) ? open_sum : 0.f;
        acc1 = 0.f;
        row_addr = open ? open_addr : row_origin;
    };

    // The ring holds my first D tiles; now: take a slot, refill it, process.  Every step issues
    // exactly two loads (a "no tile" address once the range is exhausted), so a slot's loads are
    // always followed by those of the D - 1 other slots when it is awaited.
    for (u32 tile0 = first_tile; tile0 < last_tile; tile0 += D) {
        static_for<D>([&](auto slot) {
            constexpr int J = decltype(slot)::value;
            const u32 tile = tile0 + J;
            if (tile >= last_tile) return;  // wave-uniform; nothing is awaited or issued after this
            u32x4 vj;
            u32 dj;
            ring_take<D, J, kTileLoads - 2>(vj, dj);
            issue_slot(slot, tile + D, tile + D < last_tile, tile + D + 1 < last_tile);  // refill at once: the copy is out
            const int tb = (int)(tile_origin + (tile << kTileShift));
            const int tile_end = tb + kTile;
            if (e0 <= tb && e1 >= tile_end) {  // the common case for rows longer than a tile
                full_tile_pass(vj, dj);
                if (e1 == tile_end) finish_row(NB == 1 ? wave_sum(acc0 + acc1) : 0.f);
            } else {
                const int lim = tile_end < s_end ? tile_end : s_end;
                int pos = tb > e0 ? tb : e0;  // e0 > tb only in my first tile
                while (pos < lim) {
                    if constexpr (ROWS) {
                        // several rows end in what is left of this tile: all of them in one pass
                        const int ahead = r + (int)a.rows_pass_min;
                        if (ahead <= row_last && ahead <= win_base + 63 && row_start(ahead) <= lim) {
                            const int known = row_last < win_base + 63 ? row_last : win_base + 63;
                            const int known_start = row_start(known);
                            const int stop = known_start < lim ? known_start : lim;
                            if (__builtin_expect(stop <= pos, 0)) {  // see below: only a broken row_ptr does this
                                last_tile = 0;
                                break;
                            }
                            rows_pass(vj, dj, tb, pos, stop);
                            pos = stop;
                            continue;
                        }
                    }
                    const int seg_end = e1 < lim ? e1 : lim;
                    const bool row_done = seg_end == e1;
                    if constexpr (X_LDS && NB == 1) {
                        // Entries behind a row's end are masked where they are read (CHECKED), which
                        // costs a compare and a select per entry.  They can only matter if what they
                        // read is Inf or NaN, and then the row's sum is not finite: so run unmasked,
                        // and repeat the row's last piece masked in that rare case.  (A masked
                        // entry that reads a finite number adds +-0 to a sum that started at +0.)
                        const float keep0 = acc0, keep1 = acc1;
                        const u32 keep_addr = row_addr;
                        segment_pass(vj, dj, tb, pos, seg_end, index_constant<0>{});
                        if (row_done) {
                            float total = wave_sum(acc0 + acc1);
                            const u32 bits = __builtin_bit_cast(u32, total);
                            if (__builtin_expect((bits & 0x7f800000u) == 0x7f800000u, 0) && ((seg_end - tb) & 7) != 0) {
                                acc0 = keep0;
                                acc1 = keep1;
                                row_addr = keep_addr;
                                segment_pass(vj, dj, tb, pos, seg_end, index_constant<1>{});
                                total = wave_sum(acc0 + acc1);
                            }
                            finish_row(total);
                        }
                    } else {
                        segment_pass(vj, dj, tb, pos, seg_end, index_constant<1>{});
                        if (row_done) finish_row(NB == 1 ? wave_sum(acc0 + acc1) : 0.f);
                    }
                    pos = seg_end;
                }
            }
        });
    }
    MACKO_STAMP(6);
}

// y[r] = 0 (or beta*y[r]) for matrices without stored entries.
template <bool AXPBY>
__global__ void spmv_empty_kernel(uint16_t *y, int rows, float beta)
{
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r < rows) y[r] = AXPBY ? float_to_half_bits(beta * half_bits_to_float(y[r])) : (uint16_t)0;
}

// How the rows are dealt to n_waves owners: fills the fields of `a` the kernels (and the kernel that
// prepares a plan) derive the cuts from.
void set_cut_fields(SpmvArgs &a, u32 n_waves)
{
    // the sum the waves share evenly: stored entries plus row_cost per row (kept below 2^31)
    const long long room = ((1ll << 31) - 1 - a.padded) / (a.rows > 0 ? a.rows : 1);
    if ((long long)a.row_cost > room) a.row_cost = (u32)room;
    const long long weight = a.padded + (long long)a.row_cost * a.rows;
    a.entries_q = (u32)(weight / n_waves);
    a.entries_rem = (u32)(weight % n_waves);
    a.rows_q = (u32)a.rows / n_waves;
    a.rows_frac = (u32)(((unsigned long long)((u32)a.rows % n_waves) << 32) / n_waves);
    a.row_even = (u32)a.rows <= n_waves ? 1u : 0u;
}

template <int BLOCK, int D, bool X_LDS, bool AXPBY, int VB = 2, int NB = 1, int XF = 0, bool ROWS = false,
          bool PLAN = false>
int launch_stream(SpmvArgs a, int grid, size_t lds_bytes, hipStream_t stream)
{
    auto kernel = spmv_stream_kernel<BLOCK, D, X_LDS, AXPBY, VB, NB, XF, ROWS, PLAN>;
    set_cut_fields(a, (u32)grid * (BLOCK / kWave));
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

// What a row weighs, in entries, when rows are dealt to waves (SpmvArgs::row_cost): one tile.
// Measured on 14336 x 4096 matrices whose row lengths follow a Pareto law (41 to 3900 entries a
// row): 5 to 9 % faster than cuts on entries alone; matrices of equal rows do not change.
constexpr u32 kRowCost = 512;

// Row ends in (what is left of) a tile from which on the tile is worked in one pass over all its rows.
constexpr u32 kRowsPassMin = 3;
// Mean stored entries per row below which the variant with that pass is launched.
constexpr int kRowsPassBelow = 192;
// ... and rows per wave from which on: the pass costs three round trips to LDS, which a wave with
// a handful of rows in its only tile cannot hide (20000 x 300 at density 0.02, 32 rows per wave:
// 15.0 -> 8.0 us; 5000 x 64 at 0.5, 8 rows: 10.0 -> 7.6 us; 1000 x 1000 at 0.05, 3 rows: 6.0 -> 6.4 us).
constexpr long long kRowsPassRowsPerWave = 6;

#ifdef MACKO_DEV_HOOKS
// Launch-shape overrides for tuning runs (0 = built-in default); development builds only.
struct Tuning {
    int depth;  // tiles in flight per wave: 1 or 2
    int grid;   // workgroups
    int split;  // 1: always the split kernel, -1: never
    int row_cost;  // what a row weighs in the cuts, in entries (-1: built-in)
    int rows_pass_min;  // row ends in a tile from which on the tile is worked in one pass (-1: built-in, 0: never)
};
Tuning g_tuning = {0, 0, 0, -1, -1};
long long *g_trace = nullptr;
#endif

// The launch a matrix gets: workgroups of the whole-row kernel, or the split kernel.
struct LaunchShape {
    long long n_tiles;
    long long grid;  // workgroups of 1024 threads of the whole-row kernel
    bool split;      // rows are split between the waves of a workgroup instead (macko_spmv_split.hip)
};

LaunchShape launch_shape(int rows, long long padded, const DeviceInfo &info)
{
    constexpr int waves = 1024 / kWave;
    LaunchShape s;
    // about one wave per tile at most, so tiny matrices get a small grid; but when rows are about
    // a tile long, prefer one wave per row over a slightly smaller wave count that would leave
    // some waves with two rows
    s.n_tiles = (padded + kTile - 1) / kTile;
    long long waves_wanted = s.n_tiles;
    if (rows > waves_wanted) waves_wanted = rows < 2 * s.n_tiles ? rows : 2 * s.n_tiles;
    s.grid = (waves_wanted + waves - 1) / waves;
    if (s.grid > (long long)info.compute_units) s.grid = (long long)info.compute_units;
    if (s.grid < 1) s.grid = 1;
    // Whole rows per wave need about as many rows as waves; with clearly fewer, the workgroups own
    // the rows and their waves split them (macko_spmv_split.hip): one workgroup per compute unit,
    // at least a tile per wave and a row per workgroup.
    // Only where rows are long (four tiles and more on average): for short rows a wave per row is
    // the cheaper way even if most waves stay idle.
    s.split = 4 * (long long)rows < 3 * s.grid * waves && s.n_tiles >= 4 * (long long)rows;
#ifdef MACKO_DEV_HOOKS
    if (g_tuning.split) s.split = g_tuning.split > 0;
    if (g_tuning.grid && !s.split) s.grid = g_tuning.grid;
#endif
    return s;
}

template <bool AXPBY, int VB = 2, int NB = 1, int XF = 0>
int spmv_dispatch(const SpmvArgs &args, hipStream_t stream)
{
    SpmvArgs a = args;
    if (a.rows == 0) return 0;
    if (a.padded == 0) {
        hipLaunchKernelGGL(spmv_empty_kernel<AXPBY>, dim3((a.rows + 255) / 256), dim3(256), 0, stream, a.y,
                           a.rows, a.beta);
        return (int)hipGetLastError();
    }
    DeviceInfo info;
    int rc = device_info(&info);
    if (rc != 0) return rc;

    constexpr int waves = 1024 / kWave;
    const LaunchShape shape = launch_shape(a.rows, a.padded, info);
    const long long n_tiles = shape.n_tiles;
    long long grid = shape.grid;
    const bool split = shape.split;
#ifdef MACKO_DEV_HOOKS
    a.trace = g_trace;
#endif
    const size_t lds_x = (size_t)NB * ((size_t)kLdsFront + 2 * (size_t)a.cols + kLdsBack) + (XF == 1 ? 64 : 0);
    constexpr size_t piece_bytes = (size_t)waves * 4 * (NB + 1) + 4;  // what the split kernel keeps behind x
    if (split) {
        long long grid_split = (n_tiles + waves - 1) / waves;
        if (grid_split > a.rows) grid_split = a.rows;
        if (grid_split > (long long)info.compute_units) grid_split = (long long)info.compute_units;
        if (grid_split < 1) grid_split = 1;
#ifdef MACKO_DEV_HOOKS
        if (g_tuning.grid) grid_split = g_tuning.grid;
#endif
        const bool fits = lds_x + piece_bytes <= (size_t)info.max_lds_bytes;
        if (!fits && (XF != 0 || NB > 1)) return MACKO_E_INVALID_ARGUMENT;
        return spmv_split_launch(a, AXPBY, VB, NB, XF, fits, (int)grid_split, fits ? lds_x : 0, stream);
    }
    // Ring depth: one tile in flight behind the one being processed is enough, and cheapest to
    // start, when a wave walks only a few tiles; from about four tiles per wave on, two do better
    // (measured on the Llama shapes and larger ones, fp16 and int8; deeper is slower).
    int depth = n_tiles >= 4 * grid * waves ? 2 : 1;
    a.row_cost = kRowCost;
#ifdef MACKO_DEV_HOOKS
    if (g_tuning.row_cost >= 0) a.row_cost = (u32)g_tuning.row_cost;
    if (g_tuning.depth) depth = g_tuning.depth;
#endif
    const bool fits = lds_x <= (size_t)info.max_lds_bytes;
    if (XF != 0) {  // fused staging: x must fit in LDS (checked by the caller too)
        if (!fits) return MACKO_E_INVALID_ARGUMENT;
        if (depth == 2) return launch_stream<1024, 2, true, AXPBY, 2, 1, XF>(a, (int)grid, lds_x, stream);
        return launch_stream<1024, 1, true, AXPBY, 2, 1, XF>(a, (int)grid, lds_x, stream);
    }
    if (NB > 1) {  // NB vectors per launch: the caller has checked that they fit in LDS
        if (!fits) return MACKO_E_INVALID_ARGUMENT;
        if (depth == 2) return launch_stream<1024, 2, true, false, 2, NB>(a, (int)grid, lds_x, stream);
        return launch_stream<1024, 1, true, false, 2, NB>(a, (int)grid, lds_x, stream);
    }
    if (!fits) return launch_stream<1024, 2, false, AXPBY, VB>(a, (int)grid, 0, stream);
    // Short rows (several ends per tile on average): the variant that works all the rows of a tile in
    // one pass, if there is room for its 2 KB per wave behind x.
    const size_t lds_rows = (lds_x + 15) & ~(size_t)15;
    const size_t lds_all = lds_rows + (size_t)waves * kTile * 4;
    bool rows_variant = a.padded < (long long)kRowsPassBelow * a.rows && (long long)a.rows >= kRowsPassRowsPerWave * grid * waves &&
                        lds_all <= (size_t)info.max_lds_bytes;
    a.rows_pass_min = kRowsPassMin;
#ifdef MACKO_DEV_HOOKS
    if (g_tuning.rows_pass_min >= 0) {
        rows_variant = g_tuning.rows_pass_min > 0 && lds_all <= (size_t)info.max_lds_bytes;
        a.rows_pass_min = (u32)g_tuning.rows_pass_min;
    }
#endif
    // A plan is used if it was built for exactly this launch (same number of waves); any other is ignored.
    const bool planned = VB == 2 && a.plan != nullptr && (long long)a.plan_entries == 2 * (grid * waves + 1);
    if (rows_variant) {
        a.rows_pass_lds = (u32)lds_rows;
        if constexpr (VB == 2) {
            if (planned) {
                if (depth == 2) return launch_stream<1024, 2, true, AXPBY, 2, 1, 0, true, true>(a, (int)grid, lds_all, stream);
                return launch_stream<1024, 1, true, AXPBY, 2, 1, 0, true, true>(a, (int)grid, lds_all, stream);
            }
        }
        if (depth == 2) return launch_stream<1024, 2, true, AXPBY, VB, 1, 0, true>(a, (int)grid, lds_all, stream);
        return launch_stream<1024, 1, true, AXPBY, VB, 1, 0, true>(a, (int)grid, lds_all, stream);
    }
    if constexpr (VB == 2) {
        if (planned) {
            if (depth == 2) return launch_stream<1024, 2, true, AXPBY, 2, 1, 0, false, true>(a, (int)grid, lds_x, stream);
            return launch_stream<1024, 1, true, AXPBY, 2, 1, 0, false, true>(a, (int)grid, lds_x, stream);
        }
    }
    if (depth == 2) return launch_stream<1024, 2, true, AXPBY, VB>(a, (int)grid, lds_x, stream);
    return launch_stream<1024, 1, true, AXPBY, VB>(a, (int)grid, lds_x, stream);
}

// One thread per cut: cut k is where wave k of the launch starts (cut n_waves: the end), by the
// rule the kernel itself applies when it has no plan: the first row r with
// row_ptr[r] + row_cost * r >= target k, or the row before if that is nearer; even shares of the
// rows when there are no more rows than waves.  plan[2k] = row, plan[2k + 1] = row_ptr[row].
__global__ void plan_kernel(const SpmvArgs a, u32 n_waves, int *__restrict__ plan)
{
    const u32 k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k > n_waves) return;
    int cut;
    if (k == 0) {
        cut = 0;
    } else if (k == n_waves) {
        cut = a.rows;
    } else if (a.row_even) {
        cut = (int)(k * a.rows_q + __umulhi(k, a.rows_frac));
    } else {
        const long long target = (long long)even_split(k, a.entries_q, a.entries_rem);
        const long long row_cost = (long long)a.row_cost;
        int lo = 0, hi = a.rows;  // cost(rows) = the whole sum >= any target
        while (lo < hi) {
            const int mid = lo + ((hi - lo) >> 1);
            if ((long long)a.row_ptr[mid] + row_cost * mid >= target) hi = mid; else lo = mid + 1;
        }
        cut = lo;
        if (cut > 0) {
            const long long after = (long long)a.row_ptr[cut] + row_cost * cut;
            const long long before = (long long)a.row_ptr[cut - 1] + row_cost * (cut - 1);
            if (target - before < after - target) cut -= 1;
        }
    }
    plan[2 * k] = cut;
    plan[2 * k + 1] = a.row_ptr[cut];
}

// Waves of the launch a plan describes, 0 if this shape takes none (no stored entries, rows split
// between waves, or x too long for LDS).
int plan_waves(int rows, int cols, long long padded, long long *n_waves)
{
    *n_waves = 0;
    if (rows == 0 || padded == 0) return 0;
    DeviceInfo info;
    const int rc = device_info(&info);
    if (rc != 0) return rc;
    const LaunchShape shape = launch_shape(rows, padded, info);
    const size_t lds_x = (size_t)kLdsFront + 2 * (size_t)cols + kLdsBack;
    if (shape.split || lds_x > (size_t)info.max_lds_bytes) return 0;
    *n_waves = shape.grid * (1024 / kWave);
    return 0;
}

// LDS the split kernel keeps behind x at most (16 waves, up to 8 vectors and a flag each)
constexpr size_t kSplitPieceBytes = 16 * 4 * 9 + 4;

int check_spmv_args(const void *values, const void *deltas, const int32_t *row_ptr, const void *x, void *y,
                    int32_t rows, int32_t cols, int64_t padded, int value_bytes = 2)
{
    if (rows < 0 || cols < 0 || padded < 0) return MACKO_E_INVALID_ARGUMENT;
    if (padded % kChunk != 0) return MACKO_E_INVALID_ARGUMENT;
    if (padded >= (1ll << 31) - 8192) return MACKO_E_INVALID_ARGUMENT;
    if (rows > 0 && (row_ptr == nullptr || y == nullptr)) return MACKO_E_INVALID_ARGUMENT;
    if (padded > 0 && (values == nullptr || deltas == nullptr || x == nullptr || cols == 0))
        return MACKO_E_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(values) & (uintptr_t)(8 * value_bytes - 1)) ||
        (reinterpret_cast<uintptr_t>(deltas) & 3) ||
        (reinterpret_cast<uintptr_t>(row_ptr) & 3) || (reinterpret_cast<uintptr_t>(x) & 1) ||
        (reinterpret_cast<uintptr_t>(y) & 1))
        return MACKO_E_INVALID_ARGUMENT;
    return 0;
}

}  // namespace
}  // namespace macko

#ifdef MACKO_DEV_HOOKS
extern "C" void macko_spmv_set_trace(long long *device_buffer) { macko::g_trace = device_buffer; }
extern "C" void macko_spmv_tune(int depth, int grid, int active, int split)
{
    // active: 0 = built-in values; else 1 + row_cost + 65536 * (1 + rows_pass_min)
    const int row_cost = active > 0 ? ((active - 1) & 0xffff) : -1;
    const int rows_pass_min = active > 0 ? ((active - 1) >> 16) - 1 : -1;
    macko::g_tuning = macko::Tuning{depth, grid, split, row_cost, rows_pass_min};
}
#endif

extern "C" int macko_spmv_f16(const void *values, const void *deltas, const int32_t *row_ptr, const void *x,
                              void *y, int32_t rows, int32_t cols, int64_t padded_entries, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries);
    if (rc != 0) return rc;
    SpmvArgs a{(const u32 *)values, (const u32 *)deltas, row_ptr, (const uint16_t *)x, (uint16_t *)y,
               rows,                cols,                padded_entries, 1.0f,          0.0f,
               0,                   0,                   0,              0,             0,
               0,                   0};
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
               rows,                cols,                padded_entries, alpha,         beta,
               0,                   0,                   0,              0,             0,
               0,                   0};
    return spmv_dispatch<true>(a, as_stream(stream));
}

// ---- prepared cuts (no counterpart upstream) ------------------------------------------------------
extern "C" int macko_spmv_plan_entries(int32_t rows, int32_t cols, int64_t padded_entries, int32_t *entries)
{
    using namespace macko;
    if (entries == nullptr || rows < 0 || cols < 0 || padded_entries < 0) return MACKO_E_INVALID_ARGUMENT;
    long long n_waves = 0;
    const int rc = plan_waves(rows, cols, padded_entries, &n_waves);
    *entries = n_waves > 0 ? (int32_t)(2 * (n_waves + 1)) : 0;
    return rc;
}

extern "C" int macko_spmv_plan_build(const int32_t *row_ptr, int32_t rows, int32_t cols, int64_t padded_entries,
                                     int32_t *plan, int32_t plan_entries, void *stream)
{
    using namespace macko;
    if (rows < 0 || cols < 0 || padded_entries < 0 || padded_entries % kChunk != 0 ||
        padded_entries >= (1ll << 31) - 8192)
        return MACKO_E_INVALID_ARGUMENT;
    long long n_waves = 0;
    const int rc = plan_waves(rows, cols, padded_entries, &n_waves);
    if (rc != 0) return rc;
    if ((long long)plan_entries != (n_waves > 0 ? 2 * (n_waves + 1) : 0)) return MACKO_E_INVALID_ARGUMENT;
    if (n_waves == 0) return 0;
    if (row_ptr == nullptr || plan == nullptr || (reinterpret_cast<uintptr_t>(row_ptr) & 3) ||
        (reinterpret_cast<uintptr_t>(plan) & 15))
        return MACKO_E_INVALID_ARGUMENT;
    SpmvArgs a{};
    a.row_ptr = row_ptr;
    a.rows = rows;
    a.cols = cols;
    a.padded = padded_entries;
    a.row_cost = kRowCost;
#ifdef MACKO_DEV_HOOKS
    if (g_tuning.row_cost >= 0) a.row_cost = (u32)g_tuning.row_cost;
#endif
    set_cut_fields(a, (u32)n_waves);
    const int threads = 256;
    hipLaunchKernelGGL(plan_kernel, dim3((unsigned)((n_waves + 1 + threads - 1) / threads)), dim3(threads), 0,
                       as_stream(stream), a, (u32)n_waves, plan);
    return (int)hipGetLastError();
}

extern "C" int macko_spmv_f16_planned(const void *values, const void *deltas, const int32_t *row_ptr,
                                      const int32_t *plan, int32_t plan_entries, const void *x, void *y,
                                      int32_t rows, int32_t cols, int64_t padded_entries, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries);
    if (rc != 0) return rc;
    if (plan_entries < 0 || (plan_entries > 0 && (plan == nullptr || (reinterpret_cast<uintptr_t>(plan) & 15))))
        return MACKO_E_INVALID_ARGUMENT;
    SpmvArgs a{};
    a.values = (const u32 *)values;
    a.deltas = (const u32 *)deltas;
    a.row_ptr = row_ptr;
    a.x = (const uint16_t *)x;
    a.y = (uint16_t *)y;
    a.rows = rows;
    a.cols = cols;
    a.padded = padded_entries;
    a.alpha = 1.0f;
    a.plan = plan_entries > 0 ? plan : nullptr;
    a.plan_entries = plan_entries;
    return spmv_dispatch<false>(a, as_stream(stream));
}

extern "C" int macko_spmv_f16_axpby_planned(const void *values, const void *deltas, const int32_t *row_ptr,
                                            const int32_t *plan, int32_t plan_entries, const void *x, void *y,
                                            int32_t rows, int32_t cols, int64_t padded_entries, float alpha,
                                            float beta, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries);
    if (rc != 0) return rc;
    if (plan_entries < 0 || (plan_entries > 0 && (plan == nullptr || (reinterpret_cast<uintptr_t>(plan) & 15))))
        return MACKO_E_INVALID_ARGUMENT;
    SpmvArgs a{};
    a.values = (const u32 *)values;
    a.deltas = (const u32 *)deltas;
    a.row_ptr = row_ptr;
    a.x = (const uint16_t *)x;
    a.y = (uint16_t *)y;
    a.rows = rows;
    a.cols = cols;
    a.padded = padded_entries;
    a.alpha = alpha;
    a.beta = beta;
    a.plan = plan_entries > 0 ? plan : nullptr;
    a.plan_entries = plan_entries;
    return spmv_dispatch<true>(a, as_stream(stream));
}

// int8 values x fp16 vector (macko_spmv_int8, src/macko_spmv/cuda/kernels.cuh:126-216).
extern "C" int macko_spmv_i8f16(const void *values, const void *deltas, const int32_t *row_ptr, const void *x,
                                void *y, int32_t rows, int32_t cols, int64_t padded_entries, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries, 1);
    if (rc != 0) return rc;
    SpmvArgs a{(const u32 *)values, (const u32 *)deltas, row_ptr, (const uint16_t *)x, (uint16_t *)y,
               rows,                cols,                padded_entries, 1.0f,          0.0f,
               0,                   0,                   0,              0,             0,
               0,                   0};
    return spmv_dispatch<false, 1>(a, as_stream(stream));
}

extern "C" int macko_spmv_i8f16_axpby(const void *values, const void *deltas, const int32_t *row_ptr,
                                      const void *x, void *y, int32_t rows, int32_t cols,
                                      int64_t padded_entries, float alpha, float beta, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries, 1);
    if (rc != 0) return rc;
    SpmvArgs a{(const u32 *)values, (const u32 *)deltas, row_ptr, (const uint16_t *)x, (uint16_t *)y,
               rows,                cols,                padded_entries, alpha,         beta,
               0,                   0,                   0,              0,             0,
               0,                   0};
    return spmv_dispatch<true, 1>(a, as_stream(stream));
}

// Y[b, :] = M X[b, :] for `batch` vectors: X is [batch, ldx] and Y [batch, ldy] row-major fp16
// (ldx >= cols, ldy >= rows).  The matrix is streamed once per group of up to eight vectors (as
// many as fit in LDS next to each other), so the cost per vector drops accordingly.  The upstream
// package has no batched entry: its LLM runner maps the single-vector operator over the batch
// dimension (python_scripts/util_run_pruned_llm.py:112-118).
extern "C" int macko_spmv_f16_batched(const void *values, const void *deltas, const int32_t *row_ptr,
                                      const void *x, void *y, int32_t rows, int32_t cols,
                                      int64_t padded_entries, int32_t batch, int64_t ldx, int64_t ldy,
                                      void *stream)
{
    using namespace macko;
    if (batch < 0 || ldx < cols || ldy < rows || ldx >= (1ll << 31) || ldy >= (1ll << 31))
        return MACKO_E_INVALID_ARGUMENT;
    if (batch == 0) return 0;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries);
    if (rc != 0) return rc;
    DeviceInfo info;
    rc = device_info(&info);
    if (rc != 0) return rc;
    const size_t per_vector = (size_t)kLdsFront + 2 * (size_t)cols + kLdsBack;
    int done = 0;
    while (done < batch) {
        const int left = batch - done;
        SpmvArgs a{(const u32 *)values, (const u32 *)deltas, row_ptr,
                   (const uint16_t *)x + (size_t)done * (size_t)ldx, (uint16_t *)y + (size_t)done * (size_t)ldy,
                   rows, cols, padded_entries, 1.0f, 0.0f, 0, 0, 0, 0, 0, (int)ldx, (int)ldy};
        int step;
        if (padded_entries > 0 && left >= 8 && 8 * per_vector + kSplitPieceBytes <= (size_t)info.max_lds_bytes) {
            step = 8;
            rc = spmv_dispatch<false, 2, 8>(a, as_stream(stream));
        } else if (padded_entries > 0 && left >= 4 && 4 * per_vector + kSplitPieceBytes <= (size_t)info.max_lds_bytes) {
            step = 4;
            rc = spmv_dispatch<false, 2, 4>(a, as_stream(stream));
        } else if (padded_entries > 0 && left >= 2 && 2 * per_vector + kSplitPieceBytes <= (size_t)info.max_lds_bytes) {
            step = 2;
            rc = spmv_dispatch<false, 2, 2>(a, as_stream(stream));
        } else {
            step = 1;
            rc = spmv_dispatch<false>(a, as_stream(stream));
        }
        if (rc != 0) return rc;
        done += step;
    }
    return 0;
}

namespace macko {
namespace {
// Extra conditions of the fused-input variants: whole 16-byte pieces only, and x must fit in LDS.
int check_fused_args(const void *x, const void *x2, int32_t cols, int64_t padded)
{
    if (padded == 0) return 0;
    if (x2 == nullptr || (cols & 7) != 0) return MACKO_E_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(x2) & 15)) return MACKO_E_INVALID_ARGUMENT;
    DeviceInfo info;
    int rc = device_info(&info);
    if (rc != 0) return rc;
    if ((size_t)kLdsFront + 2 * (size_t)cols + kLdsBack + 64 + kSplitPieceBytes > (size_t)info.max_lds_bytes) return MACKO_E_INVALID_ARGUMENT;
    return 0;
}
}  // namespace
}  // namespace macko

// y = M * rmsnorm(x), rmsnorm(x)[i] = fp16(x[i] * rsqrt(mean(x^2) + eps) * norm_weight[i]): the
// normalisation in front of a projection, folded into the product's own staging of its input.
// No upstream counterpart: the upstream harness runs the stock module for the norm
// (python_scripts/util_run_pruned_llm.py:136-160).
extern "C" int macko_spmv_f16_rmsnorm(const void *values, const void *deltas, const int32_t *row_ptr, const void *x,
                                      const void *norm_weight, float eps, void *y, int32_t rows, int32_t cols,
                                      int64_t padded_entries, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, x, y, rows, cols, padded_entries);
    if (rc != 0) return rc;
    rc = check_fused_args(x, norm_weight, cols, padded_entries);
    if (rc != 0) return rc;
    SpmvArgs a{(const u32 *)values, (const u32 *)deltas, row_ptr, (const uint16_t *)x, (uint16_t *)y,
               rows, cols, padded_entries, 1.0f, 0.0f, 0, 0, 0, 0, 0, 0, 0, (const uint16_t *)norm_weight, eps};
    return spmv_dispatch<false, 2, 1, 1>(a, as_stream(stream));
}

// y = alpha * M * (silu(gate) .* up) + beta * y: the gated activation of a Llama MLP folded into
// the down projection's staging of its input, and the residual into its epilogue.  alpha == 1
// with beta == 0 leaves y unread.  No upstream counterpart (see above).
extern "C" int macko_spmv_f16_silu_mul_axpby(const void *values, const void *deltas, const int32_t *row_ptr,
                                             const void *gate, const void *up, void *y, int32_t rows, int32_t cols,
                                             int64_t padded_entries, float alpha, float beta, void *stream)
{
    using namespace macko;
    int rc = check_spmv_args(values, deltas, row_ptr, gate, y, rows, cols, padded_entries);
    if (rc != 0) return rc;
    rc = check_fused_args(gate, up, cols, padded_entries);
    if (rc != 0) return rc;
    SpmvArgs a{(const u32 *)values, (const u32 *)deltas, row_ptr, (const uint16_t *)gate, (uint16_t *)y,
               rows, cols, padded_entries, alpha, beta, 0, 0, 0, 0, 0, 0, 0, (const uint16_t *)up, 0.0f};
    if (beta == 0.0f && alpha == 1.0f) return spmv_dispatch<false, 2, 1, 2>(a, as_stream(stream));
    return spmv_dispatch<true, 2, 1, 2>(a, as_stream(stream));
}
