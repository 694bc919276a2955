// LDS-ring grouped GEMM kernel: the fast path (persistent, 256 x 256 tiles, LDS-DMA, software-pipelined MFMA loop).
#pragma once

#include "gemm_epilogue.h"

namespace fmoe {

// --------------------------------------------------------------------- ring kernel
// NREG_ == 0: 4 slots, one K-slice issued per step, schedule tables in LDS (E <= 1024).
// NREG_  > 0: 5 slots (all 160 KB of LDS), K-slices issued in pairs so that the two
//             instructions touching the halves of a 128-byte line are adjacent and reach L2
//             as one full-line request; the schedule tables live in 3 * NREG_ registers of
//             every wave (E <= 64 * NREG_, total_rows < 2^31, K-slices per tile even).
template <int BM_, int BN_, int WGM_, int WGN_, int NREG_>
struct RingCfg {
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_, NREG = NREG_;
    static constexpr bool PAIR = NREG_ > 0;
    static constexpr int STAGES = PAIR ? 5 : 4;
    static constexpr int NW = WGM * WGN;
    static constexpr int NT = kWave * NW;
    static constexpr int TM = BM / WGM, TN = BN / WGN;
    static constexpr int FM = TM / 32, FN = TN / 32;
    static constexpr int STAGE_BYTES = (BM + BN) * 64;          // 64-byte K-slice per row
    static constexpr int RING_BYTES = STAGES * STAGE_BYTES;
    static constexpr int kMaxExperts = PAIR ? 64 * NREG_ : 1024;
    static constexpr int TAB_OFF = RING_BYTES;                   // int32 [E+1] row-tile prefix
    static constexpr int OFF_OFF = RING_BYTES + 4128;            // int64 [E+1] clamped offsets
    static constexpr int LDS_BYTES = PAIR ? RING_BYTES : OFF_OFF + (kMaxExperts + 1) * 8 + 8;
    static constexpr int XI = BM / 16 / NW, WI = BN / 16 / NW;   // LDS-DMA instructions per lane per slice
    static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "DMA passes must be whole");
    static_assert(TM % 32 == 0 && TN % 64 == 0, "wave tile must hold whole 32x32 fragments, FN even");
};

__device__ __forceinline__ int lds_off64(int row, int chunk) {   // 64-byte rows
    return row * 64 + ((chunk ^ ((row >> 2) & 3)) << 4);
}

// One 16-byte-per-lane global -> LDS transfer from base + voff: a wave-uniform base in
// SGPRs plus a 32-bit per-lane offset, so that stepping along K costs scalar adds only (VALU
// instructions queue behind the MFMAs of the SIMD's other wave).  No immediate offset: the
// hardware would add it to the LDS address as well.  The 64 lanes land on 1 KB of LDS
// starting at the wave-uniform byte address lds_addr (M0), lane l at +16*l.  Issued as
// inline asm so that the waits on it stay under this kernel's control (vmcnt is counted by
// hand below).
__device__ __forceinline__ void dma16(const uint8_t* base, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n"
                 :: "v"(voff), "s"(base), "s"(lds_addr) : "memory", "m0");
}

__device__ __forceinline__ int uniform_lane(int v, int src_lane) {
    return __builtin_amdgcn_readfirstlane(wave_bcast(v, src_lane));
}

//
// WTR: the weights are N-contiguous (B[e][k][n] with b_sn == 1, an [E, K, N]-contiguous tensor or
// the transposed view the input-gradient GEMM multiplies by) and are consumed in place.  A ring
// slot then holds the weight part of a K-slice as two blocks [32 k][128 n] of 256-byte rows (n
// 0..127 and 128..255 of the tile; gate and up columns with SWIGLU); LDS position p of row k
// holds 16-byte chunk p ^ 4*(k%4) of that row, and the fragments are read with
// ds_read_b64_tr_b16: within 16 lanes, lane j receives column j of 4 consecutive rows when lane
// i points at row i/4, columns 4*(i%4)..+3, so two reads give a lane its 8 k values of one
// column.  The four rows of a read and the two 16-lane groups served together fall into eight
// different 32-byte bank groups.  bf16, paired ring only.
//
// KWIN: every expert contracts over its own window of K (p.k_window): the weight-gradient
// GEMM.  Paired ring only; windows are whole pairs of K-slices, at least two pairs.
//
// XTR (with WTR and KWIN): both operands are given with the contraction index as their row
// index, A[m][k] = a[k * a_sk + m] and B[k][n] = b[k * b_sk + n]: the weight gradient straight
// from the row-major tensors it contracts (row gradients and input rows, both [rows, columns]
// with the rows of an expert contiguous), no transposed copies.  The activation part of a slot
// gets the layout described for WTR.  Windows are arbitrary row ranges: the slices of a tile
// cover the window rounded up to whole pairs (at least two), and in the last two double steps
// the fragments are masked beyond the window's end.  The rows read past the end belong to the
// next expert or, after the last one, to the slack the caller promises (k_slack_rows >= 128
// readable rows behind both operands; their contents do not matter).
// MSC (e4m3, paired ring): the row-wise scales are powers of two (p.scale_pow2) and are applied by
// the MFMAs themselves: every wave keeps the E8M0 codes of the reciprocal scales of its four
// activation row blocks and its two weight fragments in two registers, which are the block-scale
// operands of v_mfma_scale_f32_32x32x64_f8f6f4 (a power-of-two factor on all 64 products of an
// output element in every K-step: the accumulator holds exactly what the division in the epilogue
// would give).  The scales of the next tile are fetched inside the epilogue of the current one
// (row indices before it, the scales behind its first row block, packed at its end), so that no
// tile waits for an index -> scale chain and the epilogue multiplies nothing.
template <typename TL, bool FP8, int EPI, bool WTR = false, bool KWIN = false, bool XTR = false, bool MSC = false>
__global__ __launch_bounds__(TL::NT) void grouped_gemm_ring_kernel(const GemmParams p) {
    static_assert(!MSC || (FP8 && TL::PAIR && !KWIN && !WTR && !XTR), "MFMA-applied scales: e4m3 on the paired ring");
    static_assert(!WTR || (TL::PAIR && !FP8 && TL::BN == 256 && TL::NW == 8),
                  "in-place N-contiguous weights: bf16, paired ring, 256-column tiles of 8 waves");
    static_assert(!KWIN || TL::PAIR, "contraction windows: paired ring");
    static_assert(XTR ? (WTR && KWIN && TL::BM == 256 && EPI == FMOE_EPI_NONE) : !(KWIN && WTR),
                  "row-indexed operands come together, with a window, and without an epilogue");
    constexpr int BM = TL::BM, BN = TL::BN, NW = TL::NW, STAGES = TL::STAGES;
    constexpr int FM = TL::FM, FN = TL::FN, TM = TL::TM, TN = TL::TN;
    constexpr bool PAIR = TL::PAIR;
    // (the epilogue is instantiated with ALWAYS_VEC = true below: its stores go through
    // store16_uniform_base, are all issued, and end with a counted wait, which the first double
    // step of the following tile relies on when it skips its own)
    constexpr bool kEpilogueStoresUnconditional = true;
    constexpr int NR = PAIR ? TL::NREG : 1;
    constexpr int ESIZE = FP8 ? 1 : 2;
    constexpr int BK = 64 / ESIZE;
    constexpr bool SWIGLU = EPI == FMOE_EPI_SWIGLU;
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int XI = TL::XI, WI = TL::WI;
    constexpr int L = XI + WI;
    // the two wave rows take the tile's 32-row blocks alternately (see slot_row_to_tile_row)
    constexpr bool ROW_IL = !XTR && TL::WGM == 2 && FM == 4;
    // SPARSE: a tile whose valid rows end in its first half (a short expert, or the rows an expert
    // has beyond a multiple of the tile height) runs a second copy of the main loop that
    // multiplies only the first two of every wave's four row blocks; the others hold no valid row.
    constexpr bool SPARSE = ROW_IL && PAIR && !KWIN;
    constexpr int ACT_SPARSE = FM / 2;

    extern __shared__ __align__(16) uint8_t smem[];
    int32_t* s_tab = reinterpret_cast<int32_t*>(smem + TL::TAB_OFF);   // [E+1] row-tile prefix
    int64_t* s_off = reinterpret_cast<int64_t*>(smem + TL::OFF_OFF);   // [E+1] clamped offsets

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % TL::WGM, wn = wave / TL::WGM;
    const int khalf = lane >> 5;

    // ------------------------------------------------------------ schedule tables
    const int64_t R = p.total_rows;
    int total_m;
    // register tables: lane l of entry i describes expert 64 * i + l
    int r_end[NR];                            // row tiles up to and including this position
    // KWIN: the tables are in order of decreasing contraction window (the cost of an expert's
    // tiles), r_exp tells which expert sits at a position: dealing groups of tiles to the XCDs
    // back and forth then balances them whatever order the experts' loads come in.
    int r_exp[NR];
    if constexpr (PAIR) {
        int e_lo[NR], e_len[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int e = i * kWave + lane;
            int64_t lo = 0, len = 0;
            if (e < p.E) {
                lo = clamp_i64(p.offsets[e], 0, R);
                const int64_t hi = clamp_i64(p.offsets[e + 1], 0, R);
                len = hi > lo ? hi - lo : 0;
            }
            e_lo[i] = (int)lo;
            e_len[i] = (int)len;
            r_exp[i] = e;
        }
        if constexpr (KWIN) {
            int e_w[NR], rank[NR], s_lo[NR], s_len[NR];
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int e = i * kWave + lane;
                int64_t w = -1;                 // positions past the last expert sort to the end
                if (e < p.E) w = clamp_i64(p.k_window[e + 1] - p.k_window[e], 0, (int64_t)p.K);
                e_w[i] = (int)w;
                rank[i] = 0;
                s_lo[i] = s_len[i] = 0;
            }
            auto pick = [&](const int (&arr)[NR], int o) -> int {     // entry of expert o, wave-uniform
                int v = arr[0];
#pragma unroll
                for (int i = 1; i < NR; ++i)
                    if ((o >> 6) == i) v = arr[i];
                return uniform_lane(v, o & 63);
            };
            for (int o = 0; o < p.E; ++o) {     // rank = number of experts that sort before this one
                const int wo = pick(e_w, o);
#pragma unroll
                for (int i = 0; i < NR; ++i) {
                    const int e = i * kWave + lane;
                    rank[i] += (wo > e_w[i] || (wo == e_w[i] && o < e)) ? 1 : 0;
                }
            }
            for (int o = 0; o < p.E; ++o) {     // expert o moves to position rank[o]
                const int ro = pick(rank, o), lo = pick(e_lo, o), len = pick(e_len, o);
#pragma unroll
                for (int i = 0; i < NR; ++i)
                    if ((ro >> 6) == i && lane == (ro & 63)) {
                        r_exp[i] = o;
                        s_lo[i] = lo;
                        s_len[i] = len;
                    }
            }
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                e_lo[i] = s_lo[i];
                e_len[i] = s_len[i];
            }
        }
        int run = 0;
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int64_t lo = e_lo[i], len = e_len[i];
            const int tiles = (int)((len + BM - 1) / BM);
            const int inc = wave_inclusive_scan(tiles);
            r_end[i] = run + inc;
            run += uniform_lane(inc, kWave - 1);
        }
        total_m = run;
    } else {
        if (wave == 0) {
            int run = 0;
            for (int e0 = 0; e0 <= p.E; e0 += kWave) {
                const int e = e0 + lane;
                int64_t lo = 0, len = 0;
                if (e <= p.E) lo = clamp_i64(p.offsets[e], 0, R);
                if (e < p.E) {
                    const int64_t hi = clamp_i64(p.offsets[e + 1], 0, R);
                    len = hi > lo ? hi - lo : 0;
                }
                const int tiles = (int)((len + BM - 1) / BM);
                const int inc = wave_inclusive_scan(tiles);
                if (e < p.E) s_tab[e + 1] = run + inc;
                if (e <= p.E) s_off[e] = lo;
                run += wave_bcast(inc, kWave - 1);
            }
            if (lane == 0) s_tab[0] = 0;
        }
        __syncthreads();
        total_m = s_tab[p.E];
        r_end[0] = 0;
    }
    // The tiles of an XCD, numbered 0 .. xcd_count-1.  Paired ring: whole groups (kGroupM row
    // tiles x all column tiles: what shares operands in an XCD's L2) are dealt to the XCDs back
    // and forth (0..7, 7..0, ...).  A tile's cost follows its expert (the contraction window of
    // a weight gradient; a last row tile with few rows runs the shortened main loop), and a
    // contiguous range per XCD hands one of them all the long experts and another all the short
    // ones; a plain round robin still favours the low XCDs when the experts come sorted by
    // load.  4-slot ring: one contiguous range of the tile order per XCD.
    const int64_t total_tiles = (int64_t)total_m * p.n_tiles;
    const int nslots = gridDim.x / kNumXcd;
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    const int64_t group_span = (int64_t)kGroupM * p.n_tiles;
    constexpr bool windowed = KWIN;
    constexpr bool deal_groups = PAIR;
    int64_t xcd_begin, xcd_count;
    if (deal_groups) {
        const int64_t n_groups = (total_m + kGroupM - 1) / kGroupM;
        // rounds of 8 groups; in odd rounds XCD x takes position 7 - x
        const int64_t full_rounds = n_groups / kNumXcd, rest = n_groups % kNumXcd;
        const int pos_in_last = (full_rounds & 1) ? kNumXcd - 1 - xcd : xcd;
        const int64_t mine = full_rounds + (pos_in_last < rest ? 1 : 0);
        xcd_begin = 0;
        xcd_count = mine * group_span;
        const int64_t last = n_groups - 1;                  // the last group may be short
        const int last_pos = (int)(last % kNumXcd);
        const int last_xcd = ((last / kNumXcd) & 1) ? kNumXcd - 1 - last_pos : last_pos;
        if (n_groups > 0 && last_xcd == xcd) xcd_count -= n_groups * group_span - total_tiles;
    } else {
        const int64_t per_xcd = (total_tiles + kNumXcd - 1) / kNumXcd;
        xcd_begin = xcd * per_xcd;
        xcd_count = total_tiles - xcd_begin < per_xcd ? total_tiles - xcd_begin : per_xcd;
    }
    // tile numbers of the paired ring fit 31 bits (the launcher checks): divisions by the group
    // span are one scalar multiply by a constant the host prepared, no division sequence whose
    // per-lane pieces the compiler would keep (or spill) across the tile loop
    auto div_span = [&](int64_t v) -> int64_t {
        if constexpr (PAIR) return (int64_t)(__umulhi((uint32_t)v, p.group_magic) >> p.group_magic_shift);
        else return v / group_span;
    };
    auto to_logical = [&](int64_t j) -> int64_t {
        if (!deal_groups) return xcd_begin + j;
        const int64_t round = div_span(j);
        const int pos = (round & 1) ? kNumXcd - 1 - xcd : xcd;
        return (round * kNumXcd + pos) * group_span + (j - round * group_span);
    };

    const int KT = p.K / BK;
    struct TileInfo { int expert; int nt; int64_t row0; int rows_valid; int64_t k_begin; int kt; int m0; int klen; };
    auto locate = [&](int64_t logical) -> TileInfo {
        const int64_t group = div_span(logical);
        const int first_m = (int)(group * kGroupM);
        const int gsize = total_m - first_m < kGroupM ? total_m - first_m : kGroupM;
        const int within = (int)(logical - group * group_span);
        static_assert(kGroupM == 4, "the quotient below knows the group sizes 1..4");
        const uint32_t uw = (uint32_t)within;
        const int q = gsize == 4 ? (int)(uw >> 2)
                      : gsize == 2 ? (int)(uw >> 1)
                                   : gsize == 3 ? (int)(((uint64_t)uw * 0xAAAAAAABull) >> 33) : within;
        const int mt = first_m + (within - q * gsize);
        TileInfo t;
        t.nt = q;
        if constexpr (PAIR) {
            // the tile's position = number of positions whose row tiles all precede mt; its first
            // tile is where the position before it ends.  Only the running tile count is kept per
            // position (one register per 64 experts); the expert's first row and row count come from
            // offsets[] through the scalar cache: two loads that wait on their own counter, where a
            // table register spilled to scratch is reloaded behind a wait that drains the LDS-DMA
            // stream.  (Lane rl of every table register first, then a scalar select among them:
            // selecting the register first reads as indexing an array by a run-time value, and the
            // compiler then keeps the table in scratch memory.)
            int cnt = 0;
#pragma unroll
            for (int i = 0; i < NR; ++i) cnt += __builtin_popcountll(__ballot(r_end[i] <= mt));
            cnt = __builtin_amdgcn_readfirstlane(cnt);
            cnt = cnt < p.E ? cnt : p.E - 1;        // (unreachable for consistent offsets)
            const int ri = cnt >> 6, rl = cnt & 63, pri = (cnt - 1) >> 6, prl = (cnt - 1) & 63;
            int first = 0, ex = 0;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int f = uniform_lane(r_end[i], prl), x = KWIN ? uniform_lane(r_exp[i], rl) : 0;
                if (cnt > 0 && pri == i) first = f;
                if (ri == i) ex = x;
            }
            const int expert = KWIN ? ex : cnt;
            int64_t o_lo, o_hi;
            scalar_load_i64x2(p.offsets + expert, o_lo, o_hi);
            o_lo = clamp_i64(o_lo, 0, R);
            o_hi = clamp_i64(o_hi, 0, R);
            const int lo = (int)o_lo, len = (int)(o_hi > o_lo ? o_hi - o_lo : 0);
            const int skip = (mt - first) * BM;
            t.expert = expert;
            t.m0 = skip;
            t.row0 = (int64_t)lo + skip;
            const int left = len - skip;
            t.rows_valid = left < BM ? left : BM;
        } else {
            int lo = 0, hi = p.E;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (s_tab[mid] <= mt) lo = mid; else hi = mid;
            }
            t.expert = lo;
            const int64_t e_lo = s_off[lo], e_hi = s_off[lo + 1];
            t.row0 = e_lo + (int64_t)(mt - s_tab[lo]) * BM;
            const int64_t left = (e_hi > e_lo ? e_hi : e_lo) - t.row0;
            t.rows_valid = (int)(left < BM ? left : BM);
        }
        t.k_begin = 0;
        t.kt = KT;
        t.klen = 0;
        if constexpr (!PAIR) t.m0 = 0;
        if constexpr (XTR) {
            // any row range; whole pairs of K-slices, at least two pairs
            const int e = __builtin_amdgcn_readfirstlane(t.expert);
            const int64_t lo = clamp_i64(p.k_window[e], 0, (int64_t)p.K);
            const int64_t hi = clamp_i64(p.k_window[e + 1], lo, (int64_t)p.K);
            int64_t kt = (hi - lo + 2 * BK - 1) / (2 * BK) * 2;
            t.kt = (int)(kt < 4 ? 4 : kt);
            t.k_begin = lo;
            t.klen = (int)(hi - lo);
        } else if (windowed) {
            // whole pairs of K-slices, at least two pairs, inside the operands' columns
            const int e = __builtin_amdgcn_readfirstlane(t.expert);
            const int64_t lo = p.k_window[e], hi = p.k_window[e + 1];
            int64_t kt = ((hi > lo ? hi - lo : 0) + 2 * BK - 1) / (2 * BK) * 2;
            kt = kt < 4 ? 4 : kt;
            kt = kt > KT / 2 * 2 ? KT / 2 * 2 : kt;
            t.kt = (int)kt;
            t.k_begin = clamp_i64(lo, 0, (int64_t)p.K - kt * BK);
        }
        return t;
    };

    // ------------------------------------------------------------ LDS-DMA geometry
    // DMA instruction i of this wave fills LDS rows (i*NW + wave)*16 .. +15 of the X (or W)
    // part of a ring slot: lane l -> row + l/4, 16-byte position l%4, which holds global
    // chunk (l%4) ^ ((row >> 2) & 3) of that row's 64-byte K-slice (the read-side swizzle).
    // These are needed twice per tile and cost a few VALU instructions: they are recomputed from
    // a copy of the lane number the compiler cannot see through rather than kept in registers
    // across the main loop, where the accumulators and fragments leave none to spare.
    auto dma_row = [&](int i) -> int {          // LDS row of DMA instruction i for this lane
        int l = lane;
        asm volatile("" : "+v"(l));
        return (i * NW + wave) * 16 + (l >> 2);
    };
    auto dma_swizzle = [&](int i) -> int {      // byte position inside the row's 64-byte slice
        int l = lane;
        asm volatile("" : "+v"(l));
        return (((l & 3) ^ ((((i * NW + wave) * 16 + (l >> 2)) >> 2) & 3)) << 4);
    };
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)smem;

    // ROW_IL: row r of a ring slot's activation part (wave row r / TM reads it, as block
    // (r % TM) / 32 of its four) holds the tile's row block 2 * block + wave row: the two wave rows
    // take the tile's 32-row blocks alternately, and a tile with few valid rows leaves both the
    // same number of blocks to multiply.
    auto slot_row_to_tile_row = [&](int r) -> int {
        if constexpr (!ROW_IL) return r;
        else return (((r % TM) >> 5) * 2 + r / TM) * 32 + (r & 31);
    };
    // source rows (row_index entries) of a tile, fetched ahead of the pointer computation
    auto fetch_rows = [&](const TileInfo& t, int64_t* ridx) {
        if constexpr (XTR) return;          // rows are not indexed: make_ptrs needs the tile only
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            const int xr = slot_row_to_tile_row(dma_row(i));
            const int64_t r = t.row0 + (xr < t.rows_valid ? xr : 0);
            ridx[i] = p.row_index ? p.row_index[r] : r;
        }
    };
    // per-lane byte offsets of the rows this lane fetches, relative to wave-uniform bases
    uint32_t xoff[XI], woff[WI];
    const uint8_t* xbase = p.a;
    const uint8_t* wbase[WI];
    static_assert(!SWIGLU || (BN / 2) % (16 * NW) == 0, "a DMA instruction must not straddle gate and up rows");
    // fetched row_index entries -> this lane's byte offsets into A
    auto rows_to_offsets = [&](const int64_t* ridx, uint32_t* out) {
        if constexpr (XTR) return;
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            int64_t s = ridx[i];
            if (p.row_index) {
                if (PAIR) s = div_index32(p, (int32_t)s);      // (values below 2^31, as in the epilogue)
                else s = p.index_shift >= 0 ? (s >> p.index_shift) : s / p.index_div;
            }
            s = clamp_i64(s, 0, p.a_rows - 1);
            out[i] = (uint32_t)(s * (p.a_stride_row * ESIZE)) + dma_swizzle(i);
        }
    };
    auto make_ptrs = [&](const TileInfo& t, const uint32_t* row_offsets) {
        const int expert = __builtin_amdgcn_readfirstlane(t.expert);
        const int64_t k_begin = KWIN ? t.k_begin : 0;
        const int n0 = t.nt * BN_OUT;
        if constexpr (XTR) {
            // instruction i of this wave: k rows 4*wave + lane/16 of row block i (128 tile rows),
            // LDS position lane%16 holding chunk (lane%16) ^ 4*(lane/16)
            xbase = p.a + k_begin * p.a_sk * ESIZE;
            int l = lane;
            asm volatile("" : "+v"(l));
            const int kr = 4 * wave + (l >> 4);
            const int c = (l & 15) ^ (4 * (l >> 4));
#pragma unroll
            for (int i = 0; i < XI; ++i) {
                int m = t.m0 + i * (BM / 2) + 8 * c;
                const int last = t.m0 + t.rows_valid - 8;       // rows per expert: a multiple of 8
                m = m <= last ? m : (last > 0 ? last : 0);
                xoff[i] = (uint32_t)(((int64_t)kr * p.a_sk + m) * ESIZE);
            }
        } else {
            xbase = p.a + ((int64_t)expert * p.a_stride_e + k_begin) * ESIZE;
#pragma unroll
            for (int i = 0; i < XI; ++i) xoff[i] = row_offsets[i];
        }
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            const bool up = SWIGLU && i * NW * 16 >= BN / 2;
            if constexpr (WTR) {
                // instruction i of this wave: rows 4*wave + lane/16 of column block i, LDS position lane%16
                int l = lane;
                asm volatile("" : "+v"(l));
                const int kr = 4 * wave + (l >> 4);
                const int c = (l & 15) ^ (4 * (l >> 4));
                int n = n0 + (SWIGLU ? 0 : i * (BN / 2)) + 8 * c;
                n = n + 8 <= p.N ? n : p.N - 8;
                wbase[i] = (up ? p.b2 : p.b) + ((int64_t)expert * p.b_se + k_begin * p.b_sk) * ESIZE;
                woff[i] = (uint32_t)(((int64_t)kr * p.b_sk + n) * ESIZE);
            } else {
                int n = n0 + dma_row(i) - (up ? BN / 2 : 0);
                n = n < p.N ? n : p.N - 1;
                wbase[i] = (up ? p.b2 : p.b) + ((int64_t)expert * p.b_se + k_begin) * ESIZE;
                woff[i] = (uint32_t)((int64_t)n * p.b_sn * ESIZE) + dma_swizzle(i);
            }
        }
    };
    // bytes between the weight rows of consecutive K-slices
    const int64_t wstep = WTR ? (int64_t)BK * p.b_sk * ESIZE : 64;
    const int64_t xstep = XTR ? (int64_t)BK * p.a_sk * ESIZE : 64;
    // A second product a2 * b2 continued in the same accumulators: the K-slices from split_kt on
    // come from a2 and b2, addressed with the strides of a and b.  (A pair of slices never
    // straddles the split: k_split is a whole number of pairs.)
    constexpr bool SPLIT = WTR && PAIR && !FP8 && !SWIGLU && !KWIN && !XTR;
    const int split_kt = SPLIT && p.a2 ? p.k_split / BK : 0x7fffffff;
    const int64_t split_x = SPLIT && p.a2 ? (p.a2 - p.a) - (int64_t)split_kt * xstep : 0;
    const int64_t split_w = SPLIT && p.a2 ? (p.b2 - p.b) - (int64_t)split_kt * wstep : 0;
    // one K-slice into slot sa; in pair mode also the following slice into slot sb, the two
    // 64-byte halves of every row's 128 bytes requested by adjacent instructions
    auto issue = [&](int kt, int sa, int sb) {
        const uint32_t abase = lds_base + sa * TL::STAGE_BYTES;
        const uint32_t bbase = lds_base + sb * TL::STAGE_BYTES;
        int64_t koff = (int64_t)kt * xstep;
        int64_t wkoff = (int64_t)kt * wstep;
        if constexpr (SPLIT) {
            koff += kt >= split_kt ? split_x : 0;
            wkoff += kt >= split_kt ? split_w : 0;
        }
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            dma16(xbase + koff, xoff[i], abase + (i * NW + wave) * 1024);
            if (PAIR) dma16(xbase + koff + xstep, xoff[i], bbase + (i * NW + wave) * 1024);
        }
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            dma16(wbase[i] + wkoff, woff[i], abase + BM * 64 + (i * NW + wave) * 1024);
            if (PAIR) dma16(wbase[i] + wkoff + wstep, woff[i], bbase + BM * 64 + (i * NW + wave) * 1024);
        }
    };

    int wfrag_row[FN], xfrag_row[FM];
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
        int r;
        if (SWIGLU) r = (fn < FN / 2 ? 0 : BN / 2) + wn * (TN / 2) + (fn % (FN / 2)) * 32;
        else r = wn * TN + fn * 32;
        wfrag_row[fn] = r + (lane & 31);
    }
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) xfrag_row[fm] = wm * TM + fm * 32 + (lane & 31);
    // WTR: byte offset, inside the weight part of a slot, of this lane's first transposing read
    // of fragment fn (rows 8*khalf + l16/4 of the slice's first 16; +1024: the next 4 rows)
    int wtr_off[FN];
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
        const int l16 = lane & 15;
        const int frag0 = wfrag_row[fn] - (lane & 31);                       // first tile column of the fragment
        const int ncol = frag0 % (BN / 2) + 16 * ((lane >> 4) & 1) + 4 * (l16 & 3);
        const int row = 8 * khalf + (l16 >> 2);
        wtr_off[fn] = (frag0 / (BN / 2)) * 8192 + row * 256 + (((ncol >> 3) ^ (4 * (l16 >> 2))) << 4) + (ncol & 7) * 2;
    }
    // XTR: the same for the activation fragments (tile rows wm*TM + fm*32 ..)
    int xtr_off[FM];
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
        const int l16 = lane & 15;
        const int frag0 = wm * TM + fm * 32;
        const int ncol = frag0 % (BM / 2) + 16 * ((lane >> 4) & 1) + 4 * (l16 & 3);
        const int row = 8 * khalf + (l16 >> 2);
        xtr_off[fm] = (frag0 / (BM / 2)) * 8192 + row * 256 + (((ncol >> 3) ^ (4 * (l16 >> 2))) << 4) + (ncol & 7) * 2;
    }

    // MSC: E8M0 codes of this lane's reciprocal scales, byte fm of sc_x for activation row block fm
    // (row lane & 31 of it), byte fn of sc_w for weight fragment fn (its column lane & 31)
    uint32_t sc_x = 0x7f7f7f7fu, sc_w = 0x7f7f7f7fu;
    // (sc_idx: row_index entries (low halves) of the lane's rows, or the rows themselves)
    auto sc_fetch_rows = [&](const TileInfo& t, int32_t (&sc_idx)[FM]) {       // hop 1: which source rows
        if constexpr (MSC) {
            int l = lane;
            asm volatile("" : "+v"(l));
#pragma unroll
            for (int fm = 0; fm < FM; ++fm) {
                const int tr = (ROW_IL ? (fm * 2 + wm) * 32 : wm * TM + fm * 32) + (l & 31);
                const int32_t r = (int32_t)t.row0 + (tr < t.rows_valid ? tr : 0);
                sc_idx[fm] = p.row_index ? reinterpret_cast<const int32_t*>(p.row_index)[2 * (int64_t)r] : r;
            }
        }
    };
    auto sc_fetch_scales = [&](const TileInfo& t, const int32_t (&sc_idx)[FM], float (&sc_xraw)[FM], float (&sc_wraw)[FN]) {     // hop 2: the scales themselves
        if constexpr (MSC) {
            int l = lane;
            asm volatile("" : "+v"(l));
            const int32_t last = (int32_t)(p.a_rows - 1);
#pragma unroll
            for (int fm = 0; fm < FM; ++fm) {
                int32_t src = p.row_index ? div_index32(p, sc_idx[fm]) : sc_idx[fm];
                src = src < 0 ? 0 : (src > last ? last : src);
                sc_xraw[fm] = p.a_scale[src];
            }
            const int expert = __builtin_amdgcn_readfirstlane(t.expert);
            const int n0 = t.nt * BN_OUT;
#pragma unroll
            for (int fn = 0; fn < FN; ++fn) {
                const bool up = SWIGLU && fn >= FN / 2;
                int n = n0 + (SWIGLU ? wn * (TN / 2) + (fn % (FN / 2)) * 32 : wn * TN + fn * 32) + (l & 31);
                n = n < p.N ? n : p.N - 1;
                sc_wraw[fn] = (up ? p.b2_scale : p.b_scale)[(int64_t)expert * p.N + n];
            }
        }
    };
    auto sc_pack = [&](const float (&sc_xraw)[FM], const float (&sc_wraw)[FN]) {
        if constexpr (MSC) {
            uint32_t x = 0, w = 0x7f7f7f7fu;
#pragma unroll
            for (int fm = 0; fm < FM; ++fm) x |= e8m0_of_reciprocal(sc_xraw[fm]) << (8 * fm);
            static_assert(FM == 4 && FN <= 4, "one byte per row block / weight fragment");
#pragma unroll
            for (int fn = 0; fn < FN; ++fn) w = (w & ~(0xffu << (8 * fn))) | (e8m0_of_reciprocal(sc_wraw[fn]) << (8 * fn));
            sc_x = x;
            sc_w = w;
        }
    };

    if (slot >= xcd_count) return;
    const int my_tiles = (int)((xcd_count - slot + nslots - 1) / nslots);
    // 4-slot ring: every item of the block; paired ring: issue_next only starts the first tile
    const int total_items = PAIR ? 4 : my_tiles * KT;

    // The block's work is one flat stream of K-slices ("items"): KT per tile, tile after
    // tile.  Item i lives in ring slot i % STAGES.  The issue side runs ahead of the compute
    // side and crosses tile boundaries on its own; it only needs the row pointers of the
    // tile it is in, the compute side only the TileInfo for the epilogue.
    TileInfo cur = locate(to_logical(slot));   // tile being computed
    TileInfo nxt = cur;                     // tile after it (located one tile ahead)
    int64_t ilogical = slot;                // its number among the XCD's tiles
    int ikt = 0;                            // next K-slice to issue inside the issue tile
    int issued = 0;                         // items issued so far
    int islot = 0;                          // issued % STAGES
    // The row indices of a tile are fetched two tiles ahead, before the epilogue of the tile in
    // between, and turned into offsets right behind that epilogue: by then they have long
    // arrived, the wait the compiler needs for them counts the epilogue's stores exactly (they
    // are issued unconditionally, see store16_uniform_base), and no load the compiler knows of
    // is in flight while the main loop runs (its wait for one would also drain the LDS-DMA
    // stream, which it cannot see).
    int64_t ridx_next[XI];
    uint32_t xoff_next[XI];
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        ridx_next[i] = 0;
        xoff_next[i] = 0;
    }
    {
        int64_t r0[XI];
        uint32_t x0[XI];
        fetch_rows(cur, r0);
        rows_to_offsets(r0, x0);
        make_ptrs(cur, x0);
    }
    if constexpr (MSC) {                    // the first tile's scales: fetched here, in the open
        int32_t idx0[FM];
        float xraw0[FM], wraw0[FN];
        sc_fetch_rows(cur, idx0);
        sc_fetch_scales(cur, idx0, xraw0, wraw0);
        sc_pack(xraw0, wraw0);
    }
    auto enter_next = [&]() {               // the issue side moves on to the next tile
        make_ptrs(nxt, xoff_next);
    };
    auto issue_next = [&]() {
        if (issued >= total_items) return;
        if (ikt == KT) {                    // the issue side enters the next tile
            enter_next();
            ikt = 0;
        }
        const int sa = islot;
        islot = islot + 1 == STAGES ? 0 : islot + 1;
        if (PAIR) {
            issue(ikt, sa, islot);
            islot = islot + 1 == STAGES ? 0 : islot + 1;
            ikt += 2;
            issued += 2;
        } else {
            issue(ikt, sa, sa);
            ++ikt;
            ++issued;
        }
    };
    // The same pair issue cut into L parts (one row group, both halves of its 128-byte lines)
    // so that the parts can be spread between MFMAs: a burst of VMEM instructions from all
    // waves backs up the CU's one address path and every wave sits in its issue, unable to
    // start MFMAs, until its own instructions are through.
    uint32_t part_a = 0, part_b = 0;
    int64_t part_koff = 0, part_wkoff = 0;
    auto issue_part = [&](int j) {          // j is a compile-time constant after unrolling
        const uint8_t* base = j < XI ? xbase + part_koff : wbase[j >= XI ? j - XI : 0] + part_wkoff;
        const uint32_t voff = j < XI ? xoff[j < XI ? j : 0] : woff[j >= XI ? j - XI : 0];
        const uint32_t off = (j < XI ? (j * NW + wave) * 1024 : BM * 64 + ((j - XI) * NW + wave) * 1024);
        dma16(base, voff, part_a + off);
        dma16(base + (j < XI ? xstep : wstep), voff, part_b + off);
    };
    auto prefetch_next = [&]() {            // once per tile, early: locate the next tile and
        ilogical += nslots;                 // start fetching its source-row indices
        if (ilogical < xcd_count) {
            nxt = locate(to_logical(ilogical));
            fetch_rows(nxt, ridx_next);
        }
    };
    prefetch_next();
    rows_to_offsets(ridx_next, xoff_next);
    if (PAIR) {
        issue_next();                       // items 0..3
        issue_next();
    } else {
        for (int j = 0; j < STAGES - 1; ++j) issue_next();
    }

    // vmcnt bookkeeping.  Loads return in order, so "at most n operations outstanding"
    // means everything but the n youngest operations has landed; stores or other loads in
    // the queue only make the wait longer, never shorter.
    int landed = -1;                        // 4-slot ring: items <= landed are complete for this wave
    int c = 0;                              // 4-slot ring: item being computed
    int cslot = 0;                          // ring slot of the item being computed
    bf16x8 wfa[FN], xfa[FM], wfb[FN], xfb[FM];   // fragment double buffer of the pipelined loop
    i32x8 qwa[FN], qwb[FN], qx0[FM / 2], qx1[FM / 2];   // the same for e4m3 fragments
    for (int tile_i = 0; tile_i < my_tiles; ++tile_i) {
        f32x16 acc[FN][FM];
#pragma unroll
        for (int i = 0; i < FN; ++i)
#pragma unroll
            for (int j = 0; j < FM; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
#ifdef FMOE_TRACE
        uint64_t tstamp[18] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        FMOE_TRACE_STAMP(0);
        if (p.trace) tstamp[4] = __builtin_amdgcn_s_memtime();
#endif

        auto mma_slice = [&]() {
            const uint8_t* sx = smem + cslot * TL::STAGE_BYTES;
            const uint8_t* sw = sx + BM * 64;
            if (!FP8) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int chunk = 2 * s + khalf;
                    bf16x8 wf[FN], xf[FM];
#pragma unroll
                    for (int fn = 0; fn < FN; ++fn)
                        wf[fn] = *reinterpret_cast<const bf16x8*>(sw + lds_off64(wfrag_row[fn], chunk));
#pragma unroll
                    for (int fm = 0; fm < FM; ++fm)
                        xf[fm] = *reinterpret_cast<const bf16x8*>(sx + lds_off64(xfrag_row[fm], chunk));
#pragma unroll
                    for (int fn = 0; fn < FN; ++fn)
#pragma unroll
                        for (int fm = 0; fm < FM; ++fm)
                            acc[fn][fm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[fn], xf[fm], acc[fn][fm], 0, 0, 0);
                }
            } else {
                const int chunk = 2 * khalf;
                i32x8 wf[FN], xf[FM];
#pragma unroll
                for (int fn = 0; fn < FN; ++fn) {
                    const u32x4 lo = *reinterpret_cast<const u32x4*>(sw + lds_off64(wfrag_row[fn], chunk));
                    const u32x4 hi = *reinterpret_cast<const u32x4*>(sw + lds_off64(wfrag_row[fn], chunk + 1));
                    wf[fn] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                }
#pragma unroll
                for (int fm = 0; fm < FM; ++fm) {
                    const u32x4 lo = *reinterpret_cast<const u32x4*>(sx + lds_off64(xfrag_row[fm], chunk));
                    const u32x4 hi = *reinterpret_cast<const u32x4*>(sx + lds_off64(xfrag_row[fm], chunk + 1));
                    xf[fm] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                }
#pragma unroll
                for (int fn = 0; fn < FN; ++fn)
#pragma unroll
                    for (int fm = 0; fm < FM; ++fm)
                        acc[fn][fm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[fn], xf[fm], acc[fn][fm], 0, 0, 0, 0, 0, 0);
            }
            ++c;
            cslot = cslot + 1 == STAGES ? 0 : cslot + 1;
        };

        if constexpr (PAIR && !FP8) {
            // Software pipeline over "blocks" (half a K-slice: one 16-byte chunk per row and
            // lane half, 8 MFMAs): the fragments of block b+1 are read while block b
            // multiplies.  Two barriers per pair of items c, c+1 (a "double step"):
            //   B  after the last read of item c      -> its slot and the one of c-1 are refilled
            //   A' before the first read of item c+2  -> pair (c+2, c+3) has landed everywhere
            // Raw s_barrier (no fence): LDS reads of slots that stay valid may be in flight
            // across a barrier; the asm statements keep the compiler from moving LDS reads
            // over them.  The steady state is straight-line code: the issue side always has
            // something to fetch (past the end of the block's stream it re-reads the last
            // tile's rows into slots nobody looks at), and everything that depends on the
            // wave's half is a template parameter.
            // two transposing reads: this lane's 8 k values of one column, 16 rows of 256 bytes
            // (one MFMA's depth) starting at byte offset off of a slot part
            auto read_tr = [&](const uint8_t* a) -> bf16x8 {
                typedef __attribute__((ext_vector_type(4))) short s16x4;
                typedef __attribute__((ext_vector_type(8))) short s16x8;
                typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)a);
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(a + 1024));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                return __builtin_bit_cast(bf16x8, both);
            };
            // item: the slice's number inside the tile; mask_c: zero the weight-side values whose
            // k lies at or beyond the end of the tile's window (XTR, the tile's last slices)
            auto load_block = [&](bf16x8 (&wf)[FN], bf16x8 (&xf)[FM], int slot_i, int sub, int item, auto mask_c, auto act_c) {
                constexpr bool MASK = XTR && decltype(mask_c)::value;
                constexpr int ACT = decltype(act_c)::value;     // row blocks that are multiplied
                const uint8_t* sx = smem + slot_i * TL::STAGE_BYTES;
                const uint8_t* sw = sx + BM * 64;
                const int chunk = 2 * sub + khalf;
#pragma unroll
                for (int fn = 0; fn < FN; ++fn) {
                    if constexpr (WTR) wf[fn] = read_tr(sw + wtr_off[fn] + sub * 4096);
                    else wf[fn] = *reinterpret_cast<const bf16x8*>(sw + lds_off64(wfrag_row[fn], chunk));
                }
#pragma unroll
                for (int fm = 0; fm < ACT; ++fm) {
                    if constexpr (XTR) xf[fm] = read_tr(sx + xtr_off[fm] + sub * 4096);
                    else xf[fm] = *reinterpret_cast<const bf16x8*>(sx + lds_off64(xfrag_row[fm], chunk));
                }
                if constexpr (MASK) {
                    // register i of a fragment holds k = first + 2i, first + 2i + 1
                    const int left = cur.klen - (item * BK + 16 * sub + 8 * khalf);
                    u32x4 m;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        m[i] = left >= 2 * i + 2 ? 0xffffffffu : (left == 2 * i + 1 ? 0x0000ffffu : 0u);
#pragma unroll
                    for (int fn = 0; fn < FN; ++fn)
                        wf[fn] = __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, wf[fn]) & m);
                    // both sides: what lies behind the window need not even be finite
#pragma unroll
                    for (int fm = 0; fm < FM; ++fm)
                        xf[fm] = __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, xf[fm]) & m);
                }
            };
            // the 8 MFMAs of a block, with the L parts of the pair being issued between them
            // when DMA is set.  The two waves of a SIMD (w and w + NW/2) issue in different
            // blocks, so that while one sits in its VMEM issue the other feeds the MFMA pipe.
            auto mma_block = [&](const bf16x8 (&wf)[FN], const bf16x8 (&xf)[FM], auto dma_c, auto act_c) {
                constexpr bool DMA = decltype(dma_c)::value;
                constexpr int ACT = decltype(act_c)::value;
                constexpr int NM = FN * ACT;
                // part q of the pair goes out behind MFMA ceil((q + 1) * NM / L) - 1: evenly spread
                // whether the parts are as many as the MFMAs, a divisor or a multiple of them, or neither
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const int fn = m / ACT, fm = m % ACT;
                    acc[fn][fm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[fn], xf[fm], acc[fn][fm], 0, 0, 0);
                    if constexpr (DMA) {
                        constexpr auto slot_of = [](int q) { return ((q + 1) * NM + L - 1) / L - 1; };
                        bool any = false;
#pragma unroll
                        for (int q = 0; q < L; ++q) any |= slot_of(q) == m;
                        if (any) {
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int q = 0; q < L; ++q)
                                if (slot_of(q) == m) issue_part(q);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            };
            auto barrier = [&]() {
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            };
            // sched_barrier(0) pins the order "reads of the next block, then the MFMAs of this
            // one"; left alone the scheduler sinks the reads to just before their first use.
            int kitem = 0;                  // number, inside the tile, of the item in slot cslot
            // skip_wait (wave-uniform): the pair this step would wait for is known to have landed.  That
            // holds for the first step of every tile but the block's first: the pair was issued before
            // the previous epilogue, whose stores are all issued whatever their lanes' predicates
            // (store16_uniform_base) and followed by a wait that leaves at most that many operations
            // in flight, i.e. nothing older than the stores.  The counted wait here would sit out the
            // stores' own round trip instead (one counter serves loads and stores, in order).
            auto double_step = [&](auto half_c, auto last_c, auto mask_c, auto act_c, bool skip_wait) __attribute__((always_inline)) {
                constexpr int HALF = decltype(half_c)::value;
                constexpr int ACT = decltype(act_c)::value;
                constexpr bool LAST = decltype(last_c)::value;   // last of the tile: no fragments kept over the epilogue
                const int s1 = cslot + 1 == STAGES ? 0 : cslot + 1;
                const int s2 = s1 + 1 == STAGES ? 0 : s1 + 1;
                auto interleave = [&]() {   // one fragment read in the shadow of every MFMA
                    static_assert(ACT * FN >= ACT + FN, "more fragment reads than MFMAs to hide them under");
#pragma unroll
                    for (int i = 0; i < ACT + FN; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, (WTR || XTR) ? 2 : 1, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x008, ACT * FN - (ACT + FN), 0);
                };
                load_block(wfb, xfb, cslot, 1, kitem, mask_c, act_c);
                mma_block(wfa, xfa, std::false_type{}, act_c);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
                load_block(wfa, xfa, s1, 0, kitem + 1, mask_c, act_c);
                mma_block(wfb, xfb, std::false_type{}, act_c);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
                barrier();                  // B
                part_a = lds_base + islot * TL::STAGE_BYTES;    // pair (c+4, c+5)
                islot = islot + 1 == STAGES ? 0 : islot + 1;
                part_b = lds_base + islot * TL::STAGE_BYTES;
                islot = islot + 1 == STAGES ? 0 : islot + 1;
                part_koff = (int64_t)ikt * xstep;
                part_wkoff = WTR ? (int64_t)ikt * wstep : part_koff;
                if constexpr (SPLIT) {
                    part_koff += ikt >= split_kt ? split_x : 0;
                    part_wkoff += ikt >= split_kt ? split_w : 0;
                }
                ikt += 2;
                load_block(wfb, xfb, s1, 1, kitem + 1, mask_c, act_c);
                if constexpr (HALF == 0) __builtin_amdgcn_sched_barrier(0);
                mma_block(wfa, xfa, std::integral_constant<bool, HALF == 0>{}, act_c);
                if constexpr (HALF != 0) interleave();
                __builtin_amdgcn_sched_barrier(0);
                // pair (c+2, c+3) is older than the 2L instructions the first half just issued
                if (!skip_wait) {
                    if (HALF == 0) wait_vmcnt<2 * L>();
                    else wait_vmcnt<0>();
                }
                barrier();                  // A'
                if (!LAST) load_block(wfa, xfa, s2, 0, kitem + 2, mask_c, act_c);
                if constexpr (HALF == 1 || LAST) __builtin_amdgcn_sched_barrier(0);
                mma_block(wfb, xfb, std::integral_constant<bool, HALF == 1>{}, act_c);
                if constexpr (HALF != 1 && !LAST) interleave();
                __builtin_amdgcn_sched_barrier(0);
                cslot = s2;
                kitem += 2;
            };
            // the issue side runs 4 items ahead: it enters the next tile 4 items before the end;
            // the last two double steps hold the end of an XTR tile's window and mask it
            auto tile_steps = [&](auto half_c, auto act_c) __attribute__((always_inline)) {
                const int tile_kt = KWIN ? cur.kt : KT;
                bool landed = tile_i > 0;       // the first step's pair landed before the previous epilogue's stores
                for (int kt = 0; kt < tile_kt - 4; kt += 2) {
                    double_step(half_c, std::false_type{}, std::false_type{}, act_c, landed);
                    landed = false;
#ifdef FMOE_TRACE
                    if (kt < 8) FMOE_TRACE_STAMP(6 + kt / 2);
#endif
                }
                FMOE_TRACE_STAMP(10);
                enter_next();
                ikt = 0;
                double_step(half_c, std::false_type{}, std::true_type{}, act_c, landed);
                FMOE_TRACE_STAMP(11);
                double_step(half_c, std::true_type{}, std::true_type{}, act_c, false);
            };
            if (tile_i == 0) {              // pair 0 has landed everywhere
                wait_vmcnt<2 * L>();
                barrier();
            }
            load_block(wfa, xfa, cslot, 0, 0, std::true_type{}, std::integral_constant<int, FM>{});
            const bool sparse = SPARSE && cur.rows_valid <= p.short_tile_rows;
            if (wave < NW / 2) {
                if (sparse) tile_steps(std::integral_constant<int, 0>{}, std::integral_constant<int, SPARSE ? ACT_SPARSE : FM>{});
                else tile_steps(std::integral_constant<int, 0>{}, std::integral_constant<int, FM>{});
            } else {
                if (sparse) tile_steps(std::integral_constant<int, 1>{}, std::integral_constant<int, SPARSE ? ACT_SPARSE : FM>{});
                else tile_steps(std::integral_constant<int, 1>{}, std::integral_constant<int, FM>{});
            }
        } else if constexpr (PAIR) {
            // e4m3: the same double step; an item is one 32x32x64 MFMA deep, so its two blocks
            // split the activation fragments instead of K: block 0 reads both weight
            // fragments and activation fragments 0..FM/2-1, block 1 the other activation
            // fragments and reuses the weights.
            constexpr int HM = FM / 2;
            auto load_frag = [&](const uint8_t* base, int row) -> i32x8 {
                const int chunk = 2 * khalf;
                const u32x4 lo = *reinterpret_cast<const u32x4*>(base + lds_off64(row, chunk));
                const u32x4 hi = *reinterpret_cast<const u32x4*>(base + lds_off64(row, chunk + 1));
                return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
            };
            auto load_w_x0 = [&](i32x8 (&wf)[FN], i32x8 (&xh)[HM], int slot_i) {
                const uint8_t* sx = smem + slot_i * TL::STAGE_BYTES;
#pragma unroll
                for (int fn = 0; fn < FN; ++fn) wf[fn] = load_frag(sx + BM * 64, wfrag_row[fn]);
#pragma unroll
                for (int fm = 0; fm < HM; ++fm) xh[fm] = load_frag(sx, xfrag_row[fm]);
            };
            auto load_x1 = [&](i32x8 (&xh)[HM], int slot_i) {
                const uint8_t* sx = smem + slot_i * TL::STAGE_BYTES;
#pragma unroll
                for (int fm = 0; fm < HM; ++fm) xh[fm] = load_frag(sx, xfrag_row[HM + fm]);
            };
            // skip_c: the block's row blocks hold no valid row (sparse tile); only its share of the
            // DMA issue is left
            auto mma_block = [&](const i32x8 (&wf)[FN], const i32x8 (&xh)[HM], auto fm0_c, auto dma_c, auto skip_c) {
                constexpr bool DMA = decltype(dma_c)::value;
                constexpr int NM = FN * HM;
                if constexpr (decltype(skip_c)::value) {
                    if constexpr (DMA) {
#pragma unroll
                        for (int q = 0; q < L; ++q) issue_part(q);
                    }
                    return;
                }
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const int fn = m / HM, fm = m % HM;
                    constexpr int FM0 = decltype(fm0_c)::value;
                    if constexpr (MSC) {
                        // (the byte selectors are immediates of the instruction: after unrolling fn and
                        // fm are constants and one of the four forms is left)
                        static_assert(FN == 2 && HM == 2, "selector forms below");
                        if (fn == 0 && fm == 0) mfma_e4m3_scaled<0, FM0>(wf[0], xh[0], acc[0][FM0], sc_w, sc_x);
                        else if (fn == 0) mfma_e4m3_scaled<0, FM0 + 1>(wf[0], xh[1], acc[0][FM0 + 1], sc_w, sc_x);
                        else if (fm == 0) mfma_e4m3_scaled<1, FM0>(wf[1], xh[0], acc[1][FM0], sc_w, sc_x);
                        else mfma_e4m3_scaled<1, FM0 + 1>(wf[1], xh[1], acc[1][FM0 + 1], sc_w, sc_x);
                    } else {
                        acc[fn][FM0 + fm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            wf[fn], xh[fm], acc[fn][FM0 + fm], 0, 0, 0, 0, 0, 0);
                    }
                    if constexpr (DMA) {        // (part q behind MFMA ceil((q + 1) * NM / L) - 1, as in the bf16 loop)
                        constexpr auto slot_of = [](int q) { return ((q + 1) * NM + L - 1) / L - 1; };
                        bool any = false;
#pragma unroll
                        for (int q = 0; q < L; ++q) any |= slot_of(q) == m;
                        if (any) {
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int q = 0; q < L; ++q)
                                if (slot_of(q) == m) issue_part(q);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            };
            auto barrier = [&]() {
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            };
            auto double_step = [&](auto half_c, auto last_c, auto sparse_c, bool skip_wait) __attribute__((always_inline)) {   // skip_wait: as in the bf16 loop
                constexpr int HALF = decltype(half_c)::value;
                constexpr bool LAST = decltype(last_c)::value;
                constexpr bool SP = decltype(sparse_c)::value;  // row blocks HM.. are not multiplied
                constexpr std::false_type full{};
                const int s1 = cslot + 1 == STAGES ? 0 : cslot + 1;
                const int s2 = s1 + 1 == STAGES ? 0 : s1 + 1;
                if (!SP) load_x1(qx1, cslot);
                __builtin_amdgcn_sched_barrier(0);
                mma_block(qwa, qx0, std::integral_constant<int, 0>{}, std::false_type{}, full);
                __builtin_amdgcn_sched_barrier(0);
                load_w_x0(qwb, qx0, s1);
                __builtin_amdgcn_sched_barrier(0);
                mma_block(qwa, qx1, std::integral_constant<int, HM>{}, std::false_type{}, sparse_c);
                __builtin_amdgcn_sched_barrier(0);
                barrier();                  // B
                part_a = lds_base + islot * TL::STAGE_BYTES;    // pair (c+4, c+5)
                islot = islot + 1 == STAGES ? 0 : islot + 1;
                part_b = lds_base + islot * TL::STAGE_BYTES;
                islot = islot + 1 == STAGES ? 0 : islot + 1;
                part_koff = (int64_t)ikt * xstep;
                part_wkoff = WTR ? (int64_t)ikt * wstep : part_koff;
                ikt += 2;
                if (!SP) load_x1(qx1, s1);
                __builtin_amdgcn_sched_barrier(0);
                mma_block(qwb, qx0, std::integral_constant<int, 0>{}, std::integral_constant<bool, HALF == 0>{}, full);
                __builtin_amdgcn_sched_barrier(0);
                if (!skip_wait) {
                    if (HALF == 0) wait_vmcnt<2 * L>();
                    else wait_vmcnt<0>();
                }
                barrier();                  // A'
                if (!LAST) load_w_x0(qwa, qx0, s2);
                __builtin_amdgcn_sched_barrier(0);
                mma_block(qwb, qx1, std::integral_constant<int, HM>{}, std::integral_constant<bool, HALF == 1>{}, sparse_c);
                __builtin_amdgcn_sched_barrier(0);
                cslot = s2;
            };
            auto tile_steps = [&](auto half_c, auto sparse_c) __attribute__((always_inline)) {
                const int tile_kt = KWIN ? cur.kt : KT;
                // (whatever the compiler still counts as pending from the tile's set-up or the last
                // epilogue, spill reloads and the row-index loads, is settled by the counted wait at
                // the epilogue's end: left pending, such a wait lands inside this loop, where it
                // drains the LDS-DMA stream, which the compiler cannot see, on every iteration)
                bool landed = tile_i > 0;
                for (int kt = 0; kt < tile_kt - 4; kt += 2) {
                    double_step(half_c, std::false_type{}, sparse_c, landed);
                    landed = false;
#ifdef FMOE_TRACE
                    if (kt < 8) FMOE_TRACE_STAMP(6 + kt / 2);
#endif
                }
                FMOE_TRACE_STAMP(10);
                enter_next();
                ikt = 0;
                double_step(half_c, std::false_type{}, sparse_c, landed);
                FMOE_TRACE_STAMP(11);
                double_step(half_c, std::true_type{}, sparse_c, false);
            };
            if (tile_i == 0) {              // pair 0 has landed everywhere
                wait_vmcnt<2 * L>();
                barrier();
            }
            load_w_x0(qwa, qx0, cslot);
            const bool sparse = SPARSE && cur.rows_valid <= p.short_tile_rows;
            if (wave < NW / 2) {
                if (sparse) tile_steps(std::integral_constant<int, 0>{}, std::integral_constant<bool, SPARSE>{});
                else tile_steps(std::integral_constant<int, 0>{}, std::false_type{});
            } else {
                if (sparse) tile_steps(std::integral_constant<int, 1>{}, std::integral_constant<bool, SPARSE>{});
                else tile_steps(std::integral_constant<int, 1>{}, std::false_type{});
            }
        } else {
            for (int kt = 0; kt < KT; ++kt) {
                if (c > landed) {
                    const int younger = issued - 1 - c;
                    if (younger >= 2) wait_vmcnt<2 * L>();
                    else if (younger == 1) wait_vmcnt<L>();
                    else wait_vmcnt<0>();
                }
                // after this barrier every wave's share of item c is visible and every wave
                // has finished reading item c-1, whose slot the next issue overwrites
                __syncthreads();
                issue_next();
                mma_slice();
            }
            // All but the youngest issued slice have landed after this wait, so the first
            // slices of the next tile need no vmcnt wait and the epilogue's stores drain
            // behind them.
            wait_vmcnt<L>();
            landed = issued - 2;
        }
        if constexpr (MSC) mfma_results_guard();    // the last MFMAs' results are read by VALU code from here on
        FMOE_TRACE_STAMP(1);
        const TileInfo done = cur;
        cur = nxt;          // valid when another tile follows
        prefetch_next();    // nxt: the tile after that one; its row indices arrive during the epilogue
        FMOE_TRACE_STAMP(2);

        // MSC: the scales of the tile that is computed next (cur, when one follows): its row indices
        // are requested here, its scales behind the first row block of the epilogue (by then the
        // indices have arrived: the compiler's wait for them counts that block's stores exactly),
        // and the codes are packed at the epilogue's end, where the wait for the scale loads also
        // covers every LDS-DMA issued before the epilogue, as the counted wait there does.
        // (After the block's last tile cur is stale but still describes a tile of this launch:
        // the loads stay in bounds and their result is not used.)
        int32_t sc_idx[FM];
        float sc_xraw[FM], sc_wraw[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i) { sc_idx[i] = 0; sc_xraw[i] = 1.0f; }
#pragma unroll
        for (int i = 0; i < FN; ++i) sc_wraw[i] = 1.0f;
        if constexpr (MSC) sc_fetch_rows(cur, sc_idx);
        auto convert_rows = [&]() __attribute__((always_inline)) {
            if constexpr (MSC) sc_pack(sc_xraw, sc_wraw);
            rows_to_offsets(ridx_next, xoff_next);  // of the tile after the next one
        };
        auto scales_behind_block0 = [&](int fm) __attribute__((always_inline)) {
            if constexpr (MSC) {
                if (fm == 0) sc_fetch_scales(cur, sc_idx, sc_xraw, sc_wraw);
            }
        };
        auto hooks = make_hooks(scales_behind_block0, convert_rows);
#ifdef FMOE_TRACE
        gemm_epilogue<FM, FN, TM, TN, FP8, EPI, true, PAIR, XTR, ROW_IL, decltype(hooks), MSC>(
            p, acc, done.expert, done.nt * BN_OUT, done.row0, done.rows_valid, wm, wn, lane, hooks,
            (p.trace && tile_i < 32 && (wave == 0 || wave == NW / 2)) ? tstamp + 12 : nullptr);
#else
        static_assert(kEpilogueStoresUnconditional, "skip_wait needs an epilogue whose stores are all issued");
        gemm_epilogue<FM, FN, TM, TN, FP8, EPI, kEpilogueStoresUnconditional, PAIR, XTR, ROW_IL, decltype(hooks), MSC>(
            p, acc, done.expert, done.nt * BN_OUT, done.row0, done.rows_valid, wm, wn, lane, hooks);
#endif
#ifdef FMOE_TRACE
        FMOE_TRACE_STAMP(3);
        if (p.trace && tile_i < 32 && (wave == 0 || wave == NW / 2) && lane == 0) {
            tstamp[5] = __builtin_amdgcn_s_memtime();
            uint64_t* dst = p.trace + (((int64_t)blockIdx.x * 32 + tile_i) * 2 + (wave != 0)) * 8;
#pragma unroll
            for (int j = 0; j < 6; ++j) dst[j] = tstamp[j];
            dst[6] = (uint64_t)KT;
            dst[7] = (uint64_t)done.rows_valid;
            uint64_t* dst2 = p.trace + (int64_t)gridDim.x * 32 * 2 * 8 + (((int64_t)blockIdx.x * 32 + tile_i) * 2 + (wave != 0)) * 8;
#pragma unroll
            for (int j = 0; j < 6; ++j) dst2[j] = tstamp[6 + j];
            uint64_t* dst3 = dst2 + (int64_t)gridDim.x * 32 * 2 * 8;
#pragma unroll
            for (int j = 0; j < 6; ++j) dst3[j] = tstamp[12 + j];
        }
#endif
    }
    wait_vmcnt<0>();    // nothing may still be on its way into this block's LDS when it ends
}

}  // namespace fmoe
