// Streaming grouped GEMM kernel: experts with a handful of rows, bound by the weight stream.
#pragma once

#include "gemm_epilogue.h"

namespace fmoe {

// ------------------------------------------------------------------ streaming kernel
// The register-staged kernel above in persistent form, for the regime in which every expert holds
// a handful of rows and a launch is a stream of weights through the chip (64 x 256 tiles, 4 waves,
// two blocks per CU, bf16 or e4m3, 16-byte loads).  There a tile lasts some tens of microseconds
// and what it does besides streaming (locating itself, the first fetch with nothing to multiply
// yet, the epilogue) is a tenth of it, twice that for e4m3 whose tiles hold half the bytes.  Here a
// block walks its tiles in a loop: the next tile is located and its row indices are requested
// under the last K-slice of the current one, its first K-slice is requested before the current
// epilogue and lands while that stores (the loads precede the stores in the queue, and the
// stores are all issued, so the wait for the loads counts them exactly and does not sit out their
// round trip).  MSC (e4m3, power-of-two scales): the scales of the next tile travel with its first
// slice and are applied by the MFMAs (see the ring kernel), the epilogue has no index -> scale
// chain left.
template <int DT, int EPI, bool MSC>
__global__ __launch_bounds__(256, 2) void grouped_gemm_stream_kernel(const GemmParams p) {
    constexpr int BM = 64, BN = 256, NT = 256;
    constexpr int FM = 2, FN = 2, TM = 64, TN = 64;
    constexpr bool FP8 = DT == kDtE4m3;
    static_assert(DT == kDtBf16 || DT == kDtE4m3, "bf16 or e4m3 operands");
    static_assert(!MSC || FP8, "MFMA-applied scales are an e4m3 matter");
    constexpr int ESIZE = FP8 ? 1 : 2;
    constexpr int CHUNK_ELEMS = 16 / ESIZE;
    constexpr int BK = 128 / ESIZE;
    constexpr bool SWIGLU = EPI == FMOE_EPI_SWIGLU;
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int XP = BM * 8 / NT, WP = BN * 8 / NT;
    constexpr int STAGE_BYTES = (BM + BN) * 128;

    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave;
    const int khalf = lane >> 5;

    // ------------------------------------------------------------ schedule
    const int64_t R = p.total_rows;
    int64_t total_m = 0;
    for (int e0 = 0; e0 < p.E; e0 += kWave) {
        const int e = e0 + lane;
        int64_t len = 0;
        if (e < p.E) {
            const int64_t lo = clamp_i64(p.offsets[e], 0, R), hi = clamp_i64(p.offsets[e + 1], 0, R);
            len = hi > lo ? hi - lo : 0;
        }
        const long long inc = wave_inclusive_scan((long long)((len + BM - 1) / BM));
        total_m += wave_bcast(inc, kWave - 1);
    }
    const int64_t total_tiles = total_m * p.n_tiles;
    const int64_t per_xcd = (total_tiles + kNumXcd - 1) / kNumXcd;
    const int xcd = blockIdx.x % kNumXcd;
    const int64_t slot = blockIdx.x / kNumXcd, nslots = gridDim.x / kNumXcd;
    const int64_t xcd_begin = xcd * per_xcd;
    const int64_t xcd_count = total_tiles - xcd_begin < per_xcd ? total_tiles - xcd_begin : per_xcd;
    if (slot >= xcd_count) return;
    const int64_t group_span = (int64_t)kGroupM * p.n_tiles;

    struct Tile { int expert; int nt; int64_t row0; int rows_valid; };
    // (every wave runs this with the same arguments: ballots and broadcasts inside)
    auto locate = [&](int64_t logical) -> Tile {
        const int64_t group = logical / group_span;
        const int within = (int)(logical - group * group_span);
        const int64_t first_m = group * kGroupM;
        const int gsize = (int)(total_m - first_m < kGroupM ? total_m - first_m : kGroupM);
        const int64_t mt = first_m + within % gsize;
        Tile t;
        t.nt = within / gsize;
        t.expert = 0;
        t.row0 = 0;
        t.rows_valid = 0;
        int64_t before = 0;
        for (int e0 = 0; e0 < p.E; e0 += kWave) {
            const int e = e0 + lane;
            int64_t lo = 0, len = 0;
            if (e < p.E) {
                lo = clamp_i64(p.offsets[e], 0, R);
                const int64_t hi = clamp_i64(p.offsets[e + 1], 0, R);
                len = hi > lo ? hi - lo : 0;
            }
            const long long tiles = (len + BM - 1) / BM;
            const long long inc = wave_inclusive_scan(tiles);
            const long long excl = before + inc - tiles;
            const unsigned long long hit = __ballot(mt >= excl && mt < excl + tiles);
            if (hit) {
                const int src = __ffsll((long long)hit) - 1;
                const int64_t f_lo = wave_bcast(lo, src), f_len = wave_bcast(len, src);
                const int64_t f_excl = wave_bcast((int64_t)excl, src);
                t.expert = e0 + src;
                t.row0 = f_lo + (mt - f_excl) * BM;
                const int64_t left = f_lo + f_len - t.row0;
                t.rows_valid = (int)(left < BM ? left : BM);
                break;
            }
            before += wave_bcast(inc, kWave - 1);
        }
        return t;
    };

    // --------------------------------------------------------------- loaders
    // thread -> 16-byte chunk tid & 7 of rows tid >> 3 + 32 i (activations: 2 rows, weights: 8 rows)
    const int chunk = tid & 7;
    int xoff[XP], woff[WP];
#pragma unroll
    for (int i = 0; i < XP; ++i) xoff[i] = lds_off((tid >> 3) + i * (NT / 8), chunk);
#pragma unroll
    for (int i = 0; i < WP; ++i) woff[i] = BM * 128 + lds_off((tid >> 3) + i * (NT / 8), chunk);
    const int64_t a_row_bytes = p.a_stride_row * ESIZE;

    const uint8_t* xptr[XP];
    const uint8_t* wptr[WP];
    // row_index entries (or the rows themselves) of the rows this thread loads / of the rows whose
    // scales this lane applies
    auto fetch_rows = [&](const Tile& t, int64_t (&raw)[XP], int64_t (&sraw)[FM]) {
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int tr = (tid >> 3) + i * (NT / 8);
            const int64_t r = t.row0 + (tr < t.rows_valid ? tr : 0);
            raw[i] = p.row_index ? p.row_index[r] : r;
        }
        if constexpr (MSC) {
#pragma unroll
            for (int fm = 0; fm < FM; ++fm) {
                const int tr = fm * 32 + (lane & 31);
                const int64_t r = t.row0 + (tr < t.rows_valid ? tr : 0);
                sraw[fm] = p.row_index ? p.row_index[r] : r;
            }
        }
    };
    auto to_source = [&](int64_t v) -> int64_t {
        if (p.row_index) v = p.index_shift >= 0 ? (v >> p.index_shift) : v / p.index_div;
        return clamp_i64(v, 0, p.a_rows - 1);
    };
    auto make_ptrs = [&](const Tile& t, const int64_t (&raw)[XP]) {
        const uint8_t* a_base = p.a + (int64_t)t.expert * p.a_stride_e * ESIZE + chunk * 16;
#pragma unroll
        for (int i = 0; i < XP; ++i) xptr[i] = a_base + to_source(raw[i]) * a_row_bytes;
        const int n0 = t.nt * BN_OUT;
#pragma unroll
        for (int i = 0; i < WP; ++i) {
            const int wrow = (tid >> 3) + i * (NT / 8);
            const uint8_t* base = (SWIGLU && wrow >= BN / 2) ? p.b2 : p.b;
            int n = n0 + (SWIGLU && wrow >= BN / 2 ? wrow - BN / 2 : wrow);
            n = n < p.N ? n : p.N - 1;
            wptr[i] = base + ((int64_t)t.expert * p.b_se + (int64_t)n * p.b_sn) * ESIZE + chunk * 16;
        }
    };
    u32x4 xr[XP], wr[WP];
    const int Kdim = p.K;
    const int KT = (Kdim + BK - 1) / BK;
    auto load_global = [&](int kt) {
        const bool whole = (kt + 1) * BK <= Kdim;      // uniform: no per-lane predicate inside K
        const int k = kt * BK + chunk * CHUNK_ELEMS;
        if (whole) {        // (the uniform branch keeps the common case free of per-lane predicates)
#pragma unroll
            for (int i = 0; i < XP; ++i) xr[i] = *reinterpret_cast<const u32x4*>(xptr[i] + (int64_t)kt * 128);
#pragma unroll
            for (int i = 0; i < WP; ++i) wr[i] = *reinterpret_cast<const u32x4*>(wptr[i] + (int64_t)kt * 128);
        } else {
#pragma unroll
            for (int i = 0; i < XP; ++i)
                xr[i] = k < Kdim ? *reinterpret_cast<const u32x4*>(xptr[i] + (int64_t)kt * 128) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < WP; ++i)
                wr[i] = k < Kdim ? *reinterpret_cast<const u32x4*>(wptr[i] + (int64_t)kt * 128) : u32x4{0, 0, 0, 0};
        }
    };
    auto store_lds = [&](int stage) {
        uint8_t* st = smem + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < XP; ++i) *reinterpret_cast<u32x4*>(st + xoff[i]) = xr[i];
#pragma unroll
        for (int i = 0; i < WP; ++i) *reinterpret_cast<u32x4*>(st + woff[i]) = wr[i];
    };

    // MSC: E8M0 codes of the reciprocal scales: bytes 0, 1 the lane's rows of row blocks 0, 1,
    // bytes 2, 3 its columns of weight fragments 0, 1
    uint32_t sc = 0x7f7f7f7fu;
    auto fetch_scales = [&](const Tile& t, const int64_t (&sraw)[FM], float (&xs)[FM], float (&ws)[FN]) {
        if constexpr (MSC) {
#pragma unroll
            for (int fm = 0; fm < FM; ++fm) xs[fm] = p.a_scale[to_source(sraw[fm])];
            const int n0 = t.nt * BN_OUT;
#pragma unroll
            for (int fn = 0; fn < FN; ++fn) {
                const bool up = SWIGLU && fn >= FN / 2;
                int n = n0 + (SWIGLU ? wn * (TN / 2) + (fn % (FN / 2)) * 32 : wn * TN + fn * 32) + (lane & 31);
                n = n < p.N ? n : p.N - 1;
                ws[fn] = (up ? p.b2_scale : p.b_scale)[(int64_t)t.expert * p.N + n];
            }
        }
    };
    auto pack_scales = [&](const float (&xs)[FM], const float (&ws)[FN]) {
        if constexpr (MSC)
            sc = e8m0_of_reciprocal(xs[0]) | (e8m0_of_reciprocal(xs[1]) << 8) | (e8m0_of_reciprocal(ws[0]) << 16) |
                 (e8m0_of_reciprocal(ws[1]) << 24);
    };

    int wfrag_row[FN], xfrag_row[FM];
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
        const int r = SWIGLU ? (fn < FN / 2 ? 0 : BN / 2) + wn * (TN / 2) + (fn % (FN / 2)) * 32 : wn * TN + fn * 32;
        wfrag_row[fn] = r + (lane & 31);
    }
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) xfrag_row[fm] = fm * 32 + (lane & 31);

    // ------------------------------------------------------------- tile loop
    Tile cur = locate(xcd_begin + slot);
    {
        int64_t raw[XP], sraw[FM];
        float xs[FM], ws[FN];
        fetch_rows(cur, raw, sraw);
        make_ptrs(cur, raw);
        fetch_scales(cur, sraw, xs, ws);
        pack_scales(xs, ws);
    }
    load_global(0);
    for (int64_t j = slot; j < xcd_count; j += nslots) {
        const bool has_next = j + nslots < xcd_count;
        Tile nxt = cur;
        int64_t raw[XP], sraw[FM];
#pragma unroll
        for (int i = 0; i < XP; ++i) raw[i] = 0;
#pragma unroll
        for (int i = 0; i < FM; ++i) sraw[i] = 0;

        store_lds(0);
        __syncthreads();
        f32x16 acc[FN][FM];
#pragma unroll
        for (int i = 0; i < FN; ++i)
#pragma unroll
            for (int m = 0; m < FM; ++m)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][m][v] = 0.0f;

        auto multiply = [&](int st) __attribute__((always_inline)) {
            const uint8_t* sx = smem + st * STAGE_BYTES;
            const uint8_t* sw = sx + BM * 128;
            if constexpr (!FP8) {
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) {
                    const int ch = 2 * s4 + khalf;
                    bf16x8 wf[FN], xf[FM];
#pragma unroll
                    for (int fn = 0; fn < FN; ++fn)
                        wf[fn] = *reinterpret_cast<const bf16x8*>(sw + lds_off(wfrag_row[fn], ch));
#pragma unroll
                    for (int fm = 0; fm < FM; ++fm)
                        xf[fm] = *reinterpret_cast<const bf16x8*>(sx + lds_off(xfrag_row[fm], ch));
#pragma unroll
                    for (int fn = 0; fn < FN; ++fn)
#pragma unroll
                        for (int fm = 0; fm < FM; ++fm)
                            acc[fn][fm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[fn], xf[fm], acc[fn][fm], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2) {
                    const int ch = 4 * s2 + 2 * khalf;
                    i32x8 wf[FN], xf[FM];
#pragma unroll
                    for (int fn = 0; fn < FN; ++fn) {
                        const u32x4 lo = *reinterpret_cast<const u32x4*>(sw + lds_off(wfrag_row[fn], ch));
                        const u32x4 hi = *reinterpret_cast<const u32x4*>(sw + lds_off(wfrag_row[fn], ch + 1));
                        wf[fn] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                    }
#pragma unroll
                    for (int fm = 0; fm < FM; ++fm) {
                        const u32x4 lo = *reinterpret_cast<const u32x4*>(sx + lds_off(xfrag_row[fm], ch));
                        const u32x4 hi = *reinterpret_cast<const u32x4*>(sx + lds_off(xfrag_row[fm], ch + 1));
                        xf[fm] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                    }
                    if constexpr (MSC) {
                        // (the accumulator tied to the destination, as in the ring kernel: through the
                        // builtin it is a separate early-clobber operand and the kernel spills)
                        mfma_e4m3_scaled<2, 0>(wf[0], xf[0], acc[0][0], sc, sc);
                        mfma_e4m3_scaled<2, 1>(wf[0], xf[1], acc[0][1], sc, sc);
                        mfma_e4m3_scaled<3, 0>(wf[1], xf[0], acc[1][0], sc, sc);
                        mfma_e4m3_scaled<3, 1>(wf[1], xf[1], acc[1][1], sc, sc);
                    } else {
#pragma unroll
                        for (int fn = 0; fn < FN; ++fn)
#pragma unroll
                            for (int fm = 0; fm < FM; ++fm)
                                acc[fn][fm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[fn], xf[fm], acc[fn][fm], 0, 0, 0, 0, 0, 0);
                    }
                }
            }
        };
        // all slices but the last: fetch the next one, multiply this one, park the next one
        for (int kt = 0; kt + 1 < KT; ++kt) {
            const int st = kt & 1;
            load_global(kt + 1);
            multiply(st);
            store_lds(st ^ 1);
            __syncthreads();
        }
        if (has_next) {                     // the next tile: where it is, which rows it reads
            nxt = locate(xcd_begin + j + nslots);
            fetch_rows(nxt, raw, sraw);
        }
        multiply((KT - 1) & 1);
        if constexpr (MSC) mfma_results_guard();    // the last MFMAs' results are read by VALU code from here on
        __syncthreads();                    // every wave is done with the stages before the next tile fills stage 0

        // the next tile's first K-slice (and its scales) go out ahead of this tile's stores
        float xs[FM], ws[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i) xs[i] = 1.0f;
#pragma unroll
        for (int i = 0; i < FN; ++i) ws[i] = 1.0f;
        if (has_next) {
            make_ptrs(nxt, raw);
            load_global(0);
            fetch_scales(nxt, sraw, xs, ws);
        }
        gemm_epilogue<FM, FN, TM, TN, FP8, EPI, true, false, false, false, NoAfterStores, MSC>(
            p, acc, cur.expert, cur.nt * BN_OUT, cur.row0, cur.rows_valid, 0, wn, lane);
        if (has_next) pack_scales(xs, ws);
        cur = nxt;
    }
}

}  // namespace fmoe
