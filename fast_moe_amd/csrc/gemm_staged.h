// Register-staged grouped GEMM kernel: everything the ring and streaming kernels do not take.
#pragma once

#include "gemm_epilogue.h"

namespace fmoe {

// ----------------------------------------------------------- register-staged kernel
template <int BM_, int BN_, int WGM_, int WGN_>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
    static constexpr int NT = kWave * WGM * WGN;
    static constexpr int TM = BM / WGM, TN = BN / WGN;
    static constexpr int FM = TM / 32, FN = TN / 32;
    static constexpr int STAGE_BYTES = (BM + BN) * 128;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static_assert(TM % 32 == 0 && TN % 64 == 0, "wave tile must hold whole 32x32 fragments, FN even");
    static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "loader passes must be whole");
};

__device__ __forceinline__ int lds_off(int row, int chunk) {     // 128-byte rows
    return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4);
}

// DT: operand type, kDtBf16 / kDtE4m3 (bf16 output) or kDtF32 (fp32 operands, bias and output,
// v_mfma_f32_32x32x2_f32: full fp32 products, no tf32).
template <typename TL, int DT, int EPI, bool FAST, bool A_SILU>
__global__ __launch_bounds__(TL::NT) void grouped_gemm_kernel(const GemmParams p) {
    constexpr int BM = TL::BM, BN = TL::BN, NT = TL::NT;
    constexpr int FM = TL::FM, FN = TL::FN, TM = TL::TM, TN = TL::TN;
    constexpr bool FP8 = DT == kDtE4m3, F32 = DT == kDtF32;
    constexpr int ESIZE = FP8 ? 1 : (F32 ? 4 : 2);
    constexpr int CHUNK_ELEMS = 16 / ESIZE;         // elements per 16-byte chunk
    constexpr int BK = 128 / ESIZE;                 // elements per K-slice
    constexpr bool SWIGLU = EPI == FMOE_EPI_SWIGLU;
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;    // output columns per tile
    constexpr int XP = BM * 8 / NT, WP = BN * 8 / NT;

    extern __shared__ __align__(16) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % TL::WGM, wn = wave / TL::WGM;

    // ------------------------------------------------------------ scheduling
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
    const int64_t slot = blockIdx.x / kNumXcd;
    const int64_t group_span = (int64_t)kGroupM * p.n_tiles;
    int64_t group;
    int within;
    if (p.k_window) {
        // the cost of a tile follows its expert's contraction length, so contiguous tile ranges
        // per XCD would leave one XCD with the long experts: deal the groups out round-robin
        group = slot / group_span * kNumXcd + blockIdx.x % kNumXcd;
        within = (int)(slot % group_span);
    } else {
        if (slot >= per_xcd) return;
        const int64_t logical = (int64_t)(blockIdx.x % kNumXcd) * per_xcd + slot;
        if (logical >= total_tiles) return;
        group = logical / group_span;
        within = (int)(logical - group * group_span);
    }
    const int64_t first_m = group * kGroupM;
    if (first_m >= total_m) return;
    const int gsize = (int)(total_m - first_m < kGroupM ? total_m - first_m : kGroupM);
    if (within >= gsize * p.n_tiles) return;
    const int64_t mt = first_m + within % gsize;
    const int nt = within / gsize;

    int expert = 0;
    int64_t row0 = 0;
    int rows_valid = 0;
    {
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
            const bool mine = mt >= excl && mt < excl + tiles;
            const unsigned long long hit = __ballot(mine);
            if (hit) {
                const int src = __ffsll((long long)hit) - 1;
                const int64_t f_lo = wave_bcast(lo, src);
                const int64_t f_len = wave_bcast(len, src);
                const int64_t f_excl = wave_bcast((int64_t)excl, src);
                expert = e0 + src;
                row0 = f_lo + (mt - f_excl) * BM;
                const int64_t left = f_lo + f_len - row0;
                rows_valid = (int)(left < BM ? left : BM);
                break;
            }
            before += wave_bcast(inc, kWave - 1);
        }
    }
    if (rows_valid <= 0) return;   // unreachable for consistent offsets

    // per-expert contraction window (weight gradients): both operands start k_begin elements in
    int Kdim = p.K;
    int64_t k_begin = 0;
    if (p.k_window) {
        k_begin = p.k_window[expert];
        const int64_t span = p.k_window[expert + 1] - k_begin;
        Kdim = (int)(span < 0 ? 0 : (span < p.K ? span : p.K));
    }

    // --------------------------------------------------------------- loaders
    const uint8_t* a_base = p.a + ((int64_t)expert * p.a_stride_e + k_begin) * ESIZE;
    const int64_t a_row_bytes = p.a_stride_row * ESIZE;
    const int n0 = nt * BN_OUT;

    auto src_row_of = [&](int tile_row) -> int64_t {
        return source_row(p, row0 + (tile_row < rows_valid ? tile_row : 0));
    };
    // weight row (output column) behind LDS row `wrow`, and which matrix holds it
    auto w_row_of = [&](int wrow, const uint8_t*& base) -> int {
        int n;
        if (SWIGLU) {
            base = wrow < BN / 2 ? p.b : p.b2;
            n = n0 + (wrow < BN / 2 ? wrow : wrow - BN / 2);
        } else {
            base = p.b;
            n = n0 + wrow;
        }
        return n < p.N ? n : p.N - 1;
    };

    // FAST: thread -> (chunk = tid & 7, rows tid>>3 + i*NT/8); 16-byte global loads.
    // GENERIC: chunk id q = tid + i*NT, row = q % rows, chunk = q / rows; element loads
    // through arbitrary strides (adjacent lanes touch adjacent weight rows).
    const uint8_t* xptr[XP];
    const uint8_t* wptr[WP];
    int xoff[XP], woff[WP];     // LDS byte offsets inside a stage
    int xchunk[XP], wchunk[WP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        int row, chunk;
        if (FAST) { chunk = tid & 7; row = (tid >> 3) + i * (NT / 8); }
        else { const int q = tid + i * NT; row = q % BM; chunk = q / BM; }
        xptr[i] = a_base + src_row_of(row) * a_row_bytes;
        xoff[i] = lds_off(row, chunk);
        xchunk[i] = chunk;
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
        int row, chunk;
        if (FAST) { chunk = tid & 7; row = (tid >> 3) + i * (NT / 8); }
        else { const int q = tid + i * NT; row = q % BN; chunk = q / BN; }
        const uint8_t* base;
        const int n = w_row_of(row, base);
        wptr[i] = base + ((int64_t)expert * p.b_se + (int64_t)n * p.b_sn + k_begin * p.b_sk) * ESIZE;
        woff[i] = BM * 128 + lds_off(row, chunk);
        wchunk[i] = chunk;
    }

    u32x4 xr[XP], wr[WP];
    auto load_global = [&](int kt) {
        const bool whole = (kt + 1) * BK <= Kdim;      // uniform: no per-lane predicate inside K
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int k = kt * BK + xchunk[i] * CHUNK_ELEMS;
            if (FAST) {
                if (whole) xr[i] = *reinterpret_cast<const u32x4*>(xptr[i] + (int64_t)k * ESIZE);
                else xr[i] = k < Kdim ? *reinterpret_cast<const u32x4*>(xptr[i] + (int64_t)k * ESIZE)
                                     : u32x4{0, 0, 0, 0};
            } else {
                uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < CHUNK_ELEMS; ++j) {
                    uint32_t v = 0;
                    if (k + j < Kdim)
                        v = FP8 ? (uint32_t)xptr[i][k + j]
                            : F32 ? reinterpret_cast<const uint32_t*>(xptr[i])[k + j]
                                  : (uint32_t) reinterpret_cast<const uint16_t*>(xptr[i])[k + j];
                    w[(j * ESIZE) >> 2] |= v << (8 * ((j * ESIZE) & 3));
                }
                xr[i] = u32x4{w[0], w[1], w[2], w[3]};
            }
            if (A_SILU) xr[i] = F32 ? silu_f32x4(xr[i]) : silu_bf16x8(xr[i]);
        }
#pragma unroll
        for (int i = 0; i < WP; ++i) {
            const int k = kt * BK + wchunk[i] * CHUNK_ELEMS;
            if (FAST) {
                if (whole) wr[i] = *reinterpret_cast<const u32x4*>(wptr[i] + (int64_t)k * ESIZE);
                else wr[i] = k < Kdim ? *reinterpret_cast<const u32x4*>(wptr[i] + (int64_t)k * ESIZE)
                                     : u32x4{0, 0, 0, 0};
            } else {
                uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < CHUNK_ELEMS; ++j) {
                    uint32_t v = 0;
                    if (k + j < Kdim) {
                        const int64_t off = (int64_t)(k + j) * p.b_sk;
                        v = FP8 ? (uint32_t)wptr[i][off]
                            : F32 ? reinterpret_cast<const uint32_t*>(wptr[i])[off]
                                  : (uint32_t) reinterpret_cast<const uint16_t*>(wptr[i])[off];
                    }
                    w[(j * ESIZE) >> 2] |= v << (8 * ((j * ESIZE) & 3));
                }
                wr[i] = u32x4{w[0], w[1], w[2], w[3]};
            }
        }
    };
    auto store_lds = [&](int stage) {
        uint8_t* s = smem + stage * TL::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < XP; ++i) *reinterpret_cast<u32x4*>(s + xoff[i]) = xr[i];
#pragma unroll
        for (int i = 0; i < WP; ++i) *reinterpret_cast<u32x4*>(s + woff[i]) = wr[i];
    };

    // ------------------------------------------------------------- main loop
    f32x16 acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // LDS row of weight fragment fn / activation fragment fm for this lane
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
    const int khalf = lane >> 5;

    const int KT = (Kdim + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) load_global(kt + 1);
        const uint8_t* sx = smem + cur * TL::STAGE_BYTES;
        const uint8_t* sw = sx + BM * 128;
        if (F32) {
            // a 16-byte chunk holds 4 consecutive k of one row; MFMA j of a chunk pair contracts
            // element j of the low-half lanes' chunk with element j of the high-half lanes' chunk
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int chunk = 2 * s + khalf;
                u32x4 wf[FN], xf[FM];
#pragma unroll
                for (int fn = 0; fn < FN; ++fn)
                    wf[fn] = *reinterpret_cast<const u32x4*>(sw + lds_off(wfrag_row[fn], chunk));
#pragma unroll
                for (int fm = 0; fm < FM; ++fm)
                    xf[fm] = *reinterpret_cast<const u32x4*>(sx + lds_off(xfrag_row[fm], chunk));
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int fn = 0; fn < FN; ++fn)
#pragma unroll
                        for (int fm = 0; fm < FM; ++fm)
                            acc[fn][fm] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                                __uint_as_float(wf[fn][j]), __uint_as_float(xf[fm][j]), acc[fn][fm], 0, 0, 0);
            }
        } else if (!FP8) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int chunk = 2 * s + khalf;
                bf16x8 wf[FN], xf[FM];
#pragma unroll
                for (int fn = 0; fn < FN; ++fn)
                    wf[fn] = *reinterpret_cast<const bf16x8*>(sw + lds_off(wfrag_row[fn], chunk));
#pragma unroll
                for (int fm = 0; fm < FM; ++fm)
                    xf[fm] = *reinterpret_cast<const bf16x8*>(sx + lds_off(xfrag_row[fm], chunk));
#pragma unroll
                for (int fn = 0; fn < FN; ++fn)
#pragma unroll
                    for (int fm = 0; fm < FM; ++fm)
                        acc[fn][fm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[fn], xf[fm], acc[fn][fm], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const int chunk = 4 * s + 2 * khalf;
                i32x8 wf[FN], xf[FM];
#pragma unroll
                for (int fn = 0; fn < FN; ++fn) {
                    const u32x4 lo = *reinterpret_cast<const u32x4*>(sw + lds_off(wfrag_row[fn], chunk));
                    const u32x4 hi = *reinterpret_cast<const u32x4*>(sw + lds_off(wfrag_row[fn], chunk + 1));
                    wf[fn] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
                                   (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                }
#pragma unroll
                for (int fm = 0; fm < FM; ++fm) {
                    const u32x4 lo = *reinterpret_cast<const u32x4*>(sx + lds_off(xfrag_row[fm], chunk));
                    const u32x4 hi = *reinterpret_cast<const u32x4*>(sx + lds_off(xfrag_row[fm], chunk + 1));
                    xf[fm] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
                                   (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                }
#pragma unroll
                for (int fn = 0; fn < FN; ++fn)
#pragma unroll
                    for (int fm = 0; fm < FM; ++fm)
                        acc[fn][fm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            wf[fn], xf[fm], acc[fn][fm], 0, 0, 0, 0, 0, 0);
            }
        }
        if (kt + 1 < KT) store_lds(cur ^ 1);
        __syncthreads();
    }

    if constexpr (F32)
        gemm_epilogue_f32<FM, FN, TM, TN, EPI>(p, acc, expert, n0, row0, rows_valid, wm, wn, lane);
    else
        gemm_epilogue<FM, FN, TM, TN, FP8, EPI>(p, acc, expert, n0, row0, rows_valid, wm, wn, lane);
}

}  // namespace fmoe
