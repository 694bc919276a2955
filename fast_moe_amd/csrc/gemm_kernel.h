// Jagged ("grouped") GEMM for gfx950: out[rows of expert e] = A[gather] x B[e],
// bf16 or OCP-e4m3 operands, fp32 MFMA accumulation, fused bias / SiLU / SwiGLU
// epilogue.  Shared by gemm_bf16.hip and gemm_fp8.hip.
//
// Mapping to the hardware
//   * A tile is BM activation rows x BN weight rows; both operands are staged as
//     128-byte K-slices per row (64 bf16 or 128 e4m3) in double-buffered LDS,
//     16-byte chunks XOR-swizzled by (row >> 1) & 7 so that the ds_read_b128 of
//     an MFMA fragment and the ds_write_b128 of the loader spread over all banks.
//   * The weights feed the MFMA "A" port and the activations the "B" port
//     (v_mfma_f32_32x32x16_bf16 / v_mfma_f32_32x32x64_f8f6f4), so each lane ends
//     up with 4 consecutive output columns of one output row per register quad
//     and stores them as one 8-byte write.
//   * Activation rows are gathered through row_index while loading (no [R, K]
//     copy); rows past the end of an expert segment re-read the tile's first row
//     and are masked at the store.
//   * Scheduling is on the device: every block derives the number of row tiles
//     per expert from `offsets` with a wavefront prefix scan, so no max_seq_len
//     and no host synchronisation are needed, skewed and empty experts cost
//     nothing, and the grid is only an upper bound.  Block ids are dealt
//     round-robin to the 8 XCDs by the hardware; id -> tile is remapped so that
//     each XCD works on a contiguous range of tiles (group-of-4 row tiles x all
//     column tiles), which keeps the shared A rows / B rows in that XCD's L2.
#pragma once

#include "common.h"

namespace fmoe {

struct GemmParams {
    const int64_t* offsets;
    const int64_t* row_index;
    int E, N, K, index_div;
    int64_t total_rows, a_rows;
    const uint8_t* a;
    int64_t a_stride_row, a_stride_e;   // elements
    const float* a_scale;
    const uint8_t* b;
    const uint8_t* b2;
    int64_t b_se, b_sk, b_sn;           // elements
    const float* b_scale;
    const float* b2_scale;
    const uint16_t* bias;
    const uint16_t* bias2;
    int64_t bias_se;
    uint16_t* out;
    int64_t out_stride;
    int n_tiles;
    int vec_store;                      // 8-byte stores of 4 bf16 are legal
};

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

constexpr int kGroupM = 4;   // row tiles per scheduling group
constexpr int kNumXcd = 8;

__device__ __forceinline__ int lds_off(int row, int chunk) {
    return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4);
}

__device__ __forceinline__ int64_t clamp_i64(int64_t v, int64_t lo, int64_t hi) {
    return v < lo ? lo : (v > hi ? hi : v);
}

// SiLU on 8 packed bf16 with the rounding of F.silu on a bf16 tensor
__device__ __forceinline__ u32x4 silu_bf16x8(u32x4 v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = round_bf16(silu_f32(bf16_bits_to_f32(v[j] & 0xffffu)));
        const float hi = round_bf16(silu_f32(__uint_as_float(v[j] & 0xffff0000u)));
        v[j] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
    }
    return v;
}

template <typename TL, bool FP8, int EPI, bool FAST, bool A_SILU>
__global__ __launch_bounds__(TL::NT) void grouped_gemm_kernel(const GemmParams p) {
    constexpr int BM = TL::BM, BN = TL::BN, NT = TL::NT;
    constexpr int FM = TL::FM, FN = TL::FN, TM = TL::TM, TN = TL::TN;
    constexpr int ESIZE = FP8 ? 1 : 2;
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
    if (slot >= per_xcd) return;
    const int64_t logical = (int64_t)(blockIdx.x % kNumXcd) * per_xcd + slot;
    if (logical >= total_tiles) return;
    const int64_t group_span = (int64_t)kGroupM * p.n_tiles;
    const int64_t group = logical / group_span;
    const int64_t first_m = group * kGroupM;
    const int gsize = (int)(total_m - first_m < kGroupM ? total_m - first_m : kGroupM);
    const int within = (int)(logical - group * group_span);
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

    // --------------------------------------------------------------- loaders
    const uint8_t* a_base = p.a + (int64_t)expert * p.a_stride_e * ESIZE;
    const int64_t a_row_bytes = p.a_stride_row * ESIZE;
    const int n0 = nt * BN_OUT;

    auto src_row_of = [&](int tile_row) -> int64_t {
        const int64_t r = row0 + (tile_row < rows_valid ? tile_row : 0);
        int64_t s = r;
        if (p.row_index) s = p.row_index[r] / p.index_div;
        return clamp_i64(s, 0, p.a_rows - 1);
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
        wptr[i] = base + ((int64_t)expert * p.b_se + (int64_t)n * p.b_sn) * ESIZE;
        woff[i] = BM * 128 + lds_off(row, chunk);
        wchunk[i] = chunk;
    }

    u32x4 xr[XP], wr[WP];
    auto load_global = [&](int kt) {
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int k = kt * BK + xchunk[i] * CHUNK_ELEMS;
            if (FAST) {
                xr[i] = k < p.K ? *reinterpret_cast<const u32x4*>(xptr[i] + (int64_t)k * ESIZE)
                                : u32x4{0, 0, 0, 0};
            } else {
                uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < CHUNK_ELEMS; ++j) {
                    uint32_t v = 0;
                    if (k + j < p.K)
                        v = FP8 ? (uint32_t)xptr[i][k + j]
                                : (uint32_t) reinterpret_cast<const uint16_t*>(xptr[i])[k + j];
                    w[(j * ESIZE) >> 2] |= v << (8 * ((j * ESIZE) & 3));
                }
                xr[i] = u32x4{w[0], w[1], w[2], w[3]};
            }
            if (A_SILU) xr[i] = silu_bf16x8(xr[i]);
        }
#pragma unroll
        for (int i = 0; i < WP; ++i) {
            const int k = kt * BK + wchunk[i] * CHUNK_ELEMS;
            if (FAST) {
                wr[i] = k < p.K ? *reinterpret_cast<const u32x4*>(wptr[i] + (int64_t)k * ESIZE)
                                : u32x4{0, 0, 0, 0};
            } else {
                uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < CHUNK_ELEMS; ++j) {
                    uint32_t v = 0;
                    if (k + j < p.K) {
                        const int64_t off = (int64_t)(k + j) * p.b_sk;
                        v = FP8 ? (uint32_t)wptr[i][off]
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

    const int KT = (p.K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) load_global(kt + 1);
        const uint8_t* sx = smem + cur * TL::STAGE_BYTES;
        const uint8_t* sw = sx + BM * 128;
        if (!FP8) {
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

    // -------------------------------------------------------------- epilogue
    // Register quad g of fragment (fn, fm) holds output columns nb .. nb+3 of row
    // (lane & 31) of the fragment.  Per-column data (weight descale, bias) is
    // fetched once per quad and reused over the FM row fragments.
    constexpr int FN_OUT = SWIGLU ? FN / 2 : FN;
    const int64_t bias_row = (int64_t)expert * p.bias_se;
    float rsa[FM];
    bool row_ok[FM];
    uint16_t* orow[FM];
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
        const int tile_row = wm * TM + fm * 32 + (lane & 31);
        row_ok[fm] = tile_row < rows_valid;
        orow[fm] = p.out + (row0 + tile_row) * p.out_stride;
        rsa[fm] = FP8 ? 1.0f / p.a_scale[src_row_of(tile_row)] : 1.0f;
    }
#pragma unroll
    for (int fn = 0; fn < FN_OUT; ++fn) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int nb = n0 + (SWIGLU ? wn * (TN / 2) : wn * TN) + fn * 32 + 8 * g + 4 * khalf;
            float rsw[4], rsw2[4], bv[4], bv2[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int nc = nb + j < p.N ? nb + j : p.N - 1;
                rsw[j] = FP8 ? 1.0f / p.b_scale[(int64_t)expert * p.N + nc] : 1.0f;
                rsw2[j] = (FP8 && SWIGLU) ? 1.0f / p.b2_scale[(int64_t)expert * p.N + nc] : 1.0f;
                bv[j] = p.bias ? bf16_bits_to_f32(p.bias[bias_row + nc]) : 0.0f;
                bv2[j] = (SWIGLU && p.bias2) ? bf16_bits_to_f32(p.bias2[bias_row + nc]) : 0.0f;
            }
#pragma unroll
            for (int fm = 0; fm < FM; ++fm) {
                uint32_t packed[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float y = acc[fn][fm][4 * g + j];
                    float y2 = SWIGLU ? acc[fn + FN / 2][fm][4 * g + j] : 0.0f;
                    if (FP8) {
                        // (acc / (sa * sw)) rounded to bf16, then the bias added in bf16
                        y = round_bf16(y * (rsa[fm] * rsw[j]));
                        if (p.bias) y = round_bf16(y + bv[j]);
                        if (SWIGLU) {
                            y2 = round_bf16(y2 * (rsa[fm] * rsw2[j]));
                            if (p.bias2) y2 = round_bf16(y2 + bv2[j]);
                        }
                    } else {
                        y = round_bf16(y + bv[j]);
                        if (SWIGLU) y2 = round_bf16(y2 + bv2[j]);
                    }
                    if (EPI == FMOE_EPI_SILU) y = fast_silu_f32(y);
                    if (SWIGLU) y = round_bf16(fast_silu_f32(y)) * y2;
                    packed[j] = f32_to_bf16_bits(y);
                }
                if (!row_ok[fm]) continue;
                if (p.vec_store && nb + 3 < p.N) {
                    u32x2 o;
                    o[0] = packed[0] | (packed[1] << 16);
                    o[1] = packed[2] | (packed[3] << 16);
                    *reinterpret_cast<u32x2*>(orow[fm] + nb) = o;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (nb + j < p.N) orow[fm][nb + j] = (uint16_t)packed[j];
                }
            }
        }
    }
}

// ------------------------------------------------------------------- host side
typedef TileCfg<256, 256, 2, 4> TileBig;     // 8 waves, wave tile 128 x 64
typedef TileCfg<64, 256, 1, 4> TileSmall;    // 4 waves, wave tile 64 x 64

template <typename TL, bool FP8, int EPI, bool FAST, bool A_SILU>
int launch_gemm(GemmParams p, hipStream_t stream) {
    constexpr int bn_out = EPI == FMOE_EPI_SWIGLU ? TL::BN / 2 : TL::BN;
    p.n_tiles = (p.N + bn_out - 1) / bn_out;
    auto kern = grouped_gemm_kernel<TL, FP8, EPI, FAST, A_SILU>;
    static bool attr_done = false;
    if (!attr_done) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, TL::LDS_BYTES);
        if (err != hipSuccess)
            return fail(FMOE_ERR_LAUNCH, "fmoe_grouped_gemm: cannot reserve %d B of LDS: %s", TL::LDS_BYTES,
                        hipGetErrorString(err));
        attr_done = true;
    }
    const int64_t max_m_tiles = p.total_rows / TL::BM + p.E;
    const int64_t max_tiles = max_m_tiles * p.n_tiles;
    const int64_t grid = (max_tiles + kNumXcd - 1) / kNumXcd * kNumXcd;
    if (grid >= ((int64_t)1 << 31)) return fail(FMOE_ERR_UNSUPPORTED, "fmoe_grouped_gemm: grid too large");
    kern<<<(unsigned)grid, TL::NT, TL::LDS_BYTES, stream>>>(p);
    return check_launch("fmoe_grouped_gemm");
}

template <bool FP8, int EPI, bool A_SILU>
int dispatch_tile(const GemmParams& p, bool fast, bool big, hipStream_t stream) {
    if (!fast) return launch_gemm<TileSmall, FP8, EPI, false, A_SILU>(p, stream);
    if (big) return launch_gemm<TileBig, FP8, EPI, true, A_SILU>(p, stream);
    return launch_gemm<TileSmall, FP8, EPI, true, A_SILU>(p, stream);
}

// Entry points of the two translation units.
int run_gemm_bf16(GemmParams& p, int epilogue, bool a_silu, bool fast, bool big, hipStream_t stream);
int run_gemm_fp8(GemmParams& p, int epilogue, bool fast, bool big, hipStream_t stream);

}  // namespace fmoe
