// Host side of the grouped GEMM: tile configurations, kernel choice, launches.
#pragma once

#include "gemm_ring.h"
#include "gemm_staged.h"
#include "gemm_stream.h"

namespace fmoe {

// ------------------------------------------------------------------- host side
typedef TileCfg<256, 256, 2, 4> TileBig;        // 8 waves, wave tile 128 x 64
typedef TileCfg<64, 256, 1, 4> TileSmall;       // 4 waves, wave tile 64 x 64
typedef RingCfg<256, 256, 2, 4, 0> TileRing4;   // 8 waves, wave tile 128 x 64, 4-slot ring, LDS tables
typedef RingCfg<256, 256, 2, 4, 1> TileRing5;   // 5-slot ring, paired slices, E <= 64
// The plain forward calls take TileRing5F.  A build with -DFMOE_RING_NARROW gives them 256 x 128 tiles
// of 4 waves (one wave per SIMD, half the accumulator footprint per CU) instead: a measurement
// variant, kept so that the comparison can be repeated; 16-25 % slower than the 8-wave tile.
#ifdef FMOE_RING_NARROW
typedef RingCfg<256, 128, 2, 2, 1> TileRing5F;
#else
typedef TileRing5 TileRing5F;
#endif
typedef RingCfg<256, 256, 2, 4, 2> TileRing5M;  // 5-slot ring, paired slices, E <= 128 (the plain forward calls)
typedef RingCfg<256, 256, 2, 4, 4> TileRing5W;  // 5-slot ring, paired slices, E <= 256

enum GemmKernelSel { kSelRing = 0, kSelStagedBig = 1, kSelStagedSmall = 2, kSelGeneric = 3 };

template <typename Kern>
int reserve_lds(Kern kern, int bytes, bool& done) {
    if (done) return FMOE_OK;
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (err != hipSuccess)
        return fail(FMOE_ERR_LAUNCH, "fmoe_grouped_gemm: cannot reserve %d B of LDS: %s", bytes,
                    hipGetErrorString(err));
    done = true;
    return FMOE_OK;
}

template <typename TL, int DT, int EPI, bool FAST, bool A_SILU>
int launch_gemm(GemmParams p, hipStream_t stream) {
    constexpr int bn_out = EPI == FMOE_EPI_SWIGLU ? TL::BN / 2 : TL::BN;
    p.n_tiles = (p.N + bn_out - 1) / bn_out;
    auto kern = grouped_gemm_kernel<TL, DT, EPI, FAST, A_SILU>;
    static bool attr_done = false;
    if (int rc = reserve_lds(kern, TL::LDS_BYTES, attr_done)) return rc;
    const int64_t max_m_tiles = p.total_rows / TL::BM + p.E;
    const int64_t max_tiles = max_m_tiles * p.n_tiles;
    int64_t grid = (max_tiles + kNumXcd - 1) / kNumXcd * kNumXcd;
    if (p.k_window) {      // whole groups of kGroupM row tiles per XCD, round-robin
        const int64_t groups = (max_m_tiles + kGroupM - 1) / kGroupM;
        grid = (groups + kNumXcd - 1) / kNumXcd * kNumXcd * kGroupM * p.n_tiles;
    }
    if (grid >= ((int64_t)1 << 31)) return fail(FMOE_ERR_UNSUPPORTED, "fmoe_grouped_gemm: grid too large");
    kern<<<(unsigned)grid, TL::NT, TL::LDS_BYTES, stream>>>(p);
    return check_launch("fmoe_grouped_gemm");
}

int compute_units();   // CUs of the current device (gemm_api.hip)
int lds_per_block();   // largest LDS allocation of one block on the current device (gemm_api.hip)

// the streaming kernel takes what the 64-row register-staged kernel takes with 16-byte loads, when
// the output can be stored 16 bytes at a time and no contraction window is set
inline bool stream_kernel_takes(const GemmParams& p) { return p.vec_store && !p.k_window; }

template <int DT, int EPI>
int launch_stream(GemmParams p, hipStream_t stream) {
    constexpr int bn_out = EPI == FMOE_EPI_SWIGLU ? 128 : 256;
    constexpr int lds_bytes = 2 * (64 + 256) * 128;
    p.n_tiles = (p.N + bn_out - 1) / bn_out;
    const int64_t max_tiles = (p.total_rows / 64 + p.E) * p.n_tiles;
    // two blocks per CU (80 KB of LDS each), a multiple of the XCD count; fewer when the launch is small
    int64_t grid = 2 * (int64_t)(compute_units() / kNumXcd * kNumXcd);
    if (grid < kNumXcd) grid = kNumXcd;
    const int64_t need = (max_tiles + kNumXcd - 1) / kNumXcd * kNumXcd;
    if (need < grid) grid = need;
    auto go = [&](auto kern, bool& attr_done) -> int {
        if (int rc = reserve_lds(kern, lds_bytes, attr_done)) return rc;
        kern<<<(unsigned)grid, 256, lds_bytes, stream>>>(p);
        return check_launch("fmoe_grouped_gemm");
    };
    if constexpr (DT == kDtE4m3) {
        if (p.scale_pow2) {
            static bool done_msc = false;
            return go(grouped_gemm_stream_kernel<DT, EPI, true>, done_msc);
        }
    }
    static bool done = false;
    return go(grouped_gemm_stream_kernel<DT, EPI, false>, done);
}

template <typename TL, bool FP8, int EPI, bool WTR = false, bool KWIN = false, bool XTR = false, bool MSC = false>
int launch_ring_cfg(GemmParams p, hipStream_t stream) {
    constexpr int bn_out = EPI == FMOE_EPI_SWIGLU ? TL::BN / 2 : TL::BN;
    p.n_tiles = (p.N + bn_out - 1) / bn_out;
    if (TL::PAIR) {
        // (tile numbers run up to the row tiles rounded up to a round of kNumXcd groups)
        if ((p.total_rows / TL::BM + p.E + (kNumXcd + 1) * kGroupM) * (int64_t)p.n_tiles >= ((int64_t)1 << 31))
            return fail(FMOE_ERR_UNSUPPORTED, "fmoe_grouped_gemm: more than 2^31 output tiles");
        magic_u31((int64_t)kGroupM * p.n_tiles, &p.group_magic, &p.group_magic_shift);
        // A tile that runs the shortened main loop gets ahead of the tiles of its group, which read
        // the same weights, by about 0.2 us per K-slice; a line lives about 10 us in an XCD's L2.
        // Up to 64 slices the group keeps sharing its fills and the shortened loop pays (forward
        // GEMMs of 64 experts -0.6 %, e4m3 at 128 experts -2.4 %); with 128 slices (K = 4096 in bf16,
        // 2048 rows per expert) the fills it breaks cost more than it saves (GEMM1 +1.8 %).
        // With two row tiles or fewer per expert on average there is little sharing to break, and the
        // second tile of most experts is a short one: the shortened loop stays on whatever K is.
        p.short_tile_rows = (p.K / (FP8 ? 64 : 32) <= 64 || p.total_rows / p.E <= 2 * TL::BM) ? TL::BM / 2 : 0;
    }
    auto kern = grouped_gemm_ring_kernel<TL, FP8, EPI, WTR, KWIN, XTR, MSC>;
    static bool attr_done = false;
    if (int rc = reserve_lds(kern, TL::LDS_BYTES, attr_done)) return rc;
    // persistent: one block per CU (the LDS footprint admits no second one), a multiple of
    // the XCD count so that every XCD owns the same number of blocks
    int grid = compute_units() / kNumXcd * kNumXcd;
    if (grid < kNumXcd) grid = kNumXcd;
    kern<<<(unsigned)grid, TL::NT, TL::LDS_BYTES, stream>>>(p);
    return check_launch("fmoe_grouped_gemm");
}

// The 5-slot ring needs every byte of a 160 KB LDS, an even number of K-slices per tile,
// row numbers that fit 32 bits and few enough experts for the register tables.
template <bool FP8, int EPI>
int launch_ring(const GemmParams& p, hipStream_t stream) {
    const int slices = p.K / (FP8 ? 64 : 32);
    const bool pair_ok = slices % 2 == 0 && slices >= 4 && p.total_rows < ((int64_t)1 << 31) &&
                         lds_per_block() >= TileRing5::LDS_BYTES;
    // contraction windows: only the paired ring follows them, and only whole pairs of slices
    const int pair_elems = FP8 ? 128 : 64;
    const bool window_ok = !p.k_window || (p.k_window_multiple >= pair_elems && p.k_window_multiple % pair_elems == 0);
    if (p.a_sk != 1) {                     // both operands row-indexed (the caller checked the rest)
        if constexpr (!FP8 && EPI == FMOE_EPI_NONE) {
            if (p.E <= TileRing5::kMaxExperts) return launch_ring_cfg<TileRing5, FP8, EPI, true, true, true>(p, stream);
            return launch_ring_cfg<TileRing5W, FP8, EPI, true, true, true>(p, stream);
        }
        return fail(FMOE_ERR_UNSUPPORTED, "fmoe_grouped_gemm: row-indexed operands need bf16 and no epilogue");
    }
    if (p.b_sn == 1 && p.b_sk != 1) {      // N-contiguous weights in place (the caller checked pair_ok's terms)
        if constexpr (!FP8) {
            if (p.E <= TileRing5::kMaxExperts) return launch_ring_cfg<TileRing5, FP8, EPI, true>(p, stream);
            return launch_ring_cfg<TileRing5W, FP8, EPI, true>(p, stream);
        }
        return fail(FMOE_ERR_UNSUPPORTED, "fmoe_grouped_gemm: no in-place path for these weights");
    }
    if (p.k_window) {                      // built for the weight gradient: bf16, no epilogue
        if constexpr (!FP8 && EPI == FMOE_EPI_NONE) {
            if (pair_ok && window_ok && p.E <= TileRing5::kMaxExperts)
                return launch_ring_cfg<TileRing5, FP8, EPI, false, true>(p, stream);
            if (pair_ok && window_ok && p.E <= TileRing5W::kMaxExperts)
                return launch_ring_cfg<TileRing5W, FP8, EPI, false, true>(p, stream);
        }
        return launch_gemm<TileBig, FP8 ? kDtE4m3 : kDtBf16, EPI, true, false>(p, stream);
    }
    if constexpr (FP8) {                   // power-of-two scales: applied by the MFMAs (row numbers fit 31 bits: pair_ok)
        if (p.scale_pow2 && pair_ok && p.E <= TileRing5::kMaxExperts)
            return launch_ring_cfg<TileRing5F, FP8, EPI, false, false, false, true>(p, stream);
        if (p.scale_pow2 && pair_ok && p.E <= TileRing5M::kMaxExperts)
            return launch_ring_cfg<TileRing5M, FP8, EPI, false, false, false, true>(p, stream);
        if (p.scale_pow2 && pair_ok && p.E <= TileRing5W::kMaxExperts)
            return launch_ring_cfg<TileRing5W, FP8, EPI, false, false, false, true>(p, stream);
    }
    if (pair_ok && p.E <= TileRing5::kMaxExperts) return launch_ring_cfg<TileRing5F, FP8, EPI>(p, stream);
    if (pair_ok && p.E <= TileRing5M::kMaxExperts) return launch_ring_cfg<TileRing5M, FP8, EPI>(p, stream);
    if (pair_ok && p.E <= TileRing5W::kMaxExperts) return launch_ring_cfg<TileRing5W, FP8, EPI>(p, stream);
    return launch_ring_cfg<TileRing4, FP8, EPI>(p, stream);
}

template <int DT, int EPI, bool A_SILU>
int dispatch_tile(const GemmParams& p, int sel, hipStream_t stream) {
    switch (sel) {
        case kSelRing:
            if constexpr (!A_SILU && DT != kDtF32) return launch_ring<DT == kDtE4m3, EPI>(p, stream);
            else return launch_gemm<TileBig, DT, EPI, true, A_SILU>(p, stream);
        case kSelStagedBig: return launch_gemm<TileBig, DT, EPI, true, A_SILU>(p, stream);
        case kSelStagedSmall:
            if constexpr (!A_SILU && DT != kDtF32 && EPI != FMOE_EPI_GATED) {
                if (stream_kernel_takes(p)) return launch_stream<DT, EPI>(p, stream);
            }
            return launch_gemm<TileSmall, DT, EPI, true, A_SILU>(p, stream);
        default: return launch_gemm<TileSmall, DT, EPI, false, A_SILU>(p, stream);
    }
}

// Entry points of the translation units (one per operand type).
int run_gemm_bf16(GemmParams& p, int epilogue, bool a_silu, int sel, hipStream_t stream);
int run_gemm_fp8(GemmParams& p, int epilogue, int sel, hipStream_t stream);
int run_gemm_f32(GemmParams& p, int epilogue, bool a_silu, int sel, hipStream_t stream);

}  // namespace fmoe
