// Launch parameters of the grouped GEMM kernels and the small device helpers they share.
#pragma once

#include "common.h"
#include <cstdlib>
#include <type_traits>

namespace fmoe {


typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

struct GemmParams {
    const int64_t* offsets;
    const int64_t* row_index;
    int E, N, K, index_div;
    int index_shift;                    // log2(index_div) when it is a power of two, else -1
    // otherwise, for 0 <= v < 2^31: v / index_div == mulhi(v, index_magic) >> index_magic_shift
    // (magic = ceil(2^p / d), p = 31 + ceil(log2 d): the error of the product stays below 2^p)
    uint32_t index_magic;
    int index_magic_shift;
    // the same for the tile scheduler of the paired ring: v / (kGroupM * n_tiles) for v < 2^31
    uint32_t group_magic;
    int group_magic_shift;
    int64_t total_rows, a_rows;
    const uint8_t* a;
    int64_t a_stride_row, a_stride_e;   // elements
    int64_t a_sk;                       // element stride of A along k (1 unless A is given transposed)
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
    int vec_store;                      // 16-byte stores of 8 bf16 are legal
    int scale_vec;                      // e4m3: 16-byte loads of 4 weight scales are legal
    int scale_pow2;                     // e4m3: the caller promises that every scale is an exact power of two
    int gate_vec;                       // GATED: 8-byte loads of 4 gate values are legal
    int gate_vec16;                     // GATED: 16-byte loads of 8 gate values are legal
    int short_tile_rows;                // paired ring: tiles with at most this many valid rows run the shortened
                                        // main loop (BM / 2, or 0: never)
    const int64_t* k_window;            // [E+1] per-expert contraction range, or null
    int k_window_multiple;              // every window is a multiple of this and at least twice it (0: unknown)
    uint16_t* aux;                      // SWIGLU: the two pre-activations, or null
    uint16_t* aux2;
    int64_t aux_stride;
    uint16_t* out2;                     // XTR: rows [out_half, 2 * out_half) of every expert's result go here, or null
    int64_t out_half;
    const uint8_t* a2;                  // second product a2 * b2 summed into the same output, or null
    int k_split;                        // ... whose contraction covers k in [k_split, K)
#ifdef FMOE_TRACE
    uint64_t* trace;                    // debug builds: per-tile time stamps of the ring kernel
#endif
};

#ifdef FMOE_TRACE
// Debug builds (-DFMOE_TRACE): wave 0 and wave NW/2 of every block record real-time stamps (100 MHz)
// per tile into p.trace, two planes of [block][tile < 32][wave group][8]: plane 0 = tile start, end
// of the main loop, next tile located, epilogue done, shader clock at start and end, K-slices, valid
// rows; plane 1 = after the first four double steps, before and after the second last one.
#define FMOE_TRACE_STAMP(slot_)                                                                   \
    do {                                                                                         \
        if (p.trace && tile_i < 32 && (wave == 0 || wave == NW / 2))                             \
            tstamp[slot_] = __builtin_amdgcn_s_memrealtime();                                    \
    } while (0)
#else
#define FMOE_TRACE_STAMP(slot_) do {} while (0)
#endif

constexpr int kDtBf16 = 0, kDtE4m3 = 1, kDtF32 = 2;
constexpr int kGroupM = 4;   // row tiles per scheduling group
constexpr int kNumXcd = 8;

__device__ __forceinline__ int64_t clamp_i64(int64_t v, int64_t lo, int64_t hi) {
    return v < lo ? lo : (v > hi ? hi : v);
}

// two consecutive int64 from a wave-uniform address through the scalar cache (read only)
__device__ __forceinline__ void scalar_load_i64x2(const int64_t* ptr, int64_t& a, int64_t& b) {
    typedef __attribute__((ext_vector_type(4))) int i32x4;
    i32x4 v;
    asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(ptr) : "memory");
    a = (int64_t)(((uint64_t)(uint32_t)v[1] << 32) | (uint32_t)v[0]);
    b = (int64_t)(((uint64_t)(uint32_t)v[3] << 32) | (uint32_t)v[2]);
}

// row_index value -> source row, for values below 2^31 (the paired ring: total_rows < 2^31): a
// shift or one multiply by wave-uniform constants, no division sequence and nothing per lane for
// the compiler to keep across the tile loop.  Negative (malformed) values give some row; the
// callers clamp.
__device__ __forceinline__ int32_t div_index32(const GemmParams& p, int32_t v) {
    if (p.index_shift >= 0) return v >> p.index_shift;
    return (int32_t)(__umulhi((uint32_t)v, p.index_magic) >> p.index_magic_shift);
}

// magic and shift with v / d == mulhi(v, magic) >> shift for every 0 <= v < 2^31 (d >= 3, or any
// d >= 2 that is no power of two; powers of two from 4 on work as well)
inline void magic_u31(int64_t d, uint32_t* magic, int* shift) {
    int cl = 0;                             // ceil(log2 d)
    while (((int64_t)1 << cl) < d) ++cl;
    const int pw = 31 + cl;
    const unsigned __int128 one = 1;
    *magic = (uint32_t)((((one << pw) + (unsigned __int128)d - 1) / (unsigned __int128)d) & 0xffffffffu);
    *shift = pw - 32;
}

__device__ __forceinline__ int64_t source_row(const GemmParams& p, int64_t r) {
    int64_t s = r;
    if (p.row_index) {
        const int64_t v = p.row_index[r];
        s = p.index_shift >= 0 ? (v >> p.index_shift) : v / p.index_div;
    }
    return clamp_i64(s, 0, p.a_rows - 1);
}

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {   // v_cvt_pk_bf16_f32, RNE
    f32x2 v = {a, b};
    bf16x2 r = __builtin_convertvector(v, bf16x2);
    return *reinterpret_cast<uint32_t*>(&r);
}
__device__ __forceinline__ float rbf(float a) {   // round to bf16 and back
    return (float)(__bf16)a;
}
// the same for two values with one conversion instruction
__device__ __forceinline__ void rbf2(float& a, float& b) {
    const uint32_t pk = pack_bf16(a, b);
    a = __uint_as_float(pk << 16);
    b = __uint_as_float(pk & 0xffff0000u);
}

// SiLU on 8 packed bf16 with the rounding of F.silu on a bf16 tensor
__device__ __forceinline__ u32x4 silu_bf16x8(u32x4 v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = silu_f32(bf16_bits_to_f32(v[j] & 0xffffu));
        const float hi = silu_f32(__uint_as_float(v[j] & 0xffff0000u));
        v[j] = pack_bf16(lo, hi);
    }
    return v;
}

__device__ __forceinline__ u32x4 silu_f32x4(u32x4 v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = __float_as_uint(silu_f32(__uint_as_float(v[j])));
    return v;
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {   // s_waitcnt vmcnt(N) only
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// 16-byte store through a buffer descriptor over [base, base + 2 GiB): a lane whose offset is
// kDropLane lies outside the descriptor's range and the hardware drops its part, so the
// instruction is issued whatever the lanes' predicates are.  The compiler then knows how many
// stores follow an older load and waits for that load with an exact count; behind stores it
// may or may not have branched around it has to wait for everything in flight, the LDS-DMA
// stream and the stores' own round trip included.  base is wave-uniform (scalar registers).
constexpr uint32_t kDropLane = 0x80000000u;
__device__ __forceinline__ void store16_uniform_base(const void* base, uint32_t lane_offset, u32x4 v) {
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)kDropLane, 0x00020000);
    __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, (int)lane_offset, 0, 0);
}

}  // namespace fmoe
