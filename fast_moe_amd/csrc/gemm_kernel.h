// Jagged ("grouped") GEMM for gfx950: out[rows of expert e] = A[gather] x B[e],
// bf16 or OCP-e4m3 operands, fp32 MFMA accumulation, fused bias / SiLU / SwiGLU
// epilogue.  Shared by gemm_bf16.hip and gemm_fp8.hip.
//
// Three kernels share the scheduler and the epilogue:
//
//   grouped_gemm_ring_kernel   the fast path.  Persistent (one block per CU), 256 x 256 tiles,
//       8 wavefronts.  Operand K-slices of 64 bytes per row travel global -> LDS with
//       global_load_lds_dwordx4 (no VGPR staging) into a ring of 32 KB slots; the ring runs
//       across tile boundaries, so the loads of the next tile are already under way while
//       the current tile's epilogue stores drain.  With few experts the ring takes all of
//       LDS (5 slots), slices are fetched in pairs as full 128-byte lines and the K loop is
//       a software pipeline of 8-MFMA blocks (see RingCfg); otherwise 4 slots, one slice at
//       a time, schedule tables in LDS.
//   grouped_gemm_stream_kernel experts with a handful of rows (the weights are streamed once
//       and that stream is the cost).  Persistent 64 x 256 tiles, 4 wavefronts, two blocks per
//       CU; a K-slice travels global -> registers -> LDS while the previous one is multiplied,
//       and the next tile's first slice is loaded before the current tile's epilogue, so the
//       weight stream does not stop at tile boundaries.
//   grouped_gemm_kernel        register-staged, double-buffered LDS; serves everything the
//       other two do not: arbitrary B strides and K / N tails (element loads), SiLU applied
//       to A on load, fp32 operands.
//
// e4m3 row-wise scales that are exact powers of two (GemmParams::scale_pow2) are handed to
// v_mfma_scale_f32_32x32x64_f8f6f4 as E8M0 codes of their reciprocals instead of being divided
// out in the epilogue (ring and streaming kernels; template parameter MSC).
//
// Mapping to the hardware
//   * LDS rows are XOR-swizzled in 16-byte chunks so that the ds_read_b128 of an MFMA
//     fragment is conflict free; for the ring kernel the swizzle is applied by permuting
//     which global chunk each lane fetches, because LDS-DMA lays lanes out linearly.
//   * The weights feed the MFMA "A" port and the activations the "B" port
//     (v_mfma_f32_32x32x16_bf16 / v_mfma_f32_32x32x64_f8f6f4), so a lane holds 4 consecutive
//     output columns of one output row per register quad; v_permlane32_swap pairs two
//     quads into 16 contiguous bytes for the store.
//   * Activation rows are gathered through row_index while loading (no [R, K] copy); rows
//     past the end of an expert segment re-read the tile's first row and are masked at the
//     store.
//   * Scheduling is on the device: the number of row tiles per expert comes from `offsets`
//     (wavefront prefix scan), so no max_seq_len and no host synchronisation are needed and
//     skewed or empty experts cost nothing.  Block ids are dealt round-robin to the 8 XCDs by
//     the hardware; id -> tile is remapped so that each XCD works on whole groups of tiles
//     (4 row tiles x all column tiles, what shares operands), which keeps them in its L2: the
//     paired ring deals the groups to the XCDs back and forth, the other kernels give every
//     XCD one contiguous range of the tile order.
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

// ------------------------------------------------------------------------ epilogue
// acc[fn][fm][v]: fragment (fn, fm) of the wave tile, v = 4*g + j <-> output row
// (lane & 31) of fragment row block fm, output column 32*fn + 8*g + 4*(lane >> 5) + j.
// Rounding points follow the reference's bf16 path: GEMM result (+bias) rounded to bf16,
// SiLU rounded to bf16, product rounded to bf16; e4m3 operands: (acc / (s_a * s_w)) rounded,
// then the bias added in bf16.
// ALWAYS_VEC: the caller has checked p.vec_store (the ring kernel is only chosen with it), so
// the element-store path is not even compiled in.  ROWS32: total_rows < 2^31 (the paired ring's
// condition), so row numbers and row_index values fit 32 bits.
// OUT2: an expert's output rows are split in two halves that go to two tensors (p.out2; the
// weight gradients of two matrices from one GEMM); a 32-row block lies in one half.
// ROW_IL: the two wave rows share the tile's 32-row blocks alternately (block 2*fm + wm belongs to
// wave row wm) instead of owning one half of the tile each, so that a tile with few valid rows
// leaves both with the same number of blocks to compute.
// after_stores(): called at the very end, in the same straight-line code as the stores and the
// counted wait behind them, where the compiler's own count of what is still in flight is exact
// (behind the join of the epilogue's variants it is not: it has to assume the path that stored
// nothing).  The ring kernel converts the row indices it fetched before the epilogue there.
struct NoAfterStores {
    __device__ __forceinline__ void operator()() const {}
    __device__ __forceinline__ void block_done(int) const {}
};
// block_done(fm): called behind the stores of the wave's row block fm (straight-line code as well);
// the ring kernel issues the next tile's scale loads there, under the arithmetic of the blocks left.
template <typename BlockDone, typename AfterAll>
struct EpilogueHooks {
    BlockDone on_block;
    AfterAll on_end;
    __device__ __forceinline__ void operator()() const { on_end(); }
    __device__ __forceinline__ void block_done(int fm) const { on_block(fm); }
};
template <typename BlockDone, typename AfterAll>
__device__ __forceinline__ EpilogueHooks<BlockDone, AfterAll> make_hooks(BlockDone b, AfterAll a) {
    return EpilogueHooks<BlockDone, AfterAll>{b, a};
}

// E8M0 code (2^(code - 127)) of the reciprocal of a power-of-two fp32 scale: what the scale
// operands of v_mfma_scale_f32_32x32x64_f8f6f4 take.  2^127 (the quantiser's scale of an all-zero
// or non-finite row) gives code 0 = 2^-127.
__device__ __forceinline__ uint32_t e8m0_of_reciprocal(float scale) {
    return (254u - (__float_as_uint(scale) >> 23)) & 0xffu;
}
// one e4m3 MFMA whose products are scaled by 2^(byte OA of sa - 127) per weight row and
// 2^(byte OB of sb - 127) per activation row (lane l: row l % 32 of its fragment).
// Written as inline assembly with the accumulator tied to the destination: through the builtin the
// destination is a separate early-clobber operand, which costs the ring kernel (at 256 registers
// with 128 of them accumulators) about 50 spilled registers per lane around the tile boundary.
// The compiler therefore does not know that this is an MFMA and inserts none of the wait states
// the matrix pipe needs around VALU accesses to its registers.  VALU write -> MFMA read (the
// clears of a tile's accumulators, the packed scale codes): two idle issue cycles stand in front
// of every one of these instructions, inside the same statement (they pass while the pipe works
// on the MFMA before).  MFMA write -> VALU read (the epilogue): mfma_results_guard() behind the
// main loop.
template <int OA, int OB>
__device__ __forceinline__ void mfma_e4m3_scaled(const i32x8& a, const i32x8& b, f32x16& c, uint32_t sa, uint32_t sb) {
    asm volatile("s_nop 1\n\tv_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%8,0]"
                 : "+v"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb), "n"(OA & 1), "n"(OB & 1), "n"(OA >> 1), "n"(OB >> 1));
}
// 32 idle issue cycles behind the last of those MFMAs (a 16-pass MFMA needs 18 before the VALU may
// read its result), and nothing that follows in the program may be scheduled in front of them.
__device__ __forceinline__ void mfma_results_guard() {
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// MSC (e4m3): the scales were applied by the MFMAs themselves (power-of-two scales as block scales of
// the instruction): acc already holds sum / (s_a * s_w) and the epilogue loads and multiplies nothing.
template <int FM, int FN, int TM, int TN, bool FP8, int EPI, bool ALWAYS_VEC = false, bool ROWS32 = false,
          bool OUT2 = false, bool ROW_IL = false, typename AfterStores = NoAfterStores, bool MSC = false>
__device__ __forceinline__ void gemm_epilogue(const GemmParams& p, f32x16 (&acc)[FN][FM], int expert,
                                              int n0, int64_t row0, int rows_valid, int wm, int wn,
                                              int lane, AfterStores after_stores = AfterStores(),
                                              uint64_t* ets = nullptr) {
    constexpr bool SWIGLU = EPI == FMOE_EPI_SWIGLU;
    constexpr bool GATED = EPI == FMOE_EPI_GATED;   // out = silu(gate from p.aux) * (acc + bias); bf16 operands
    static_assert(!(GATED && FP8), "the gated epilogue is built for bf16 operands");
    constexpr int FN_OUT = SWIGLU ? FN / 2 : FN;
    // (ring kernel: everything derived from the lane number below is recomputed per tile; as
    // tile-loop invariants the compiler keeps such values in registers across the main loop, or
    // spills them and reloads them here behind a wait that drains the LDS-DMA stream)
    if (ALWAYS_VEC) asm volatile("" : "+v"(lane));
    const int khalf = lane >> 5;
    const int64_t bias_row = (int64_t)expert * p.bias_se;
#ifdef FMOE_TRACE
#define FMOE_EPI_STAMP(i_) do { if (ets) ets[i_] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define FMOE_EPI_STAMP(i_) do {} while (0)
#endif
    // Output addresses are a wave-uniform 64-bit base (tile row block, column group: scalar
    // registers and scalar arithmetic) plus one 32-bit per-lane byte offset (the lane's row
    // inside the 32-row block and its 16-byte half): no per-row pointers to keep in vector
    // registers over an epilogue whose accumulators and column constants already fill them.
    wm = __builtin_amdgcn_readfirstlane(wm);
    wn = __builtin_amdgcn_readfirstlane(wn);
    row0 = (int64_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(row0 >> 32)) << 32) |
                     (uint32_t)__builtin_amdgcn_readfirstlane((int)row0));
    // (computed afresh at every store from a copy of the lane number the compiler cannot see
    // through: hoisted out of the loops it becomes a 64-bit offset that is spilled and reloaded,
    // with a full vmcnt(0) wait, before every single store)
    auto lane_offset = [&](int64_t stride) -> uint32_t {
        int l = lane;
        asm volatile("" : "+v"(l));
        return (uint32_t)(l & 31) * (uint32_t)stride * 2u + (uint32_t)(l >> 5) * 16u;
    };
    // first tile row of the wave's row block fm
    auto frag_row = [&](int fm) -> int { return ROW_IL ? (fm * 2 + wm) * 32 : wm * TM + fm * 32; };
    float rsa[FM];
    bool row_ok[FM];
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
        row_ok[fm] = frag_row(fm) + (lane & 31) < rows_valid;
        rsa[fm] = 1.0f;
    }
    // per-column reciprocal weight scales of this lane (e4m3): [fn][gp][q][j] <-> column
    // nq + 8*q + 4*khalf + j with nq = first column of register-quad pair gp of fragment fn
    float rsw[FN_OUT][2][2][4], rsw2[FN_OUT][2][2][4];
    const int col0 = n0 + (SWIGLU ? wn * (TN / 2) : wn * TN);
    constexpr bool SCALE = FP8 && !MSC;         // divide the scales out here
    if (SCALE) {
        // the activation scales of this lane's rows: all index loads, then all scale loads (two
        // memory latencies, not two per row block)
        typedef typename std::conditional<ROWS32, int32_t, int64_t>::type row_t;
        row_t src[FM];
#pragma unroll
        for (int fm = 0; fm < FM; ++fm)
            src[fm] = (row_t)(row0 + (row_ok[fm] ? frag_row(fm) + (lane & 31) : 0));
        if (p.row_index) {
#pragma unroll
            for (int fm = 0; fm < FM; ++fm) {
                if (ROWS32) src[fm] = reinterpret_cast<const int32_t*>(p.row_index)[2 * (int64_t)src[fm]];   // low half
                else src[fm] = (row_t)p.row_index[src[fm]];
            }
#pragma unroll
            for (int fm = 0; fm < FM; ++fm)
                if (ROWS32) src[fm] = (row_t)div_index32(p, (int32_t)src[fm]);
                else src[fm] = p.index_shift >= 0 ? (src[fm] >> p.index_shift) : src[fm] / (row_t)p.index_div;
        }
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
            const row_t last = (row_t)(p.a_rows - 1);
            src[fm] = src[fm] < 0 ? 0 : (src[fm] > last ? last : src[fm]);
        }
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) rsa[fm] = p.a_scale[src[fm]];
        // The weight-scale loads go out right behind the activation-scale loads, before anything
        // waits for either, so that the two round trips overlap (one memory latency per tile less;
        // the raw values wait in the registers their reciprocals end up in).
        constexpr int WCOLS = FN_OUT * 32;          // output columns of this wave
        if (p.scale_vec && col0 + WCOLS <= p.N) {
            // the wave's columns lie inside N: the 4 scales of a register quad in one 16-byte load
            // from a wave-uniform base plus the lane half's 16 bytes plus a constant
            const float* sb = p.b_scale + ((int64_t)expert * p.N + col0);
            const float* sb2 = SWIGLU ? p.b2_scale + ((int64_t)expert * p.N + col0) : sb;
            const int half4 = 4 * khalf;
            typedef __attribute__((ext_vector_type(4))) float f32x4;
#pragma unroll
            for (int fn = 0; fn < FN_OUT; ++fn)
#pragma unroll
                for (int gp = 0; gp < 2; ++gp)
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const int c = fn * 32 + 16 * gp + 8 * q;
                        const f32x4 s1 = *reinterpret_cast<const f32x4*>(sb + half4 + c);
                        f32x4 s2 = s1;
                        if (SWIGLU) s2 = *reinterpret_cast<const f32x4*>(sb2 + half4 + c);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            rsw[fn][gp][q][j] = s1[j];
                            rsw2[fn][gp][q][j] = s2[j];
                        }
                    }
        } else {
            // the last column tile, or scale tensors off a 16-byte boundary: one clamped load a column
#pragma unroll
            for (int fn = 0; fn < FN_OUT; ++fn)
#pragma unroll
                for (int gp = 0; gp < 2; ++gp)
#pragma unroll
                    for (int q = 0; q < 2; ++q)
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int n = col0 + fn * 32 + 16 * gp + 8 * q + 4 * khalf + j;
                            const int nc = n < p.N ? n : p.N - 1;
                            rsw[fn][gp][q][j] = rsw2[fn][gp][q][j] = p.b_scale[(int64_t)expert * p.N + nc];
                            if (SWIGLU) rsw2[fn][gp][q][j] = p.b2_scale[(int64_t)expert * p.N + nc];
                        }
        }
        __builtin_amdgcn_sched_barrier(0);
        // (v_rcp_f32 is exact on the powers of two the reference's scales are)
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) rsa[fm] = __builtin_amdgcn_rcpf(rsa[fm]);
#pragma unroll
        for (int fn = 0; fn < FN_OUT; ++fn)
#pragma unroll
            for (int gp = 0; gp < 2; ++gp)
#pragma unroll
                for (int q = 0; q < 2; ++q)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        rsw[fn][gp][q][j] = __builtin_amdgcn_rcpf(rsw[fn][gp][q][j]);
                        if (SWIGLU) rsw2[fn][gp][q][j] = __builtin_amdgcn_rcpf(rsw2[fn][gp][q][j]);
                    }
    }
    // the bias-free form (FastMoE's SwiGLU experts, every fp8 call without bias) skips the adds
    auto run = [&](auto has_bias_c, auto has_aux_c) {
        constexpr bool HAS_BIAS = decltype(has_bias_c)::value;
        constexpr bool HAS_AUX = SWIGLU && decltype(has_aux_c)::value;   // keep the pre-activations (training)
        constexpr bool QUAD = ALWAYS_VEC && !SWIGLU && FN_OUT == 2;   // plain and SiLU epilogues of the ring kernel, bf16 and e4m3
        // per-column biases of this lane, indexed like rsw
        float bv[FN_OUT][2][2][4], bv2[FN_OUT][2][2][4];
        // with a bias, at least one of the two pointers is set: both loads go through a valid
        // pointer and a select drops the value of a missing one (a branch per load would make
        // every load wait for the one before)
        const uint16_t* bias_a = p.bias ? p.bias : p.bias2;
        const uint16_t* bias_b = p.bias2 ? p.bias2 : p.bias;
#pragma unroll
        for (int fn = 0; fn < FN_OUT; ++fn)
#pragma unroll
            for (int gp = 0; gp < 2; ++gp)
#pragma unroll
                for (int q = 0; q < 2; ++q)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int n = col0 + fn * 32 + 16 * gp + 8 * q + 4 * khalf + j;
                        const int nc = n < p.N ? n : p.N - 1;
                        bv[fn][gp][q][j] = bv2[fn][gp][q][j] = 0.0f;
                        if (HAS_BIAS) {
                            const float a = bf16_bits_to_f32(bias_a[bias_row + nc]);
                            bv[fn][gp][q][j] = p.bias ? a : 0.0f;
                        }
                        if (HAS_BIAS && SWIGLU) {
                            const float b = bf16_bits_to_f32(bias_b[bias_row + nc]);
                            bv2[fn][gp][q][j] = p.bias2 ? b : 0.0f;
                        }
                    }
        __builtin_amdgcn_sched_barrier(0);
        FMOE_EPI_STAMP(0);
        // GATED in the rearranged form: a lane's gate values are the 16 bytes at the position its
        // store i of a row block writes; the four loads of block fm + 1 go out before block fm's
        // arithmetic, so that one memory latency per tile is waited for, not one per block.
        u32x4 gate_next[4] = {};
        auto fetch_gate = [&](int fm, u32x4 (&g)[4]) {
            int l = lane;
            asm volatile("" : "+v"(l));
            const int quad_row = 4 * ((l & 31) >> 2);
            const int col = col0 + 32 * (l >> 5) + 8 * (l & 3);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool ok = frag_row(fm) + quad_row + i < rows_valid && col + 7 < p.N;
                const uint16_t* src = p.aux + (row0 + (ok ? frag_row(fm) + quad_row + i : 0)) * p.aux_stride + (ok ? col : 0);
                if (p.gate_vec16) {
                    g[i] = *reinterpret_cast<const u32x4*>(src);
                } else {
                    uint32_t e[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) e[j] = ok ? (uint32_t)src[j] : 0u;
                    g[i] = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
                }
            }
        };
        if constexpr (QUAD && GATED) fetch_gate(0, gate_next);
        // rows outermost: the stores that complete a row's 128-byte line follow each other
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
            if (fm > 0) FMOE_EPI_STAMP(fm);
            if constexpr (QUAD) {
                u32x4 gate_cur[4];
                if constexpr (GATED) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) gate_cur[i] = gate_next[i];
                    if (fm + 1 < FM) fetch_gate(fm + 1, gate_next);
                }
                // The store unit merges what ADJACENT lanes write: a lane and its partner 32 lanes
                // away cost two requests even for neighbouring bytes, four adjacent lanes on 64
                // contiguous bytes cost one (a 128 KB tile drains in 1.3 us instead of 3.9).  So:
                // the halves of the wave trade pieces until a low lane owns columns 0..31 of its row
                // and its partner 32..63, then every quad of lanes transposes its 4 rows x 4 chunks
                // of 16 bytes, and store i of the block writes row 4q + i from the 4 lanes of quad q.
                uint32_t pk[8][2];          // piece g: columns 8g + 4*khalf + 0..3 of the wave's 64
#pragma unroll
                for (int fn = 0; fn < 2; ++fn)
#pragma unroll
                    for (int gp = 0; gp < 2; ++gp)
#pragma unroll
                        for (int q = 0; q < 2; ++q)
#pragma unroll
                            for (int j = 0; j < 4; j += 2) {
                                const int v = 4 * (2 * gp + q) + j;
                                float ya = acc[fn][fm][v], yb = acc[fn][fm][v + 1];
                                if (FP8) {
                                    if (SCALE) {
                                        ya *= rsa[fm] * rsw[fn][gp][q][j];
                                        yb *= rsa[fm] * rsw[fn][gp][q][j + 1];
                                    }
                                    if (HAS_BIAS && p.bias) {
                                        rbf2(ya, yb);
                                        ya += bv[fn][gp][q][j];
                                        yb += bv[fn][gp][q][j + 1];
                                    }
                                } else if (HAS_BIAS) {
                                    ya += bv[fn][gp][q][j];
                                    yb += bv[fn][gp][q][j + 1];
                                }
                                if (EPI == FMOE_EPI_SILU) {
                                    rbf2(ya, yb);
                                    ya = fast_silu_f32(ya);
                                    yb = fast_silu_f32(yb);
                                }
                                pk[4 * fn + 2 * gp + q][j / 2] = pack_bf16(ya, yb);
                            }
                uint32_t ch[4][4];          // chunk c: columns 32*khalf + 8c + 0..7, afterwards row 4q + c's
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int d = 0; d < 2; ++d) {
                        const u32x2 s = __builtin_amdgcn_permlane32_swap(pk[c][d], pk[c + 4][d], false, false);
                        ch[c][d] = s[0];
                        ch[c][2 + d] = s[1];
                    }
                int l = lane;
                asm volatile("" : "+v"(l));
                const bool odd = (l & 1) != 0, up = (l & 2) != 0;
#pragma unroll
                for (int pr = 0; pr < 4; pr += 2)       // lanes j, j ^ 1 trade across slots (pr, pr + 1)
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const uint32_t send = odd ? ch[pr][d] : ch[pr + 1][d];
                        const uint32_t recv = (uint32_t)__builtin_amdgcn_mov_dpp((int)send, 0xB1, 0xF, 0xF, true);
                        ch[pr][d] = odd ? recv : ch[pr][d];
                        ch[pr + 1][d] = odd ? ch[pr + 1][d] : recv;
                    }
#pragma unroll
                for (int pr = 0; pr < 2; ++pr)          // lanes j, j ^ 2 trade across slots (pr, pr + 2)
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const uint32_t send = up ? ch[pr][d] : ch[pr + 2][d];
                        const uint32_t recv = (uint32_t)__builtin_amdgcn_mov_dpp((int)send, 0x4E, 0xF, 0xF, true);
                        ch[pr][d] = up ? recv : ch[pr][d];
                        ch[pr + 2][d] = up ? ch[pr + 2][d] : recv;
                    }
                const int64_t block_row = row0 + frag_row(fm);
                uint16_t* obase = p.out + block_row * p.out_stride;
                if constexpr (OUT2) {
                    if (p.out2) {       // (as below: wave-uniform, forced into the two tensors)
                        int64_t m = block_row - (int64_t)expert * (2 * p.out_half);
                        m = m < 0 ? 0 : (m > 2 * p.out_half - 32 ? 2 * p.out_half - 32 : m);
                        m &= ~(int64_t)31;
                        const bool upper = m >= p.out_half;
                        obase = (upper ? p.out2 : p.out) +
                                ((int64_t)expert * p.out_half + (upper ? m - p.out_half : m)) * p.out_stride;
                    }
                }
                const int quad_row = 4 * ((l & 31) >> 2);
                const int col = col0 + 32 * (l >> 5) + 8 * (l & 3);
                const uint32_t lane_off = ((uint32_t)quad_row * (uint32_t)p.out_stride + (uint32_t)(32 * (l >> 5) + 8 * (l & 3))) * 2u;
                if constexpr (GATED) {      // ch holds round(acc + bias): times the rounded SiLU of the gate
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            float ga = __uint_as_float(gate_cur[i][d] << 16), gb = __uint_as_float(gate_cur[i][d] & 0xffff0000u);
                            ga = fast_silu_f32(ga);
                            gb = fast_silu_f32(gb);
                            rbf2(ga, gb);
                            ch[i][d] = pack_bf16(ga * __uint_as_float(ch[i][d] << 16), gb * __uint_as_float(ch[i][d] & 0xffff0000u));
                        }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    uint16_t* base = obase + i * p.out_stride + col0;
                    const bool ok = frag_row(fm) + quad_row + i < rows_valid && col + 7 < p.N;
                    store16_uniform_base(base, ok ? lane_off : kDropLane, u32x4{ch[i][0], ch[i][1], ch[i][2], ch[i][3]});
                }
                __builtin_amdgcn_sched_barrier(0);
                after_stores.block_done(fm);
                continue;
            }
            // GATED: the row block's gate values, all loads of the block issued together (one memory
            // latency per 32-row block; loaded where they are used, every group of 8 waits out its own)
            u32x2 graw[FN_OUT][2][2];
            if constexpr (GATED) {
                const int64_t grow = row0 + (row_ok[fm] ? frag_row(fm) + (lane & 31) : 0);
                const uint16_t* gp_row = p.aux + grow * p.aux_stride;
#pragma unroll
                for (int fn = 0; fn < FN_OUT; ++fn)
#pragma unroll
                    for (int gp = 0; gp < 2; ++gp)
#pragma unroll
                        for (int q = 0; q < 2; ++q) {
                            const int n = col0 + fn * 32 + 16 * gp + 8 * q + 4 * khalf;
                            if (p.gate_vec && n + 3 < p.N) {
                                graw[fn][gp][q] = *reinterpret_cast<const u32x2*>(gp_row + n);
                            } else {
                                uint32_t e[4];
#pragma unroll
                                for (int j = 0; j < 4; ++j) e[j] = n + j < p.N ? (uint32_t)gp_row[n + j] : 0u;
                                graw[fn][gp][q] = u32x2{e[0] | (e[1] << 16), e[2] | (e[3] << 16)};
                            }
                        }
            }
#pragma unroll
            for (int fn = 0; fn < FN_OUT; ++fn) {
#pragma unroll
                for (int gp = 0; gp < 2; ++gp) {
                    const int nq = col0 + fn * 32 + 16 * gp;
                    float o[2][4], pg[2][4], pu[2][4];
                    // GATED: this lane's 2 x 4 gate values (its row, columns nq + 8q + 4*khalf + 0..3)
                    float gate[2][4];
                    if constexpr (GATED) {
#pragma unroll
                        for (int q = 0; q < 2; ++q) {
                            const u32x2 g2 = graw[fn][gp][q];
                            gate[q][0] = __uint_as_float(g2[0] << 16);
                            gate[q][1] = __uint_as_float(g2[0] & 0xffff0000u);
                            gate[q][2] = __uint_as_float(g2[1] << 16);
                            gate[q][3] = __uint_as_float(g2[1] & 0xffff0000u);
                        }
                    }
                    // two columns at a time: one conversion instruction rounds a pair
#pragma unroll
                    for (int q = 0; q < 2; ++q)
#pragma unroll
                        for (int j = 0; j < 4; j += 2) {
                            const int v = 4 * (2 * gp + q) + j;
                            float ya = acc[fn][fm][v], yb = acc[fn][fm][v + 1];
                            float ua = SWIGLU ? acc[fn + FN / 2][fm][v] : 0.0f;
                            float ub = SWIGLU ? acc[fn + FN / 2][fm][v + 1] : 0.0f;
                            if (FP8) {
                                if (SCALE) {
                                    ya *= rsa[fm] * rsw[fn][gp][q][j];
                                    yb *= rsa[fm] * rsw[fn][gp][q][j + 1];
                                }
                                rbf2(ya, yb);
                                if (HAS_BIAS && p.bias) {
                                    ya += bv[fn][gp][q][j];
                                    yb += bv[fn][gp][q][j + 1];
                                    rbf2(ya, yb);
                                }
                                if (SWIGLU) {
                                    if (SCALE) {
                                        ua *= rsa[fm] * rsw2[fn][gp][q][j];
                                        ub *= rsa[fm] * rsw2[fn][gp][q][j + 1];
                                    }
                                    rbf2(ua, ub);
                                    if (HAS_BIAS && p.bias2) {
                                        ua += bv2[fn][gp][q][j];
                                        ub += bv2[fn][gp][q][j + 1];
                                        rbf2(ua, ub);
                                    }
                                }
                            } else {
                                if (HAS_BIAS) {
                                    ya += bv[fn][gp][q][j];
                                    yb += bv[fn][gp][q][j + 1];
                                }
                                rbf2(ya, yb);
                                if (SWIGLU) {
                                    if (HAS_BIAS) {
                                        ua += bv2[fn][gp][q][j];
                                        ub += bv2[fn][gp][q][j + 1];
                                    }
                                    rbf2(ua, ub);
                                }
                                if constexpr (GATED) {      // the product so far is the factor, the gate the argument
                                    ua = ya;
                                    ub = yb;
                                    ya = gate[q][j];
                                    yb = gate[q][j + 1];
                                }
                            }
                            pg[q][j] = ya;
                            pg[q][j + 1] = yb;
                            pu[q][j] = ua;
                            pu[q][j + 1] = ub;
                            if (EPI == FMOE_EPI_SILU) {
                                ya = fast_silu_f32(ya);
                                yb = fast_silu_f32(yb);
                            }
                            if (SWIGLU || GATED) {
                                ya = fast_silu_f32(ya);
                                yb = fast_silu_f32(yb);
                                rbf2(ya, yb);
                                ya *= ua;
                                yb *= ub;
                            }
                            o[q][j] = ya;
                            o[q][j + 1] = yb;
                        }
                    // base: first element of the 32-row block's first row (wave-uniform)
                    auto store = [&](const float (&val)[2][4], uint16_t* base, int64_t stride) {
                        if constexpr (ALWAYS_VEC) {
                            const uint32_t lane_off = lane_offset(stride);
                            const u32x2 s0 = __builtin_amdgcn_permlane32_swap(pack_bf16(val[0][0], val[0][1]),
                                                                              pack_bf16(val[1][0], val[1][1]), false, false);
                            const u32x2 s1 = __builtin_amdgcn_permlane32_swap(pack_bf16(val[0][2], val[0][3]),
                                                                              pack_bf16(val[1][2], val[1][3]), false, false);
                            const int nb = nq + 8 * khalf;
                            const bool ok = row_ok[fm] && nb + 7 < p.N;
                            store16_uniform_base(base + nq, ok ? lane_off : kDropLane, u32x4{s0[0], s1[0], s0[1], s1[1]});
                        } else if (p.vec_store) {
                            const uint32_t lane_off = lane_offset(stride);
                            // pair the quads of the two lane halves: low lanes end up with columns
                            // nq..nq+7, high lanes with nq+8..nq+15 of their row
                            const u32x2 s0 = __builtin_amdgcn_permlane32_swap(pack_bf16(val[0][0], val[0][1]),
                                                                              pack_bf16(val[1][0], val[1][1]), false, false);
                            const u32x2 s1 = __builtin_amdgcn_permlane32_swap(pack_bf16(val[0][2], val[0][3]),
                                                                              pack_bf16(val[1][2], val[1][3]), false, false);
                            const int nb = nq + 8 * khalf;
                            if (row_ok[fm] && nb + 7 < p.N)
                                *reinterpret_cast<u32x4*>(reinterpret_cast<uint8_t*>(base + nq) + lane_off) =
                                    u32x4{s0[0], s1[0], s0[1], s1[1]};
                        } else if (row_ok[fm]) {
                            uint16_t* dst = base + (int64_t)(lane & 31) * stride;
#pragma unroll
                            for (int q = 0; q < 2; ++q)
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    const int n = nq + 8 * q + 4 * khalf + j;
                                    if (n < p.N) dst[n] = (uint16_t)f32_to_bf16_bits(val[q][j]);
                                }
                        }
                    };
                    const int64_t block_row = row0 + frag_row(fm);
                    uint16_t* obase = p.out + block_row * p.out_stride;
                    if constexpr (OUT2) {
                        if (p.out2) {       // (scalar arithmetic: everything here is wave-uniform)
                            // (offsets that are not the promised e * 2h are not followed out of
                            // the two tensors: the block's row is forced into [0, 2h), whole blocks)
                            int64_t m = block_row - (int64_t)expert * (2 * p.out_half);
                            m = m < 0 ? 0 : (m > 2 * p.out_half - 32 ? 2 * p.out_half - 32 : m);
                            m &= ~(int64_t)31;
                            const bool upper = m >= p.out_half;
                            obase = (upper ? p.out2 : p.out) +
                                    ((int64_t)expert * p.out_half + (upper ? m - p.out_half : m)) * p.out_stride;
                        }
                    }
                    store(o, obase, p.out_stride);
                    if (HAS_AUX) {
                        store(pg, p.aux + block_row * p.aux_stride, p.aux_stride);
                        store(pu, p.aux2 + block_row * p.aux_stride, p.aux_stride);
                    }
                    // one column group at a time: interleaving the groups for more parallelism
                    // is what runs the scheduler out of registers here
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            after_stores.block_done(fm);
        }
        // Everything older than this epilogue's own stores has completed: a wait that costs
        // nothing (the loads it names were needed above) but tells the compiler so.  Without it
        // a spill reload that one of the branches above leaves unused stays "pending" in the
        // compiler's count, and the wait for it lands where its register is next written:
        // inside the caller's steady-state loop, where it would also drain the LDS-DMA stream,
        // which the compiler cannot see, on every iteration.
        FMOE_EPI_STAMP(FM);
        // The number of store instructions issued above, whatever the lanes' predicates: 4 per row
        // block in the rearranged form, one per column group (and per output tensor) otherwise.
        // The ring kernel's first double step of the next tile skips its own counted wait on the
        // strength of this one (see skip_wait there), which is only sound when every one of these
        // stores was issued unconditionally, i.e. through store16_uniform_base (ALWAYS_VEC).
        constexpr int kStoresIssued = FM * (QUAD ? 4 : FN_OUT * 2 * (HAS_AUX ? 3 : 1));
        static_assert(!QUAD || FN_OUT * 2 == 4, "the rearranged form stores as many pieces as the column-group form");
        static_assert(kStoresIssued <= 63, "vmcnt is a 6-bit field");
        wait_vmcnt<kStoresIssued>();      // (the scalar-store path issues more)
        after_stores();
    };
    if (SWIGLU && p.aux) {
        if (p.bias || p.bias2) run(std::true_type{}, std::true_type{});
        else run(std::false_type{}, std::true_type{});
    } else {
        if (p.bias || p.bias2) run(std::true_type{}, std::false_type{});
        else run(std::false_type{}, std::false_type{});
    }
}

// fp32 operands: fp32 bias and output, no intermediate rounding, exact SiLU.
template <int FM, int FN, int TM, int TN, int EPI>
__device__ __forceinline__ void gemm_epilogue_f32(const GemmParams& p, f32x16 (&acc)[FN][FM], int expert,
                                                  int n0, int64_t row0, int rows_valid, int wm, int wn,
                                                  int lane) {
    constexpr bool SWIGLU = EPI == FMOE_EPI_SWIGLU;
    constexpr int FN_OUT = SWIGLU ? FN / 2 : FN;
    const int khalf = lane >> 5;
    const float* bias = reinterpret_cast<const float*>(p.bias);
    const float* bias2 = reinterpret_cast<const float*>(p.bias2);
    float* out = reinterpret_cast<float*>(p.out);
    const int64_t bias_row = (int64_t)expert * p.bias_se;
#pragma unroll
    for (int fn = 0; fn < FN_OUT; ++fn) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int nb = n0 + (SWIGLU ? wn * (TN / 2) : wn * TN) + fn * 32 + 8 * g + 4 * khalf;
            float bv[4], bv2[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int nc = nb + j < p.N ? nb + j : p.N - 1;
                bv[j] = bias ? bias[bias_row + nc] : 0.0f;
                bv2[j] = (SWIGLU && bias2) ? bias2[bias_row + nc] : 0.0f;
            }
#pragma unroll
            for (int fm = 0; fm < FM; ++fm) {
                const int tile_row = wm * TM + fm * 32 + (lane & 31);
                if (tile_row >= rows_valid) continue;
                float* orow = out + (row0 + tile_row) * p.out_stride;
                float o[4], pg[4], pu[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float y = acc[fn][fm][4 * g + j] + bv[j];
                    pg[j] = y;
                    pu[j] = SWIGLU ? acc[fn + FN / 2][fm][4 * g + j] + bv2[j] : 0.0f;
                    if (EPI == FMOE_EPI_SILU) y = silu_f32(y);
                    if (SWIGLU) y = silu_f32(y) * pu[j];
                    o[j] = y;
                }
                auto store = [&](const float (&val)[4], float* dst) {
                    if (p.vec_store && nb + 3 < p.N) {
                        *reinterpret_cast<f32x4*>(dst + nb) = f32x4{val[0], val[1], val[2], val[3]};
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (nb + j < p.N) dst[nb + j] = val[j];
                    }
                };
                store(o, orow);
                if (SWIGLU && p.aux) {
                    store(pg, reinterpret_cast<float*>(p.aux) + (row0 + tile_row) * p.aux_stride);
                    store(pu, reinterpret_cast<float*>(p.aux2) + (row0 + tile_row) * p.aux_stride);
                }
            }
        }
    }
}

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
                        acc[0][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[0], xf[0], acc[0][0], 0, 0, 2, (int)sc, 0, (int)sc);
                        acc[0][1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[0], xf[1], acc[0][1], 0, 0, 2, (int)sc, 1, (int)sc);
                        acc[1][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[1], xf[0], acc[1][0], 0, 0, 3, (int)sc, 0, (int)sc);
                        acc[1][1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[1], xf[1], acc[1][1], 0, 0, 3, (int)sc, 1, (int)sc);
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
                static_assert(NM % L == 0 || L % NM == 0, "DMA parts must spread evenly over the MFMAs");
                constexpr int PER = L >= NM ? L / NM : 1, EVERY = L >= NM ? 1 : NM / L;
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const int fn = m / ACT, fm = m % ACT;
                    acc[fn][fm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[fn], xf[fm], acc[fn][fm], 0, 0, 0);
                    if (DMA && (m + 1) % EVERY == 0) {
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int q = 0; q < PER; ++q) issue_part(((m + 1) / EVERY - 1) * PER + q);
                        __builtin_amdgcn_sched_barrier(0);
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
                static_assert(NM % L == 0 || L % NM == 0, "DMA parts must spread evenly over the MFMAs");
                constexpr int PER = L >= NM ? L / NM : 1, EVERY = L >= NM ? 1 : NM / L;
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
                    if (DMA && (m + 1) % EVERY == 0) {
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int q = 0; q < PER; ++q) issue_part(((m + 1) / EVERY - 1) * PER + q);
                        __builtin_amdgcn_sched_barrier(0);
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


// ------------------------------------------------------------------- host side
typedef TileCfg<256, 256, 2, 4> TileBig;        // 8 waves, wave tile 128 x 64
typedef TileCfg<64, 256, 1, 4> TileSmall;       // 4 waves, wave tile 64 x 64
typedef RingCfg<256, 256, 2, 4, 0> TileRing4;   // 8 waves, wave tile 128 x 64, 4-slot ring, LDS tables
typedef RingCfg<256, 256, 2, 4, 1> TileRing5;   // 5-slot ring, paired slices, E <= 64
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
            return launch_ring_cfg<TileRing5, FP8, EPI, false, false, false, true>(p, stream);
        if (p.scale_pow2 && pair_ok && p.E <= TileRing5W::kMaxExperts)
            return launch_ring_cfg<TileRing5W, FP8, EPI, false, false, false, true>(p, stream);
    }
    if (pair_ok && p.E <= TileRing5::kMaxExperts) return launch_ring_cfg<TileRing5, FP8, EPI>(p, stream);
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
