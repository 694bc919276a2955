// The epilogue all grouped GEMM kernels share: scales, bias, SiLU / SwiGLU / gating, bf16 rounding,
// and the stores (rearranged in registers so that adjacent lanes write contiguous bytes).
#pragma once

#include "gemm_params.h"

namespace fmoe {

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

}  // namespace fmoe
