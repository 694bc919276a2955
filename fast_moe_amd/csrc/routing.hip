// Routing for the MoE forward: top-k selection with L1-renormalised gates, the
// per-expert histogram / prefix sum ("jagged offsets") and the stable
// expert-major permutation with its inverse.  All integer outputs are a pure
// function of the selected ids (a stable counting sort), so they are
// reproducible bit for bit.
//
// Two launches on one stream, no host synchronisation.  The tokens are cut into up to 256
// chunks (one block each: 16 waves up to 256 experts, 4 beyond; a wave owns a contiguous
// share of its chunk):
//   1. topk_hist_kernel (or compact_hist_kernel for caller-supplied ids): a token's scores sit
//      in a group of 8 or 16 lanes (4 to 8 tokens per wave); K rounds of a group argmax on the
//      DPP network select in descending order, ties to the lower expert id; every wave counts
//      the experts of its tokens in LDS -> sub_hist[chunk][wave][e], tot_hist[chunk][e]
//   2. scan_scatter_kernel: every block sums tot_hist over the chunks before it (and over all
//      chunks: lengths; wave scan over the experts: offsets), every wave adds the counts of
//      the waves before it in its chunk and then places its positions: a wave-level
//      match/rank gives each position its slot inside its expert segment
#include "common.h"

#include <mutex>

namespace fmoe {
namespace {

constexpr int kMaxChunks = 256;
constexpr int kMaxRouteWaves = 16;
// waves per block of both kernels: 16 while the per-wave expert tables fit LDS comfortably
inline int route_waves(int E) { return E <= 256 ? 16 : 4; }
constexpr uint16_t kBadExpert = 0xFFFF;

struct RoutePlan {
    int64_t tokens_per_wave;
    int num_chunks;
    int wpb;                // waves per block
    size_t compact_bytes;   // uint16 expert id per routed position
    size_t sub_bytes;       // int32 [num_chunks][wpb][E]
    size_t tot_bytes;       // int32 [num_chunks][E]
    size_t bad_bytes;       // int32 [num_chunks] out-of-range ids per chunk
    size_t total_bytes;
};

RoutePlan make_plan(int64_t T, int E, int K) {
    RoutePlan p;
    const int kRouteWaves = route_waves(E);
    p.wpb = kRouteWaves;
    const int64_t waves = (int64_t)kMaxChunks * kRouteWaves;
    p.tokens_per_wave = (T + waves - 1) / waves;
    if (p.tokens_per_wave < 1) p.tokens_per_wave = 1;
    const int64_t per_chunk = p.tokens_per_wave * kRouteWaves;
    p.num_chunks = (int)((T + per_chunk - 1) / per_chunk);
    if (p.num_chunks < 1) p.num_chunks = 1;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    p.compact_bytes = up((size_t)T * (size_t)K * sizeof(uint16_t));
    p.sub_bytes = up((size_t)p.num_chunks * kRouteWaves * (size_t)E * sizeof(int32_t));
    p.tot_bytes = up((size_t)p.num_chunks * (size_t)E * sizeof(int32_t));
    p.bad_bytes = up((size_t)p.num_chunks * sizeof(int32_t));
    p.total_bytes = p.compact_bytes + p.sub_bytes + p.tot_bytes + p.bad_bytes + 256;
    return p;
}

struct RouteScratch {
    uint16_t* compact;
    int32_t* sub_hist;
    int32_t* tot_hist;
    int32_t* bad_part;
};

RouteScratch carve(void* workspace, const RoutePlan& plan) {
    char* w = (char*)workspace;
    RouteScratch r;
    r.compact = (uint16_t*)w;
    r.sub_hist = (int32_t*)(w + plan.compact_bytes);
    r.tot_hist = (int32_t*)(w + plan.compact_bytes + plan.sub_bytes);
    r.bad_part = (int32_t*)(w + plan.compact_bytes + plan.sub_bytes + plan.tot_bytes);
    return r;
}

template <typename T>
__device__ __forceinline__ float load_score(const T* p);
template <>
__device__ __forceinline__ float load_score<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_score<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }

template <typename T>
__device__ __forceinline__ float round_to(float v);
template <>
__device__ __forceinline__ float round_to<float>(float v) { return v; }
template <>
__device__ __forceinline__ float round_to<uint16_t>(float v) { return round_bf16(v); }

template <typename T>
__device__ __forceinline__ void store_score(T* p, float v);
template <>
__device__ __forceinline__ void store_score<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_score<uint16_t>(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }

// Total order on scores as unsigned keys: NaN above +inf (where torch.topk and torch.sort put
// it), -0 equal to +0, otherwise the order of the values.  With keys every token fills exactly K
// distinct slots whatever its scores hold; a float comparison ranks every NaN first at once.
__device__ __forceinline__ uint32_t order_key(float v) {
    const uint32_t b = __float_as_uint(v);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return 0xFFFFFFFFu;     // NaN
    if ((b & 0x7FFFFFFFu) == 0u) return 0x80000000u;             // +-0
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// Largest value over each group of LPT (8 or 16) consecutive lanes, in every lane of the group:
// butterfly steps on the DPP network inside a row of 16 lanes (quad permutes, mirrors).
template <int LPT>
__device__ __forceinline__ uint32_t group_max_u32(uint32_t v) {
    static_assert(LPT == 8 || LPT == 16, "a group is half a DPP row or a whole one");
#define FMOE_DPP_MAX(ctrl) v = max(v, (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, ctrl, 0xF, 0xF, false))
    FMOE_DPP_MAX(0xB1);      // quad_perm [1,0,3,2]
    FMOE_DPP_MAX(0x4E);      // quad_perm [2,3,0,1]
    FMOE_DPP_MAX(0x141);     // row_half_mirror
    if (LPT == 16) FMOE_DPP_MAX(0x140);     // row_mirror
#undef FMOE_DPP_MAX
    return v;
}

// Orders this wave's LDS accesses for the compiler.  The hardware runs a wave's LDS instructions in
// order, and the regions touched between two of these belong to one wave: no block barrier needed.
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One token per LPT lanes (8 or 16: a token's lanes sit in one DPP row), VPL scores per lane
// (expert id = v*LPT + sub).  K rounds of "largest remaining key, lowest expert id among equal
// keys", each two group maxima on the DPP network; the round is the slot (descending score,
// ties -> lower expert id).
template <typename T, int LPT, int VPL, int WPB>
__global__ __launch_bounds__(WPB * kWave) void topk_hist_kernel(const T* __restrict__ scores, int64_t num_tokens,
                                                        int E, int K, int renorm, int64_t tokens_per_wave,
                                                        int64_t* __restrict__ topk_idx,
                                                        T* __restrict__ gates,
                                                        uint16_t* __restrict__ compact,
                                                        int32_t* __restrict__ sub_hist,
                                                        int32_t* __restrict__ tot_hist) {
    constexpr int TPW = kWave / LPT;          // tokens per wave and pass
    constexpr int NT = WPB * kWave;
    __shared__ float s_sel[WPB][TPW][64];     // selected scores by slot (K <= 64)
    extern __shared__ int32_t s_hist[];       // [WPB][E] experts chosen by this wave's tokens
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int sub = lane % LPT;
    const int grp = lane / LPT;
    for (int i = threadIdx.x; i < WPB * E; i += NT) s_hist[i] = 0;
    __syncthreads();
    // this wave's tokens: a contiguous range, TPW of them per pass; every wave of the grid makes
    // the same number of passes (the block-wide barriers below sit inside the loop)
    const int64_t w_begin = ((int64_t)blockIdx.x * WPB + wave) * tokens_per_wave;
    int64_t w_end = w_begin + tokens_per_wave;
    if (w_end > num_tokens) w_end = num_tokens;
    const int64_t passes = (tokens_per_wave + TPW - 1) / TPW;
    const float ninf = -__builtin_inff();
    // the scores of the next pass are fetched while this one is ranked (as long as registers allow)
    constexpr bool AHEAD = VPL <= 8;
    float ahead[AHEAD ? VPL : 1];
#pragma unroll
    for (int v = 0; v < (AHEAD ? VPL : 0); ++v) {
        const int e = v * LPT + sub;
        const int64_t t0 = w_begin + grp;
        ahead[v] = (t0 < w_end && e < E) ? load_score<T>(scores + t0 * E + e) : ninf;
    }
    for (int64_t pass = 0; pass < passes; ++pass) {
        const int64_t t = w_begin + pass * TPW + grp;
        const bool live = t < w_end;

        float my[VPL];
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            const int e = v * LPT + sub;
            if (AHEAD) {
                my[v] = ahead[v];
                const int64_t tn = t + TPW;
                ahead[v] = (tn < w_end && e < E) ? load_score<T>(scores + tn * E + e) : ninf;
            } else {
                my[v] = (live && e < E) ? load_score<T>(scores + t * E + e) : ninf;
            }
        }
        // modes 2 and 3: the inputs are logits; they are L2-normalised over the experts first
        // (F.normalize: l / max(||l||, 1e-12), rounded to the logits' dtype), and it is the
        // normalised values that are ranked: rounding can tie values that differed before
        if (renorm >= 2) {
            float sq = 0.0f;
#pragma unroll
            for (int v = 0; v < VPL; ++v) {
                const int e = v * LPT + sub;
                if (live && e < E) sq += my[v] * my[v];
            }
#pragma unroll
            for (int o = LPT / 2; o >= 1; o >>= 1) sq += __shfl_xor(sq, o, kWave);
            const float norm = fmaxf(round_to<T>(sqrtf(sq)), 1e-12f);
#pragma unroll
            for (int v = 0; v < VPL; ++v) {
                const int e = v * LPT + sub;
                if (live && e < E) my[v] = round_to<T>(my[v] / norm);
            }
        }
        int rank[VPL];
        uint32_t work[VPL];
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            rank[v] = K;                                                   // not selected
            // (a key is never 0: -inf maps to 0x007fffff; 0 marks "taken" and the lanes past E)
            work[v] = (live && v * LPT + sub < E) ? order_key(my[v]) : 0u;
        }
        for (int r = 0; r < K; ++r) {
            uint32_t best = work[0];
            int bv = 0;
#pragma unroll
            for (int v = 1; v < VPL; ++v)
                if (work[v] > best) {                  // strictly: equal keys keep the lower expert id
                    best = work[v];
                    bv = v;
                }
            const uint32_t top = group_max_u32<LPT>(best);
            const uint32_t cand = best == top ? 0x3FFu - (uint32_t)(bv * LPT + sub) : 0u;
            const int win = (int)(0x3FFu - group_max_u32<LPT>(cand));     // this round's winner in the group
#pragma unroll
            for (int v = 0; v < VPL; ++v)
                if (v * LPT + sub == win) {
                    rank[v] = r;
                    work[v] = 0u;
                }
        }
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            const int e = v * LPT + sub;
            if (live && e < E && rank[v] < K) s_sel[wave][grp][rank[v]] = my[v];
        }
        // gates of modes 2 and 3: softmax of the normalised logits over all experts (2) or over
        // the K selected ones (3)
        float soft_sum = 0.0f;
        wave_lds_fence();
        if (renorm == 2) {
            // the largest normalised logit is slot 0; exp(n_i - n_max) summed over all experts
            const float nmax0 = live ? s_sel[wave][grp][0] : 0.0f;
#pragma unroll
            for (int v = 0; v < VPL; ++v) {
                const int e = v * LPT + sub;
                if (live && e < E) soft_sum += expf(my[v] - nmax0);
            }
#pragma unroll
            for (int o = LPT / 2; o >= 1; o >>= 1) soft_sum += __shfl_xor(soft_sum, o, kWave);
        }
        if (live) {
            float denom = 1.0f;
            if (renorm == 1) {
                float s = 0.0f;
                for (int j = 0; j < K; ++j) s = s + fabsf(s_sel[wave][grp][j]);   // slot order
                // (clamp_min keeps a NaN norm, fmaxf would drop it)
                denom = s != s ? s : fmaxf(round_to<T>(s), round_to<T>(1e-12f));
            }
            float nmax = 0.0f;
            if (renorm >= 2) {
                nmax = s_sel[wave][grp][0];
                if (renorm == 3) {
                    soft_sum = 0.0f;
                    for (int j = 0; j < K; ++j) soft_sum += expf(s_sel[wave][grp][j] - nmax);
                }
            }
#pragma unroll
            for (int v = 0; v < VPL; ++v) {
                const int e = v * LPT + sub;
                if (e < E && rank[v] < K) {
                    const int64_t p = t * K + rank[v];
                    topk_idx[p] = e;
                    compact[p] = (uint16_t)e;
                    atomicAdd(&s_hist[wave * E + e], 1);      // integer counts in LDS: exact
                    float g = my[v];
                    if (renorm == 1) g = round_to<T>(my[v] / denom);
                    else if (renorm >= 2) g = round_to<T>(expf(my[v] - nmax) / soft_sum);
                    store_score<T>(gates + p, g);
                }
            }
        }
        wave_lds_fence();       // s_sel is rewritten by the next pass
    }
    __syncthreads();
    for (int i = threadIdx.x; i < WPB * E; i += NT) sub_hist[(int64_t)blockIdx.x * WPB * E + i] = s_hist[i];
    for (int e = threadIdx.x; e < E; e += NT) {
        int32_t tot = 0;
#pragma unroll
        for (int w = 0; w < WPB; ++w) tot += s_hist[w * E + e];
        tot_hist[(int64_t)blockIdx.x * E + e] = tot;
    }
}

// Expert ids supplied by the caller (int64): narrow to the compact form, count them per wave
// and chunk as above, count the out-of-range ids of the chunk.
__global__ __launch_bounds__(1024) void compact_hist_kernel(const int64_t* __restrict__ topk_idx,
                                                            int64_t num_tokens, int E, int K,
                                                            int64_t tokens_per_wave,
                                                            uint16_t* __restrict__ compact,
                                                            int32_t* __restrict__ sub_hist,
                                                            int32_t* __restrict__ tot_hist,
                                                            int32_t* __restrict__ bad_part) {
    const int WPB = blockDim.x / kWave, NT = blockDim.x;
    extern __shared__ int32_t s_hist[];       // [WPB][E], then [WPB] bad counts
    int32_t* s_bad = s_hist + WPB * E;
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    for (int i = threadIdx.x; i < WPB * E + WPB; i += NT) s_hist[i] = 0;
    __syncthreads();
    const int64_t w_begin = ((int64_t)blockIdx.x * WPB + wave) * tokens_per_wave;
    int64_t w_end = w_begin + tokens_per_wave;
    if (w_end > num_tokens) w_end = num_tokens;
    int bad = 0;
    for (int64_t p = w_begin * K + lane; p < w_end * K; p += kWave) {
        const int64_t e = topk_idx[p];
        const bool ok = e >= 0 && e < E;
        compact[p] = ok ? (uint16_t)e : kBadExpert;
        if (ok) atomicAdd(&s_hist[wave * E + (int)e], 1);
        else ++bad;
    }
    if (bad) atomicAdd(&s_bad[wave], bad);
    __syncthreads();
    for (int i = threadIdx.x; i < WPB * E; i += NT) sub_hist[(int64_t)blockIdx.x * WPB * E + i] = s_hist[i];
    for (int e = threadIdx.x; e < E; e += NT) {
        int32_t tot = 0;
        for (int w = 0; w < WPB; ++w) tot += s_hist[w * E + e];
        tot_hist[(int64_t)blockIdx.x * E + e] = tot;
    }
    if (threadIdx.x == 0) {
        int32_t b = 0;
        for (int w = 0; w < WPB; ++w) b += s_bad[w];
        bad_part[blockIdx.x] = b;
    }
}

// Block = chunk, 4 or 16 waves.  Phase 1: per expert, the rows of all chunks (lengths) and of the chunks
// before this one.  Phase 2: wave scan over the experts = offsets.  Phase 3: every wave starts
// from offsets + rows of earlier chunks + rows of the earlier waves of its chunk and places its
// positions.  Each pass takes TPI = 64/K whole tokens, lane i <-> position begin + pass*TPI*K + i,
// so the K slots of a token sit in one pass.  s_next[e] is the next free slot of expert e.
__global__ __launch_bounds__(1024) void scan_scatter_kernel(const uint16_t* __restrict__ compact,
                                                           int64_t num_tokens, int64_t tokens_per_wave,
                                                           int E, int K, int ebits, int num_chunks,
                                                           const int32_t* __restrict__ sub_hist,
                                                           const int32_t* __restrict__ tot_hist,
                                                           const int32_t* __restrict__ bad_part,
                                                           int64_t* __restrict__ lengths,
                                                           int64_t* __restrict__ offsets,
                                                           int64_t* __restrict__ gate_index,
                                                           int64_t* __restrict__ token_index,
                                                           int64_t* __restrict__ reverse_index,
                                                           int64_t* __restrict__ bad_count) {
    const int WPB = blockDim.x / kWave;
    extern __shared__ int32_t smem[];
    int32_t* s_tot = smem;                    // [WPB][E] partial sums over a share of the chunks
    int32_t* s_bef = smem + WPB * E;          // [WPB][E] ... restricted to the chunks before this one
    int32_t* s_base = smem + 2 * WPB * E;     // [E] first slot of this chunk's rows of expert e
    int32_t* s_next = smem + 2 * WPB * E + E; // [WPB][E]: first this chunk's counts per wave, then the next free slots
    const int c = blockIdx.x;
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    {   // phase 1: wave w sums chunks [w * q, (w + 1) * q)
        const int q = (num_chunks + WPB - 1) / WPB;
        const int c_lo = wave * q, c_hi = (wave + 1) * q < num_chunks ? (wave + 1) * q : num_chunks;
        for (int e0 = 0; e0 < E; e0 += kWave) {
            const int e = e0 + lane;
            int32_t tot = 0, bef = 0;
            if (e < E) {
                // (this wave's own counts of the chunk ride along with the first loads)
                s_next[wave * E + e] = sub_hist[((int64_t)c * WPB + wave) * E + e];
#pragma unroll 8
                for (int cc = c_lo; cc < c_hi; ++cc) {
                    const int32_t v = tot_hist[(int64_t)cc * E + e];
                    tot += v;
                    bef += cc < c ? v : 0;
                }
                s_tot[wave * E + e] = tot;
                s_bef[wave * E + e] = bef;
            }
        }
    }
    __syncthreads();
    if (wave == 0) {    // phase 2: exclusive prefix of the lengths over the experts; chunk 0 publishes
        long long run = 0;
        for (int e0 = 0; e0 < E; e0 += kWave) {
            const int e = e0 + lane;
            long long len = 0;
            int32_t bef = 0;
            if (e < E)
                for (int w = 0; w < WPB; ++w) {
                    len += s_tot[w * E + e];
                    bef += s_bef[w * E + e];
                }
            const long long inc = wave_inclusive_scan(len);
            if (e < E) {
                s_base[e] = (int32_t)(run + inc - len) + bef;
                if (c == 0) {
                    lengths[e] = len;
                    offsets[e] = run + inc - len;
                }
            }
            run += wave_bcast(inc, kWave - 1);
        }
        if (c == 0) {
            if (lane == 0) offsets[E] = run;
            // positions dropped for an out-of-range expert id leave a tail behind the last expert's
            // rows: it holds zeros rather than whatever the buffer held (normally the tail is empty)
            for (long long i = run + lane; i < (long long)num_tokens * K; i += kWave) {
                gate_index[i] = 0;
                token_index[i] = 0;
            }
            if (bad_count) {
                long long bad = 0;
                if (bad_part)
                    for (int cc = lane; cc < num_chunks; cc += kWave) bad += bad_part[cc];
#pragma unroll
                for (int o = 32; o >= 1; o >>= 1) bad += __shfl_xor(bad, o, kWave);
                if (lane == 0) *bad_count = bad;
            }
        }
    }
    __syncthreads();
    // phase 3: the counts of the earlier waves of the chunk (LDS) on top of the chunk's base
    int32_t at[16];             // E <= 1024: at most 16 entries per lane
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int e = i * kWave + lane;
        at[i] = 0;
        if (e < E) {
            at[i] = s_base[e];
            for (int w = 0; w < wave; ++w) at[i] += s_next[w * E + e];
        }
    }
    __syncthreads();            // every wave has read the counts before anyone overwrites them
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int e = i * kWave + lane;
        if (e < E) s_next[wave * E + e] = at[i];
    }
    __syncthreads();
    int32_t* next = s_next + wave * E;
    const int tpi = kWave / K;
    const int64_t t_begin = ((int64_t)c * WPB + wave) * tokens_per_wave;
    int64_t t_end = t_begin + tokens_per_wave;
    if (t_end > num_tokens) t_end = num_tokens;
    const int64_t passes = (tokens_per_wave + tpi - 1) / tpi;     // the same for every wave (barriers below)
    const int tok_in_iter = lane / K;
    const int slot = lane - tok_in_iter * K;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int64_t pass = 0; pass < passes; ++pass) {
        const int64_t t = t_begin + pass * tpi + tok_in_iter;
        const bool live = tok_in_iter < tpi && t < t_end;
        const int64_t p = t * K + slot;
        const uint32_t e = live ? compact[p] : (uint32_t)kBadExpert;
        const bool counted = live && e != kBadExpert;
        // lanes holding the same expert id
        uint64_t same = __ballot(counted);
        for (int b = 0; b < ebits; ++b) {
            const uint64_t bal = __ballot((e >> b) & 1u);
            same &= ((e >> b) & 1u) ? bal : ~bal;
        }
        const int before = __popcll(same & lt_mask);
        const int count = __popcll(same);
        int32_t base = 0;
        if (counted) base = next[e];
        wave_lds_fence();
        if (counted && before == 0) next[e] = base + count;
        wave_lds_fence();
        const int64_t dst = (int64_t)base + before;
        // rank of this slot among the token's K slots, ordered by (expert, slot)
        int rank = 0;
        for (int j = 0; j < K; ++j) {
            const uint32_t oe = __shfl(e, tok_in_iter * K + j, kWave);
            rank += (oe < e || (oe == e && j < slot)) ? 1 : 0;
        }
        if (counted) {
            gate_index[dst] = p;
            token_index[dst] = t;
            reverse_index[t * K + rank] = dst;
        } else if (live) {
            reverse_index[t * K + rank] = 0;    // a dropped position (out-of-range id): sorts last in its token
        }
    }
}

int ceil_log2(int v) {
    int b = 0;
    while ((1 << b) < v) ++b;
    return b;
}

int launch_sort(const RouteScratch& ws, const RoutePlan& plan, bool have_bad, int64_t T, int E, int K,
                int64_t* lengths, int64_t* offsets, int64_t* gate_index, int64_t* token_index,
                int64_t* reverse_index, int64_t* bad_count, hipStream_t stream) {
    const size_t lds = (size_t)(3 * plan.wpb + 1) * E * sizeof(int32_t);
    scan_scatter_kernel<<<plan.num_chunks, plan.wpb * kWave, lds, stream>>>(
        ws.compact, T, plan.tokens_per_wave, E, K, ceil_log2(E), plan.num_chunks, ws.sub_hist, ws.tot_hist,
        have_bad ? ws.bad_part : nullptr, lengths, offsets, gate_index, token_index, reverse_index, bad_count);
    return check_launch("routing sort");
}

template <typename T, int LPT, int VPL>
void launch_topk(const void* scores, int64_t T_, int E, int K, int renorm, int64_t* topk_idx,
                 void* gates, const RouteScratch& ws, const RoutePlan& plan, hipStream_t stream) {
    const size_t lds = (size_t)plan.wpb * E * sizeof(int32_t);
    if (plan.wpb == 16)
        topk_hist_kernel<T, LPT, VPL, 16><<<plan.num_chunks, 16 * kWave, lds, stream>>>(
            (const T*)scores, T_, E, K, renorm, plan.tokens_per_wave, topk_idx, (T*)gates, ws.compact, ws.sub_hist,
            ws.tot_hist);
    else
        topk_hist_kernel<T, LPT, VPL, 4><<<plan.num_chunks, 4 * kWave, lds, stream>>>(
            (const T*)scores, T_, E, K, renorm, plan.tokens_per_wave, topk_idx, (T*)gates, ws.compact, ws.sub_hist,
            ws.tot_hist);
}

template <typename T>
int dispatch_topk(const void* scores, int64_t T_, int E, int K, int renorm, int64_t* topk_idx,
                  void* gates, const RouteScratch& ws, const RoutePlan& plan, hipStream_t stream) {
#define FMOE_TOPK(LPT, VPL) launch_topk<T, LPT, VPL>(scores, T_, E, K, renorm, topk_idx, gates, ws, plan, stream)
    if (E <= 8) FMOE_TOPK(8, 1);
    else if (E <= 16) FMOE_TOPK(16, 1);
    else if (E <= 32) FMOE_TOPK(16, 2);
    else if (E <= 64) FMOE_TOPK(16, 4);
    else if (E <= 128) FMOE_TOPK(16, 8);
    else if (E <= 256) FMOE_TOPK(16, 16);
    else if (E <= 512) FMOE_TOPK(16, 32);
    else return fail(FMOE_ERR_UNSUPPORTED, "fmoe_route_topk: E=%d > 512", E);
#undef FMOE_TOPK
    return FMOE_OK;
}

int check_common(int64_t T, int E, int K, const void* workspace, size_t ws_bytes, const char* who) {
    FMOE_REQUIRE(T >= 0 && E >= 1 && K >= 1, "%s: need T >= 0, E >= 1, K >= 1 (T=%lld E=%d K=%d)", who,
                 (long long)T, E, K);
    FMOE_REQUIRE(K <= 64, "%s: K=%d > 64 is not supported", who, K);
    FMOE_REQUIRE(E <= 1024, "%s: E=%d > 1024 is not supported", who, E);
    FMOE_REQUIRE(T * (int64_t)K < (int64_t)1 << 31, "%s: T*K must be below 2^31", who);
    const RoutePlan plan = make_plan(T, E, K);
    if (T > 0) {
        FMOE_REQUIRE(workspace != nullptr, "%s: workspace is NULL", who);
        if (ws_bytes < plan.total_bytes)
            return fail(FMOE_ERR_WORKSPACE, "%s: workspace %zu B < required %zu B", who, ws_bytes,
                        plan.total_bytes);
    }
    return FMOE_OK;
}

__global__ void empty_routing_kernel(int E, int64_t* lengths, int64_t* offsets, int64_t* bad_count) {
    for (int e = threadIdx.x; e < E; e += blockDim.x) lengths[e] = 0;
    for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = 0;
    if (bad_count && threadIdx.x == 0) *bad_count = 0;
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

extern "C" size_t fmoe_route_workspace_bytes(int64_t T, int E, int K) {
    if (T < 0 || E < 1 || K < 1) return 0;
    return make_plan(T, E, K).total_bytes;
}

static int route_topk_impl(const char* who, const void* scores, int score_dtype, int64_t T, int E, int K, int renorm,
                           int64_t* topk_idx, void* gates, int64_t* lengths, int64_t* offsets,
                           int64_t* gate_index, int64_t* token_index, int64_t* reverse_index,
                           void* workspace, size_t workspace_bytes, hipStream_t stream) {
    if (int rc = check_common(T, E, K, workspace, workspace_bytes, who)) return rc;
    FMOE_REQUIRE(K <= E, "%s: K=%d > E=%d", who, K, E);
    FMOE_REQUIRE(renorm >= 0 && renorm <= 3, "%s: gate mode %d is not one of 0..3", who, renorm);
    FMOE_REQUIRE(score_dtype == FMOE_F32 || score_dtype == FMOE_BF16, "%s: scores must be fp32 or bf16", who);
    FMOE_REQUIRE(lengths && offsets, "%s: lengths/offsets are NULL", who);
    if (T == 0) {
        empty_routing_kernel<<<1, 256, 0, stream>>>(E, lengths, offsets, nullptr);
        return check_launch(who);
    }
    FMOE_REQUIRE(scores && topk_idx && gates && gate_index && token_index && reverse_index,
                 "%s: NULL tensor pointer", who);
    const RoutePlan plan = make_plan(T, E, K);
    const RouteScratch ws = carve(workspace, plan);
    int rc = score_dtype == FMOE_F32
                 ? dispatch_topk<float>(scores, T, E, K, renorm, topk_idx, gates, ws, plan, stream)
                 : dispatch_topk<uint16_t>(scores, T, E, K, renorm, topk_idx, gates, ws, plan, stream);
    if (rc) return rc;
    return launch_sort(ws, plan, false, T, E, K, lengths, offsets, gate_index, token_index, reverse_index, nullptr,
                       stream);
}

extern "C" int fmoe_route_topk(const void* scores, int score_dtype, int64_t T, int E, int K, int renorm,
                               int64_t* topk_idx, void* gates, int64_t* lengths, int64_t* offsets,
                               int64_t* gate_index, int64_t* token_index, int64_t* reverse_index,
                               void* workspace, size_t workspace_bytes, fmoe_stream_t stream_) {
    return route_topk_impl("fmoe_route_topk", scores, score_dtype, T, E, K, renorm, topk_idx, gates, lengths,
                           offsets, gate_index, token_index, reverse_index, workspace, workspace_bytes,
                           (hipStream_t)stream_);
}

// ------------------------------------------------------------ allocation-free variant
// The routing scratch (one uint16 expert id per routed position + the per-chunk histograms) in
// device memory that belongs to the library image: one copy per GPU the library runs on, held
// until the process ends.  In host code `scratch` is only a handle for hipGetSymbolAddress;
// the address kernels and copies use is the per-device pointer looked up below.
static constexpr size_t kStaticCompactBytes = (size_t)FMOE_ROUTE_STATIC_MAX_POSITIONS * sizeof(uint16_t);
// (16 waves per block up to 256 experts, 4 beyond: 17 * 256 > 5 * 512)
static constexpr size_t kStaticHistBytes = (size_t)kMaxChunks * (kMaxRouteWaves + 1) * 256 * sizeof(int32_t);
static constexpr size_t kStaticScratchBytes = kStaticCompactBytes + kStaticHistBytes + kMaxChunks * 4 + 1280;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];     // device address of `scratch` on each GPU, 0 = not looked up yet
static std::mutex g_scratch_mutex;

// Device address of this GPU's copy of `scratch` (looked up once per device, with that device current).
static int static_scratch(void** out, const char* who) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(FMOE_ERR_LAUNCH, "%s: no current device (or device index beyond %d)", who, kMaxDevices - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess || ptr == nullptr)
            return fail(FMOE_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev,
                        hipGetErrorString(err));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return FMOE_OK;
}

extern "C" int fmoe_route_topk_static(const void* scores, int score_dtype, int64_t T, int E, int K, int renorm,
                                      int64_t* topk_idx, void* gates, int64_t* lengths, int64_t* offsets,
                                      int64_t* gate_index, int64_t* token_index, int64_t* reverse_index,
                                      fmoe_stream_t stream_) {
    const char* who = "fmoe_route_topk_static";
    FMOE_REQUIRE(T >= 0 && E >= 1 && K >= 1, "%s: need T >= 0, E >= 1, K >= 1 (T=%lld E=%d K=%d)", who,
                 (long long)T, E, K);
    FMOE_REQUIRE(E <= FMOE_ROUTE_STATIC_MAX_EXPERTS, "%s: E=%d exceeds the %d experts the built-in scratch holds",
                 who, E, FMOE_ROUTE_STATIC_MAX_EXPERTS);
    FMOE_REQUIRE(T <= FMOE_ROUTE_STATIC_MAX_POSITIONS && T * (int64_t)K <= FMOE_ROUTE_STATIC_MAX_POSITIONS,
                 "%s: T*K=%lld routed positions exceed the %d the built-in scratch holds (use fmoe_route_topk "
                 "with a workspace)", who, (long long)T * K, FMOE_ROUTE_STATIC_MAX_POSITIONS);
    // every check that can refuse the call comes before the scratch lookup, so that a refused call
    // never touches the runtime (the first lookup on a device calls hipGetSymbolAddress)
    FMOE_REQUIRE(K <= 64 && K <= E, "%s: K=%d must be at most 64 and at most E=%d", who, K, E);
    FMOE_REQUIRE(renorm >= 0 && renorm <= 3, "%s: gate mode %d is not one of 0..3", who, renorm);
    FMOE_REQUIRE(score_dtype == FMOE_F32 || score_dtype == FMOE_BF16, "%s: scores must be fp32 or bf16", who);
    FMOE_REQUIRE(lengths && offsets, "%s: lengths/offsets are NULL", who);
    if (T > 0)
        FMOE_REQUIRE(scores && topk_idx && gates && gate_index && token_index && reverse_index,
                     "%s: NULL tensor pointer", who);
    if (make_plan(T, E, K).total_bytes > kStaticScratchBytes)
        return fail(FMOE_ERR_WORKSPACE, "%s: the call needs %zu B of scratch, the built-in buffer has %zu B", who,
                    make_plan(T, E, K).total_bytes, kStaticScratchBytes);
    void* ptr = nullptr;
    if (int rc = static_scratch(&ptr, who)) return rc;
    // nothing in the buffer has to start at zero: the first two kernels overwrite every byte the later ones read
    return route_topk_impl(who, scores, score_dtype, T, E, K, renorm, topk_idx, gates, lengths, offsets, gate_index,
                           token_index, reverse_index, ptr, kStaticScratchBytes, (hipStream_t)stream_);
}

extern "C" int fmoe_route_from_topk(const int64_t* topk_idx, int64_t T, int E, int K, int64_t* lengths,
                                    int64_t* offsets, int64_t* gate_index, int64_t* token_index,
                                    int64_t* reverse_index, int64_t* bad_count, void* workspace,
                                    size_t workspace_bytes, fmoe_stream_t stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (int rc = check_common(T, E, K, workspace, workspace_bytes, "fmoe_route_from_topk")) return rc;
    FMOE_REQUIRE(lengths && offsets, "fmoe_route_from_topk: lengths/offsets are NULL");
    if (T == 0) {
        empty_routing_kernel<<<1, 256, 0, stream>>>(E, lengths, offsets, bad_count);
        return check_launch("fmoe_route_from_topk");
    }
    FMOE_REQUIRE(topk_idx && gate_index && token_index && reverse_index,
                 "fmoe_route_from_topk: NULL tensor pointer");
    const RoutePlan plan = make_plan(T, E, K);
    const RouteScratch ws = carve(workspace, plan);
    compact_hist_kernel<<<plan.num_chunks, plan.wpb * kWave, ((size_t)plan.wpb * E + plan.wpb) * sizeof(int32_t), stream>>>(
        topk_idx, T, E, K, plan.tokens_per_wave, ws.compact, ws.sub_hist, ws.tot_hist, ws.bad_part);
    return launch_sort(ws, plan, true, T, E, K, lengths, offsets, gate_index, token_index, reverse_index, bad_count,
                       stream);
}
