// Routing for the MoE forward: top-k selection with L1-renormalised gates, the
// per-expert histogram / prefix sum ("jagged offsets") and the stable
// expert-major permutation with its inverse.  All integer outputs are a pure
// function of the selected ids (a stable counting sort), so they are
// reproducible bit for bit.
//
// Pipeline (4 launches on one stream, no host synchronisation):
//   1. topk_kernel     rank-by-counting selection, one token per LPT lanes
//   2. hist_kernel     one wave per chunk of tokens: LDS histogram -> chunk_hist[c][e]
//   3. scan_kernel     one block per expert: exclusive scan of chunk_hist over the
//                      chunks (in place, wave scans), lengths[e]
//   4. scatter_kernel  one wave per chunk: offsets = wave scan of lengths, then a
//                      wave-level match/rank gives each position its slot inside
//                      its expert segment
#include "common.h"

#include <mutex>

namespace fmoe {
namespace {

constexpr int kMaxChunks = 512;
constexpr uint16_t kBadExpert = 0xFFFF;

struct RoutePlan {
    int64_t tokens_per_chunk;
    int num_chunks;
    size_t compact_bytes;   // uint16 expert id per routed position
    size_t hist_bytes;      // int32 [num_chunks][E]
    size_t total_bytes;
};

RoutePlan make_plan(int64_t T, int E, int K) {
    RoutePlan p;
    p.tokens_per_chunk = (T + kMaxChunks - 1) / kMaxChunks;
    if (p.tokens_per_chunk < 1) p.tokens_per_chunk = 1;
    p.num_chunks = (int)((T + p.tokens_per_chunk - 1) / p.tokens_per_chunk);
    if (p.num_chunks < 1) p.num_chunks = 1;
    size_t compact = (size_t)T * (size_t)K * sizeof(uint16_t);
    p.compact_bytes = (compact + 255) & ~(size_t)255;
    p.hist_bytes = ((size_t)p.num_chunks * (size_t)E * sizeof(int32_t) + 255) & ~(size_t)255;
    p.total_bytes = p.compact_bytes + p.hist_bytes + 256;
    return p;
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

// One token per LPT lanes, VPL scores per lane (expert id = v*LPT + sub).  The
// rank of a score is the number of scores that beat it (greater key, or equal key with
// a lower expert id); rank < K selects it and is its slot.
template <typename T, int LPT, int VPL>
__global__ __launch_bounds__(256) void topk_kernel(const T* __restrict__ scores, int64_t num_tokens,
                                                   int E, int K, int renorm,
                                                   int64_t* __restrict__ topk_idx,
                                                   T* __restrict__ gates,
                                                   uint16_t* __restrict__ compact) {
    constexpr int TPW = kWave / LPT;          // tokens per wave
    constexpr int WPB = 256 / kWave;
    __shared__ float s_sel[WPB][TPW][64];     // selected scores by slot (K <= 64)
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int sub = lane % LPT;
    const int grp = lane / LPT;
    const int64_t t = ((int64_t)blockIdx.x * WPB + wave) * TPW + grp;
    const bool live = t < num_tokens;

    float my[VPL];
    const float ninf = -__builtin_inff();
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const int e = v * LPT + sub;
        my[v] = (live && e < E) ? load_score<T>(scores + t * E + e) : ninf;
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
    uint32_t key[VPL];
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        rank[v] = 0;
        key[v] = order_key(my[v]);
    }
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            // a full wave per token: the broadcast lane is a compile-time constant (v_readlane)
            const uint32_t other = LPT == kWave ? (uint32_t)__builtin_amdgcn_readlane((int)key[u], i)
                                                : (uint32_t)__shfl((int)key[u], grp * LPT + i, kWave);
            const int oe = u * LPT + i;
#pragma unroll
            for (int v = 0; v < VPL; ++v) {
                const int e = v * LPT + sub;
                rank[v] += (other > key[v] || (other == key[v] && oe < e)) ? 1 : 0;
            }
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
    __syncthreads();
    if (renorm == 2) {
        // the largest normalised logit is slot 0; exp(n_i - n_max) summed over all experts
        const float nmax = live ? s_sel[wave][grp][0] : 0.0f;
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            const int e = v * LPT + sub;
            if (live && e < E) soft_sum += expf(my[v] - nmax);
        }
#pragma unroll
        for (int o = LPT / 2; o >= 1; o >>= 1) soft_sum += __shfl_xor(soft_sum, o, kWave);
    }
    if (!live) return;
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
            float g = my[v];
            if (renorm == 1) g = round_to<T>(my[v] / denom);
            else if (renorm >= 2) g = round_to<T>(expf(my[v] - nmax) / soft_sum);
            store_score<T>(gates + p, g);
        }
    }
}

// Expert ids supplied by the caller (int64): narrow to the compact form, flag
// out-of-range ids.
__global__ __launch_bounds__(256) void compact_kernel(const int64_t* __restrict__ topk_idx, int64_t n,
                                                      int E, uint16_t* __restrict__ compact,
                                                      int64_t* __restrict__ bad_count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t e = topk_idx[i];
    const bool ok = e >= 0 && e < E;
    compact[i] = ok ? (uint16_t)e : kBadExpert;
    if (!ok && bad_count) atomicAdd((unsigned long long*)bad_count, 1ull);
}

__global__ void zero_i64_kernel(int64_t* p) { *p = 0; }

// One wave per chunk of tokens; counts are integers, so LDS atomics are exact.
__global__ __launch_bounds__(kWave) void hist_kernel(const uint16_t* __restrict__ compact,
                                                     int64_t total_pos, int64_t pos_per_chunk, int E,
                                                     int32_t* __restrict__ chunk_hist) {
    extern __shared__ int32_t s_cnt[];
    const int c = blockIdx.x;
    for (int e = threadIdx.x; e < E; e += kWave) s_cnt[e] = 0;
    __syncthreads();
    const int64_t begin = (int64_t)c * pos_per_chunk;
    int64_t end = begin + pos_per_chunk;
    if (end > total_pos) end = total_pos;
    for (int64_t p = begin + threadIdx.x; p < end; p += kWave) {
        const uint16_t e = compact[p];
        if (e != kBadExpert) atomicAdd(&s_cnt[e], 1);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += kWave) chunk_hist[(int64_t)c * E + e] = s_cnt[e];
}

// One block per expert: exclusive scan of that expert's counts over the chunks (in place)
// and its total.  256 threads, two chunks per thread (num_chunks <= 512).
__global__ __launch_bounds__(256) void scan_kernel(int32_t* __restrict__ chunk_hist, int num_chunks, int E,
                                                   int64_t* __restrict__ lengths) {
    __shared__ int32_t s_wave[4];
    const int e = blockIdx.x;
    const int c0 = threadIdx.x * 2, c1 = c0 + 1;
    const int32_t v0 = c0 < num_chunks ? chunk_hist[(int64_t)c0 * E + e] : 0;
    const int32_t v1 = c1 < num_chunks ? chunk_hist[(int64_t)c1 * E + e] : 0;
    const int inc = wave_inclusive_scan((int)(v0 + v1));
    const int wave = threadIdx.x / kWave;
    if (lane_id() == kWave - 1) s_wave[wave] = inc;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += s_wave[w];
    const int excl = base + inc - (v0 + v1);
    if (c0 < num_chunks) chunk_hist[(int64_t)c0 * E + e] = excl;
    if (c1 < num_chunks) chunk_hist[(int64_t)c1 * E + e] = excl + v0;
    if (threadIdx.x == 255) lengths[e] = base + inc;
}

// One wave per chunk.  Each iteration takes TPI = 64/K whole tokens, lane i <->
// position chunk_begin + it*TPI*K + i, so the K slots of a token sit in one
// iteration.  s_next[e] is the next free slot of expert e for this chunk.
__global__ __launch_bounds__(kWave) void scatter_kernel(const uint16_t* __restrict__ compact,
                                                        int64_t num_tokens, int64_t tokens_per_chunk,
                                                        int E, int K, int ebits,
                                                        const int32_t* __restrict__ chunk_base,
                                                        const int64_t* __restrict__ lengths,
                                                        int64_t* __restrict__ offsets,
                                                        int64_t* __restrict__ gate_index,
                                                        int64_t* __restrict__ token_index,
                                                        int64_t* __restrict__ reverse_index) {
    extern __shared__ int32_t s_next[];
    const int c = blockIdx.x;
    const int lane = threadIdx.x;
    {   // exclusive prefix of lengths over the experts = offsets (wave scan); chunk 0 publishes it
        long long run = 0;
        for (int e0 = 0; e0 < E; e0 += kWave) {
            const int e = e0 + lane;
            const long long v = e < E ? (long long)lengths[e] : 0;
            const long long inc = wave_inclusive_scan(v);
            if (e < E) {
                s_next[e] = (int32_t)(run + inc - v) + chunk_base[(int64_t)c * E + e];
                if (c == 0) offsets[e] = run + inc - v;
            }
            run += wave_bcast(inc, kWave - 1);
        }
        if (c == 0 && lane == 0) offsets[E] = run;
        // positions dropped for an out-of-range expert id leave a tail behind the last expert's
        // rows: it holds zeros rather than whatever the buffer held (normally the tail is empty)
        if (c == 0)
            for (long long i = run + lane; i < (long long)num_tokens * K; i += kWave) {
                gate_index[i] = 0;
                token_index[i] = 0;
            }
    }
    __syncthreads();
    const int tpi = kWave / K;
    const int64_t t_begin = (int64_t)c * tokens_per_chunk;
    int64_t t_end = t_begin + tokens_per_chunk;
    if (t_end > num_tokens) t_end = num_tokens;
    const int tok_in_iter = lane / K;
    const int slot = lane - tok_in_iter * K;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int64_t t0 = t_begin; t0 < t_end; t0 += tpi) {
        const int64_t t = t0 + tok_in_iter;
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
        if (counted) base = s_next[e];
        __syncthreads();
        if (counted && before == 0) s_next[e] = base + count;
        __syncthreads();
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

int launch_sort(const uint16_t* compact, int32_t* chunk_hist, const RoutePlan& plan, int64_t T, int E,
                int K, int64_t* lengths, int64_t* offsets, int64_t* gate_index, int64_t* token_index,
                int64_t* reverse_index, hipStream_t stream) {
    const int64_t total_pos = T * K;
    hist_kernel<<<plan.num_chunks, kWave, E * sizeof(int32_t), stream>>>(
        compact, total_pos, plan.tokens_per_chunk * K, E, chunk_hist);
    scan_kernel<<<E, 256, 0, stream>>>(chunk_hist, plan.num_chunks, E, lengths);
    scatter_kernel<<<plan.num_chunks, kWave, E * sizeof(int32_t), stream>>>(
        compact, T, plan.tokens_per_chunk, E, K, ceil_log2(E), chunk_hist, lengths, offsets, gate_index,
        token_index, reverse_index);
    return check_launch("routing sort");
}

template <typename T, int LPT, int VPL>
void launch_topk(const void* scores, int64_t T_, int E, int K, int renorm, int64_t* topk_idx,
                 void* gates, uint16_t* compact, hipStream_t stream) {
    constexpr int tokens_per_block = (256 / kWave) * (kWave / LPT);
    const int64_t blocks = (T_ + tokens_per_block - 1) / tokens_per_block;
    topk_kernel<T, LPT, VPL><<<(unsigned)blocks, 256, 0, stream>>>(
        (const T*)scores, T_, E, K, renorm, topk_idx, (T*)gates, compact);
}

template <typename T>
int dispatch_topk(const void* scores, int64_t T_, int E, int K, int renorm, int64_t* topk_idx,
                  void* gates, uint16_t* compact, hipStream_t stream) {
#define FMOE_TOPK(LPT, VPL) launch_topk<T, LPT, VPL>(scores, T_, E, K, renorm, topk_idx, gates, compact, stream)
    if (E <= 8) FMOE_TOPK(8, 1);
    else if (E <= 16) FMOE_TOPK(16, 1);
    else if (E <= 32) FMOE_TOPK(32, 1);
    else if (E <= 64) FMOE_TOPK(64, 1);
    else if (E <= 128) FMOE_TOPK(64, 2);
    else if (E <= 256) FMOE_TOPK(64, 4);
    else if (E <= 512) FMOE_TOPK(64, 8);
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

__global__ void empty_routing_kernel(int E, int64_t* lengths, int64_t* offsets) {
    for (int e = threadIdx.x; e < E; e += blockDim.x) lengths[e] = 0;
    for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = 0;
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
        empty_routing_kernel<<<1, 256, 0, stream>>>(E, lengths, offsets);
        return check_launch(who);
    }
    FMOE_REQUIRE(scores && topk_idx && gates && gate_index && token_index && reverse_index,
                 "%s: NULL tensor pointer", who);
    const RoutePlan plan = make_plan(T, E, K);
    uint16_t* compact = (uint16_t*)workspace;
    int32_t* chunk_hist = (int32_t*)((char*)workspace + plan.compact_bytes);
    int rc = score_dtype == FMOE_F32
                 ? dispatch_topk<float>(scores, T, E, K, renorm, topk_idx, gates, compact, stream)
                 : dispatch_topk<uint16_t>(scores, T, E, K, renorm, topk_idx, gates, compact, stream);
    if (rc) return rc;
    return launch_sort(compact, chunk_hist, plan, T, E, K, lengths, offsets, gate_index, token_index,
                       reverse_index, stream);
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
static constexpr size_t kStaticHistBytes = (size_t)kMaxChunks * FMOE_ROUTE_STATIC_MAX_EXPERTS * sizeof(int32_t);
static constexpr size_t kStaticScratchBytes = kStaticCompactBytes + kStaticHistBytes + 512;
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
    if (bad_count) zero_i64_kernel<<<1, 1, 0, stream>>>(bad_count);
    if (T == 0) {
        empty_routing_kernel<<<1, 256, 0, stream>>>(E, lengths, offsets);
        return check_launch("fmoe_route_from_topk");
    }
    FMOE_REQUIRE(topk_idx && gate_index && token_index && reverse_index,
                 "fmoe_route_from_topk: NULL tensor pointer");
    const RoutePlan plan = make_plan(T, E, K);
    uint16_t* compact = (uint16_t*)workspace;
    int32_t* chunk_hist = (int32_t*)((char*)workspace + plan.compact_bytes);
    const int64_t n = T * K;
    compact_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(topk_idx, n, E, compact, bad_count);
    return launch_sort(compact, chunk_hist, plan, T, E, K, lengths, offsets, gate_index, token_index,
                       reverse_index, stream);
}
