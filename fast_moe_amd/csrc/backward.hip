// Backward helpers of the MoE path: operand transposition for the weight-gradient GEMM,
// bias gradients, SwiGLU / SiLU backward and the backward of the weighted merge.
#include "common.h"

namespace fmoe {
namespace {

template <typename T> struct Val;
template <> struct Val<uint16_t> {
    __device__ static float load(const uint16_t* p) { return bf16_bits_to_f32(*p); }
    __device__ static void store(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
    __device__ static float round(float v) { return round_bf16(v); }
};
template <> struct Val<float> {
    __device__ static float load(const float* p) { return *p; }
    __device__ static void store(float* p, float v) { *p = v; }
    __device__ static float round(float v) { return v; }
};

// 64 (padded rows) x 64 (columns) tile: every thread column finds the expert that owns its
// padded row by binary search in pad_offsets, reads the source row it maps to (or zero for
// padding) and the tile is written transposed through LDS.
template <typename T>
__global__ __launch_bounds__(256) void jagged_transpose_kernel(
    const T* __restrict__ src, int64_t src_rows, int64_t cols, int64_t src_stride,
    const int64_t* __restrict__ row_index, int index_div, const int64_t* __restrict__ offsets,
    const int64_t* __restrict__ pad_offsets, int E, T* __restrict__ dst, int64_t dst_stride,
    int64_t dst_cols, int apply_silu) {
    __shared__ T tile[64][64 + 2];
    __shared__ int64_t s_src[64];
    const int64_t p0 = (int64_t)blockIdx.x * 64, c0 = (int64_t)blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    if (threadIdx.x < 64) {
        const int64_t pcol = p0 + threadIdx.x;
        int64_t srow = -1;
        if (pcol < pad_offsets[E]) {
            int lo = 0, hi = E;               // largest e with pad_offsets[e] <= pcol
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (pad_offsets[mid] <= pcol) lo = mid; else hi = mid;
            }
            const int64_t j = pcol - pad_offsets[lo];
            const int64_t len = offsets[lo + 1] - offsets[lo];
            if (j >= 0 && j < len) {
                int64_t r = offsets[lo] + j;
                if (row_index) r = row_index[r] / index_div;
                if (r >= 0 && r < src_rows) srow = r;
            }
        }
        s_src[threadIdx.x] = srow;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int64_t r = s_src[i], c = c0 + tx;
        T v = 0;
        if (r >= 0 && c < cols) {
            v = src[r * src_stride + c];
            if (apply_silu) {
                float f = Val<T>::load(&v);
                Val<T>::store(&v, silu_f32(f));
            }
        }
        tile[i][tx] = v;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int64_t c = c0 + i, pcol = p0 + tx;
        if (c < cols && pcol < dst_cols) dst[c * dst_stride + pcol] = tile[tx][i];
    }
}

// bf16 fast path: 64 (padded rows) x 128 (columns) tile.  Source rows come in with 16-byte
// loads and go to LDS row-major; ds_read_b64_tr_b16 reads them back transposed (within 16
// lanes, lane j receives element j of 4 consecutive rows when lane i points at row i/4,
// elements 4*(i%4)..+3), so two such reads give a lane 8 consecutive padded rows of one
// column: one 16-byte store.  LDS rows are 320 bytes apart: the four rows of a 16-lane group
// and the two groups served in one pass then fall into eight different 32-byte bank groups.
typedef __attribute__((ext_vector_type(4))) short s16x4;
__global__ __launch_bounds__(256) void jagged_transpose_tr_kernel(
    const uint16_t* __restrict__ src, int64_t src_rows, int64_t cols, int64_t src_stride,
    const int64_t* __restrict__ row_index, int index_div, const int64_t* __restrict__ offsets,
    const int64_t* __restrict__ pad_offsets, int E, uint16_t* __restrict__ dst, int64_t dst_stride,
    int64_t dst_cols, int apply_silu) {
    constexpr int ROWB = 320;
    __shared__ __align__(16) uint8_t tile[64 * ROWB];
    __shared__ int64_t s_src[64];
    const int64_t p0 = (int64_t)blockIdx.x * 64, c0 = (int64_t)blockIdx.y * 128;
    const int tid = threadIdx.x;
    if (tid < 64) {
        const int64_t pcol = p0 + tid;
        int64_t srow = -1;
        if (pcol < pad_offsets[E]) {
            int lo = 0, hi = E;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (pad_offsets[mid] <= pcol) lo = mid; else hi = mid;
            }
            const int64_t j = pcol - pad_offsets[lo];
            const int64_t len = offsets[lo + 1] - offsets[lo];
            if (j >= 0 && j < len) {
                int64_t r = offsets[lo] + j;
                if (row_index) r = row_index[r] / index_div;
                if (r >= 0 && r < src_rows) srow = r;
            }
        }
        s_src[tid] = srow;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = (tid >> 4) + 16 * i, chunk = tid & 15;
        const int64_t r = s_src[row], c = c0 + chunk * 8;
        u32x4 v = {0, 0, 0, 0};
        if (r >= 0 && c < cols) {          // cols is a multiple of 8 on this path
            v = *reinterpret_cast<const u32x4*>(src + r * src_stride + c);
            if (apply_silu) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float lo = silu_f32(bf16_bits_to_f32(v[q] & 0xffffu));
                    const float hi = silu_f32(__uint_as_float(v[q] & 0xffff0000u));
                    v[q] = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
                }
            }
        }
        *reinterpret_cast<u32x4*>(tile + row * ROWB + chunk * 16) = v;
    }
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6;
    const int grp = lane >> 4, j = lane & 15;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        // the four 16-lane groups of a wave take four consecutive row blocks of the same 16
        // columns: their 16-byte stores fill 64 contiguous bytes of each column's line
        const int unit = 4 * wave + it;
        const int pb = 4 * (unit >> 3) + grp;
        const int cbase = 16 * (unit & 7);
        // this lane's read address: row 8*pb + j/4 (+4 for the second read), columns cbase + 4*(j%4)..+3
        uint8_t* a = tile + (8 * pb + (j >> 2)) * ROWB + (cbase + 4 * (j & 3)) * 2;
        typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)a);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(a + 4 * ROWB));
        const int64_t c = c0 + cbase + j, pcol = p0 + 8 * pb;
        if (c < cols && pcol < dst_cols) {   // dst_cols is a multiple of 8 on this path
            u32x4 o;
            o[0] = (uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
            o[1] = (uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
            o[2] = (uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
            o[3] = (uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
            *reinterpret_cast<u32x4*>(dst + c * dst_stride + pcol) = o;
        }
    }
}

// one block per (expert, 64 columns): 4 row lanes add every 4th row, then a fixed-order tree
template <typename T>
__global__ __launch_bounds__(256) void segment_colsum_kernel(const T* __restrict__ src, int64_t total_rows,
                                                             int64_t cols, int64_t stride,
                                                             const int64_t* __restrict__ offsets,
                                                             T* __restrict__ out) {
    __shared__ float part[4][64];
    const int e = blockIdx.y;
    const int64_t c = (int64_t)blockIdx.x * 64 + (threadIdx.x & 63);
    const int ty = threadIdx.x >> 6;
    int64_t lo = offsets[e], hi = offsets[e + 1];
    lo = lo < 0 ? 0 : lo;
    hi = hi > total_rows ? total_rows : hi;
    float acc = 0.0f;
    if (c < cols)
        for (int64_t r = lo + ty; r < hi; r += 4) acc += Val<T>::load(src + r * stride + c);
    part[ty][threadIdx.x & 63] = acc;
    __syncthreads();
    if (ty == 0 && c < cols) {
        const int x = threadIdx.x;
        Val<T>::store(out + (int64_t)e * cols + c, (part[0][x] + part[1][x]) + (part[2][x] + part[3][x]));
    }
}

// bf16 rows of whole 16-byte chunks: one block per (expert, 64 columns) as above, but a lane
// reads 8 columns at a time, 8 lanes cover the 128 bytes of a row segment and the 32 row lanes
// of the block (8 per wave) take every 32nd row, four rows in flight per lane.  Sums in fp32 in
// a fixed order: a lane's rows in ascending order, then the row lanes of a wave by a butterfly,
// then the four waves.
__global__ __launch_bounds__(256) void segment_colsum_bf16x8_kernel(const uint16_t* __restrict__ src,
                                                                    int64_t total_rows, int64_t cols, int64_t stride,
                                                                    const int64_t* __restrict__ offsets,
                                                                    uint16_t* __restrict__ out) {
    __shared__ float part[4][64];
    const int e = blockIdx.y;
    const int lane = lane_id(), wave = threadIdx.x / kWave;
    const int cl = lane & 7, rl = wave * 8 + (lane >> 3);
    const int64_t c = (int64_t)blockIdx.x * 64 + cl * 8;
    int64_t lo = offsets[e], hi = offsets[e + 1];
    lo = lo < 0 ? 0 : lo;
    hi = hi > total_rows ? total_rows : hi;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (c < cols) {
        const uint16_t* col = src + c;
        int64_t r = lo + rl;
        for (; r + 96 < hi; r += 128) {
            u32x4 v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = *reinterpret_cast<const u32x4*>(col + (r + 32 * i) * stride);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[2 * j] += bf16_bits_to_f32(v[i][j] & 0xffffu);
                    acc[2 * j + 1] += __uint_as_float(v[i][j] & 0xffff0000u);
                }
        }
        for (; r < hi; r += 32) {
            const u32x4 v = *reinterpret_cast<const u32x4*>(col + r * stride);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[2 * j] += bf16_bits_to_f32(v[j] & 0xffffu);
                acc[2 * j + 1] += __uint_as_float(v[j] & 0xffff0000u);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float a = acc[j];
        a += __shfl_xor(a, 8);
        a += __shfl_xor(a, 16);
        a += __shfl_xor(a, 32);
        acc[j] = a;
    }
    if (lane < 8) {
#pragma unroll
        for (int j = 0; j < 8; ++j) part[wave][lane * 8 + j] = acc[j];
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        const int64_t cc = (int64_t)blockIdx.x * 64 + threadIdx.x;
        const int x = threadIdx.x;
        if (cc < cols)
            out[(int64_t)e * cols + cc] = (uint16_t)f32_to_bf16_bits((part[0][x] + part[1][x]) + (part[2][x] + part[3][x]));
    }
}

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename T, bool GATED>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ g, const T* __restrict__ u,
                                                         const T* __restrict__ dh, T* __restrict__ dg,
                                                         T* __restrict__ du, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float gv = Val<T>::load(g + i), d = Val<T>::load(dh + i);
    const float s = sigmoid_f32(gv);
    const float dsilu = s * (1.0f + gv * (1.0f - s));
    if (GATED) {
        const float uv = Val<T>::load(u + i);
        Val<T>::store(du + i, d * Val<T>::round(gv * s));
        Val<T>::store(dg + i, Val<T>::round(d * uv) * dsilu);
    } else {
        Val<T>::store(dg + i, d * dsilu);
    }
}

// bf16, 8 elements per thread (16-byte loads and stores)
template <bool GATED>
__global__ __launch_bounds__(256) void swiglu_bwd_bf16x8_kernel(const uint16_t* __restrict__ g,
                                                                const uint16_t* __restrict__ u,
                                                                const uint16_t* __restrict__ dh,
                                                                uint16_t* __restrict__ dg,
                                                                uint16_t* __restrict__ du, int64_t n8,
                                                                int64_t cols8, int64_t out_stride8) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    // outputs with a row pitch of their own (out_stride8 chunks per row of cols8 chunks)
    int64_t o = i;
    if (out_stride8 != cols8) {
        const int64_t row = i / cols8;
        o = row * out_stride8 + (i - row * cols8);
    }
    const u32x4 vg = reinterpret_cast<const u32x4*>(g)[i];
    const u32x4 vd = reinterpret_cast<const u32x4*>(dh)[i];
    u32x4 vu = {0, 0, 0, 0}, og, ou = {0, 0, 0, 0};
    if (GATED) vu = reinterpret_cast<const u32x4*>(u)[i];
#pragma unroll
    for (int q = 0; q < 4; ++q) {       // two elements at a time: every bf16 rounding is one pack instruction
        const float g0 = bf16_bits_to_f32(vg[q] & 0xffffu), g1 = __uint_as_float(vg[q] & 0xffff0000u);
        const float d0 = bf16_bits_to_f32(vd[q] & 0xffffu), d1 = __uint_as_float(vd[q] & 0xffff0000u);
        const float s0 = sigmoid_f32(g0), s1 = sigmoid_f32(g1);
        const float ds0 = s0 * (1.0f + g0 * (1.0f - s0)), ds1 = s1 * (1.0f + g1 * (1.0f - s1));
        if (GATED) {
            const float u0 = bf16_bits_to_f32(vu[q] & 0xffffu), u1 = __uint_as_float(vu[q] & 0xffff0000u);
            float a0 = g0 * s0, a1 = g1 * s1;       // silu(g), rounded as the forward rounds it
            round_bf16_pair(a0, a1);
            ou[q] = cvt_pk_bf16(d0 * a0, d1 * a1);
            float b0 = d0 * u0, b1 = d1 * u1;
            round_bf16_pair(b0, b1);
            og[q] = cvt_pk_bf16(b0 * ds0, b1 * ds1);
        } else {
            og[q] = cvt_pk_bf16(d0 * ds0, d1 * ds1);
        }
    }
    reinterpret_cast<u32x4*>(dg)[o] = og;
    if (GATED) reinterpret_cast<u32x4*>(du)[o] = ou;
}

// dst[i, :] = src[index[i] / index_div, :] for rows of whole 16-byte chunks: one wavefront per
// output row, ordinary (cached) loads, since a top-k router names every source row k times.
__global__ __launch_bounds__(256) void gather_rows_kernel(const u32x4* __restrict__ src, int64_t src_rows,
                                                          int64_t chunks, int64_t src_stride,
                                                          const int64_t* __restrict__ index, int index_div,
                                                          int64_t n_out, u32x4* __restrict__ dst,
                                                          int64_t dst_stride) {
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
    if (row >= n_out) return;
    int64_t s = index[row] / index_div;
    s = s < 0 ? 0 : (s >= src_rows ? src_rows - 1 : s);       // malformed index: clamped, never followed
    const u32x4* from = src + s * src_stride;
    u32x4* to = dst + row * dst_stride;
    for (int64_t c = lane_id(); c < chunks; c += kWave) to[c] = from[c];
}

struct GateArgs {
    const void* ptr;
    int64_t cols, stride_row, stride_col;
    const int64_t* index;
    int64_t numel;
};

// one wavefront per routed row
template <typename T, typename TG>
__global__ __launch_bounds__(256) void combine_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ value,
                                                          int64_t T_tokens, int64_t R, int64_t D,
                                                          int64_t value_stride,
                                                          const int64_t* __restrict__ token_index,
                                                          GateArgs gate, T* __restrict__ d_value,
                                                          float* __restrict__ d_gates, bool vec8) {
    const int lane = lane_id();
    const int64_t r = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
    if (r >= R) return;
    int64_t t = token_index[r];
    const bool ok = t >= 0 && t < T_tokens;
    if (!ok) t = 0;
    const int64_t flat = gate.index ? gate.index[r] : r;
    float w = 1.0f;
    const bool flat_ok = (uint64_t)flat < (uint64_t)gate.numel;
    if (gate.ptr) {
        w = 0.0f;
        if (flat_ok) {
            const int64_t gr = flat / gate.cols, gc = flat - gr * gate.cols;
            w = Val<TG>::load((const TG*)gate.ptr + gr * gate.stride_row + gc * gate.stride_col);
        }
    }
    float dot = 0.0f;
    if (sizeof(T) == 2 && vec8) {
        const uint16_t* dyr = (const uint16_t*)dy + t * D;
        const uint16_t* vr = (const uint16_t*)value + r * value_stride;
        uint16_t* dvr = (uint16_t*)d_value + r * D;
        for (int64_t c = (int64_t)lane * 8; c < D; c += kWave * 8) {
            u32x4 vd = {0, 0, 0, 0}, vv = {0, 0, 0, 0}, o;
            if (ok) vd = *reinterpret_cast<const u32x4*>(dyr + c);
            if (d_gates) vv = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vr + c));
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float d0 = bf16_bits_to_f32(vd[q] & 0xffffu), d1 = __uint_as_float(vd[q] & 0xffff0000u);
                o[q] = cvt_pk_bf16(d0 * w, d1 * w);
                if (d_gates) {
                    float p0 = bf16_bits_to_f32(vv[q] & 0xffffu) * d0, p1 = __uint_as_float(vv[q] & 0xffff0000u) * d1;
                    round_bf16_pair(p0, p1);
                    dot += p0;
                    dot += p1;
                }
            }
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(dvr + c));
        }
    } else {
        for (int64_t c = lane; c < D; c += kWave) {
            const float d = ok ? Val<T>::load(dy + t * D + c) : 0.0f;
            Val<T>::store(d_value + r * D + c, d * w);
            if (d_gates) dot += Val<T>::round(Val<T>::load(value + r * value_stride + c) * d);
        }
    }
    if (d_gates) {
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) dot += __shfl_xor(dot, o, kWave);
        if (lane == 0 && flat_ok) d_gates[flat] = dot;
    }
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_jagged_transpose(const void* src, int dtype, int64_t src_rows, int64_t cols,
                                     int64_t src_stride_row, const int64_t* row_index, int index_div,
                                     const int64_t* offsets, const int64_t* pad_offsets, int num_experts,
                                     void* dst, int64_t dst_stride, int64_t dst_cols, int apply_silu,
                                     fmoe_stream_t stream) {
    FMOE_REQUIRE(dtype == FMOE_BF16 || dtype == FMOE_F32, "fmoe_jagged_transpose: dtype must be bf16 or fp32");
    FMOE_REQUIRE(src_rows >= 0 && cols >= 0 && dst_cols >= 0 && num_experts >= 1,
                 "fmoe_jagged_transpose: negative extent or no experts");
    FMOE_REQUIRE(index_div >= 1, "fmoe_jagged_transpose: index_div < 1");
    if (cols == 0 || dst_cols == 0) return FMOE_OK;
    FMOE_REQUIRE(src && offsets && pad_offsets && dst, "fmoe_jagged_transpose: NULL pointer");
    FMOE_REQUIRE(src_stride_row >= cols && dst_stride >= dst_cols,
                 "fmoe_jagged_transpose: a row stride is shorter than its row");
    const int64_t gx = (dst_cols + 63) / 64, gy = (cols + 63) / 64;
    FMOE_REQUIRE(gx < ((int64_t)1 << 31) && gy <= 65535, "fmoe_jagged_transpose: grid too large");
    dim3 grid((unsigned)gx, (unsigned)gy);
    const bool vec = dtype == FMOE_BF16 && cols % 8 == 0 && src_stride_row % 8 == 0 && dst_stride % 8 == 0 &&
                     dst_cols % 8 == 0 && aligned16(src) && aligned16(dst);
    if (vec) {
        const int64_t gy2 = (cols + 127) / 128;
        dim3 grid2((unsigned)gx, (unsigned)gy2);
        jagged_transpose_tr_kernel<<<grid2, 256, 0, (hipStream_t)stream>>>(
            (const uint16_t*)src, src_rows, cols, src_stride_row, row_index, index_div, offsets, pad_offsets,
            num_experts, (uint16_t*)dst, dst_stride, dst_cols, apply_silu);
    } else if (dtype == FMOE_BF16)
        jagged_transpose_kernel<uint16_t><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint16_t*)src, src_rows, cols, src_stride_row, row_index, index_div, offsets, pad_offsets,
            num_experts, (uint16_t*)dst, dst_stride, dst_cols, apply_silu);
    else
        jagged_transpose_kernel<float><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const float*)src, src_rows, cols, src_stride_row, row_index, index_div, offsets, pad_offsets,
            num_experts, (float*)dst, dst_stride, dst_cols, apply_silu);
    return check_launch("fmoe_jagged_transpose");
}

extern "C" int fmoe_gather_rows(const void* src, int64_t src_rows, int64_t row_bytes, int64_t src_stride_bytes,
                                const int64_t* index, int index_div, int64_t n_out, void* dst,
                                int64_t dst_stride_bytes, fmoe_stream_t stream) {
    FMOE_REQUIRE(src_rows >= 0 && row_bytes >= 0 && n_out >= 0 && index_div >= 1,
                 "fmoe_gather_rows: negative extent or index_div < 1");
    if (n_out == 0 || row_bytes == 0) return FMOE_OK;
    FMOE_REQUIRE(src && index && dst && src_rows >= 1, "fmoe_gather_rows: NULL pointer or no source rows");
    FMOE_REQUIRE(row_bytes % 16 == 0 && src_stride_bytes % 16 == 0 && dst_stride_bytes % 16 == 0 && aligned16(src) &&
                     aligned16(dst) && src_stride_bytes >= row_bytes && dst_stride_bytes >= row_bytes,
                 "fmoe_gather_rows: rows and row pitches are whole, 16-byte aligned chunks (row_bytes=%lld)",
                 (long long)row_bytes);
    FMOE_REQUIRE((n_out + 3) / 4 < ((int64_t)1 << 31), "fmoe_gather_rows: too many rows");
    gather_rows_kernel<<<(unsigned)((n_out + 3) / 4), 256, 0, (hipStream_t)stream>>>(
        (const u32x4*)src, src_rows, row_bytes / 16, src_stride_bytes / 16, index, index_div, n_out, (u32x4*)dst,
        dst_stride_bytes / 16);
    return check_launch("fmoe_gather_rows");
}

extern "C" int fmoe_segment_colsum(const void* src, int dtype, int64_t total_rows, int64_t cols,
                                   int64_t src_stride_row, const int64_t* offsets, int num_experts, void* out,
                                   fmoe_stream_t stream) {
    FMOE_REQUIRE(dtype == FMOE_BF16 || dtype == FMOE_F32, "fmoe_segment_colsum: dtype must be bf16 or fp32");
    FMOE_REQUIRE(total_rows >= 0 && cols >= 0 && num_experts >= 1 && num_experts <= 65535,
                 "fmoe_segment_colsum: bad extents");
    if (cols == 0) return FMOE_OK;
    FMOE_REQUIRE((src || total_rows == 0) && offsets && out, "fmoe_segment_colsum: NULL pointer");
    FMOE_REQUIRE(src_stride_row >= cols, "fmoe_segment_colsum: row stride shorter than the row");
    dim3 grid((unsigned)((cols + 63) / 64), (unsigned)num_experts);
    if (dtype == FMOE_BF16 && cols % 8 == 0 && src_stride_row % 8 == 0 && aligned16(src))
        segment_colsum_bf16x8_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint16_t*)src, total_rows, cols, src_stride_row, offsets, (uint16_t*)out);
    else if (dtype == FMOE_BF16)
        segment_colsum_kernel<uint16_t><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint16_t*)src, total_rows, cols, src_stride_row, offsets, (uint16_t*)out);
    else
        segment_colsum_kernel<float><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const float*)src, total_rows, cols, src_stride_row, offsets, (float*)out);
    return check_launch("fmoe_segment_colsum");
}

extern "C" int fmoe_swiglu_bwd(const void* g, const void* u, const void* dh, void* dg, void* du, int dtype,
                               int64_t n, int64_t cols, int64_t out_stride_row, fmoe_stream_t stream) {
    FMOE_REQUIRE(dtype == FMOE_BF16 || dtype == FMOE_F32, "fmoe_swiglu_bwd: dtype must be bf16 or fp32");
    FMOE_REQUIRE(n >= 0, "fmoe_swiglu_bwd: n < 0");
    if (n == 0) return FMOE_OK;
    FMOE_REQUIRE(g && dh && dg && (!u || du), "fmoe_swiglu_bwd: NULL pointer");
    const bool pitched = out_stride_row != 0 && out_stride_row != cols;
    if (pitched)
        FMOE_REQUIRE(dtype == FMOE_BF16 && cols >= 8 && cols % 8 == 0 && n % cols == 0 && out_stride_row > cols &&
                         out_stride_row % 8 == 0 && aligned16(g) && aligned16(dh) && aligned16(dg) &&
                         (!u || (aligned16(u) && aligned16(du))),
                     "fmoe_swiglu_bwd: outputs with a row pitch need bf16, cols and pitch in multiples of 8, "
                     "16-byte alignment (cols=%lld pitch=%lld)", (long long)cols, (long long)out_stride_row);
    const int64_t cols8 = pitched ? cols / 8 : 1, stride8 = pitched ? out_stride_row / 8 : 1;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    FMOE_REQUIRE((n + 255) / 256 < ((int64_t)1 << 31), "fmoe_swiglu_bwd: too many elements");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FMOE_BF16 && n % 8 == 0 && aligned16(g) && aligned16(dh) && aligned16(dg) &&
        (!u || (aligned16(u) && aligned16(du)))) {
        const int64_t n8 = n / 8;
        const unsigned b8 = (unsigned)((n8 + 255) / 256);
        if (u) swiglu_bwd_bf16x8_kernel<true><<<b8, 256, 0, s>>>((const uint16_t*)g, (const uint16_t*)u, (const uint16_t*)dh, (uint16_t*)dg, (uint16_t*)du, n8, cols8, stride8);
        else swiglu_bwd_bf16x8_kernel<false><<<b8, 256, 0, s>>>((const uint16_t*)g, nullptr, (const uint16_t*)dh, (uint16_t*)dg, nullptr, n8, cols8, stride8);
    } else if (dtype == FMOE_BF16) {
        if (u) swiglu_bwd_kernel<uint16_t, true><<<blocks, 256, 0, s>>>((const uint16_t*)g, (const uint16_t*)u, (const uint16_t*)dh, (uint16_t*)dg, (uint16_t*)du, n);
        else swiglu_bwd_kernel<uint16_t, false><<<blocks, 256, 0, s>>>((const uint16_t*)g, nullptr, (const uint16_t*)dh, (uint16_t*)dg, nullptr, n);
    } else {
        if (u) swiglu_bwd_kernel<float, true><<<blocks, 256, 0, s>>>((const float*)g, (const float*)u, (const float*)dh, (float*)dg, (float*)du, n);
        else swiglu_bwd_kernel<float, false><<<blocks, 256, 0, s>>>((const float*)g, nullptr, (const float*)dh, (float*)dg, nullptr, n);
    }
    return check_launch("fmoe_swiglu_bwd");
}

extern "C" int fmoe_combine_bwd(const void* dy, const void* value, int value_dtype, int64_t T, int K, int64_t D,
                                int64_t value_stride_row, const int64_t* token_index, const void* gates,
                                int gates_dtype, int64_t gates_cols, int64_t gates_stride_row,
                                int64_t gates_stride_col, const int64_t* gates_index, void* d_value,
                                float* d_gates, fmoe_stream_t stream) {
    FMOE_REQUIRE(value_dtype == FMOE_BF16 || value_dtype == FMOE_F32, "fmoe_combine_bwd: value must be bf16 or fp32");
    FMOE_REQUIRE(T >= 0 && K >= 1 && D >= 1, "fmoe_combine_bwd: need T >= 0, K >= 1, D >= 1");
    if (T == 0) return FMOE_OK;
    FMOE_REQUIRE(dy && token_index && d_value, "fmoe_combine_bwd: NULL pointer");
    FMOE_REQUIRE(!d_gates || (value && value_stride_row >= D), "fmoe_combine_bwd: d_gates needs value rows");
    if (gates) {
        FMOE_REQUIRE(gates_dtype == FMOE_BF16 || gates_dtype == FMOE_F32, "fmoe_combine_bwd: gates must be bf16 or fp32");
        FMOE_REQUIRE(gates_cols >= 1, "fmoe_combine_bwd: gates_cols < 1");
    }
    const int64_t R = T * (int64_t)K;
    FMOE_REQUIRE((R + 3) / 4 < ((int64_t)1 << 31), "fmoe_combine_bwd: too many rows");
    GateArgs ga{gates, gates_cols, gates_stride_row, gates_stride_col, gates_index, R};
    const unsigned blocks = (unsigned)((R + 3) / 4);
    hipStream_t s = (hipStream_t)stream;
    const bool gb = gates && gates_dtype == FMOE_BF16;
    const bool vec8 = D % 8 == 0 && aligned16(dy) && aligned16(d_value) &&
                      (!d_gates || (value_stride_row % 8 == 0 && aligned16(value)));
    if (value_dtype == FMOE_BF16) {
        if (gb) combine_bwd_kernel<uint16_t, uint16_t><<<blocks, 256, 0, s>>>((const uint16_t*)dy, (const uint16_t*)value, T, R, D, value_stride_row, token_index, ga, (uint16_t*)d_value, d_gates, vec8);
        else combine_bwd_kernel<uint16_t, float><<<blocks, 256, 0, s>>>((const uint16_t*)dy, (const uint16_t*)value, T, R, D, value_stride_row, token_index, ga, (uint16_t*)d_value, d_gates, vec8);
    } else {
        if (gb) combine_bwd_kernel<float, uint16_t><<<blocks, 256, 0, s>>>((const float*)dy, (const float*)value, T, R, D, value_stride_row, token_index, ga, (float*)d_value, d_gates, false);
        else combine_bwd_kernel<float, float><<<blocks, 256, 0, s>>>((const float*)dy, (const float*)value, T, R, D, value_stride_row, token_index, ga, (float*)d_value, d_gates, false);
    }
    return check_launch("fmoe_combine_bwd");
}
