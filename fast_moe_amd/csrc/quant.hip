// Row-wise OCP e4m3fn quantisation with power-of-two multiplier scales.
//
// Fast path (contiguous bf16 rows, cols % 8 == 0): one wavefront per row, the
// row is read once with 16-byte loads and held in registers, so the traffic is
// the algorithmic 2 B in + 1 B out per element (+4 B scale per row).
// Rows too long for that (more than 8192 columns) get one block each and two
// passes.  Generic paths cover any strides, column counts and fp32 inputs.
#include "common.h"

namespace fmoe {
namespace {

// Software e4m3fn encoder: round to nearest even, non-saturating (anything that
// rounds above 448, and inf / NaN, becomes S.1111.111).
__device__ __forceinline__ uint32_t e4m3fn_encode(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7fffffffu;
    uint32_t code;
    if (a >= 0x43f00000u) {                 // >= 480, inf, NaN
        code = 0x7fu;
    } else if (a < 0x3c800000u) {           // below 2^-6: subnormal grid of 2^-9
        code = (uint32_t)rintf(__uint_as_float(a) * 512.0f);
    } else {
        a += 0x7ffffu + ((a >> 20) & 1u);
        code = (a >> 20) - (120u << 3);
    }
    return sign | code;
}

// scale = 2^floor(log2(448 / amax)); NaN / inf results -> 2^127; amax = inf -> 0.
// EXACT_EXPONENT: take the exponent field of the fp32 quotient.  For an amax
// that is a bf16 value this equals the reference's bf16 formula for every input.
// Otherwise follow the fp32 formula literally: the fp32 log2 of a quotient just
// below a power of two rounds up to the integer.
template <bool EXACT_EXPONENT>
__device__ __forceinline__ float scale_from_amax(float amax) {
    const float q = 448.0f / amax;
    const float clamp = __uint_as_float(0x7f000000u);  // 2^127
    if (!(q <= 3.4028234664e38f)) return clamp;         // inf or NaN
    if (q == 0.0f) return 0.0f;
    if (EXACT_EXPONENT) return __uint_as_float(__float_as_uint(q) & 0x7f800000u);
    const float fl = floorf((float)log2((double)q));
    if (fl >= 128.0f) return clamp;
    return __uint_as_float((uint32_t)((int)fl + 127) << 23);
}

__device__ __forceinline__ float amax_update(float m, float v, bool& nan) {
    nan |= (v != v);
    return fmaxf(m, fabsf(v));
}

__device__ __forceinline__ float finish_amax(float m, bool nan) {
    m = wave_max(m);
    if (__ballot(nan) != 0ull) m = __uint_as_float(0x7fc00000u);
    return m;
}

// eight bf16 values times the row's scale -> eight e4m3 codes.  Rows without NaN / inf take the
// hardware conversion; a row that holds one goes through the software encoder, which keeps the
// reference's non-saturating codes.
__device__ __forceinline__ u32x2 encode8(const u32x4& v, float s, bool special) {
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[2 * j] = bf16_bits_to_f32(v[j] & 0xffffu) * s;
        f[2 * j + 1] = __uint_as_float(v[j] & 0xffff0000u) * s;
    }
    u32x2 o;
    if (!special) {
        int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
        int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
        o[0] = (uint32_t)w0;
        o[1] = (uint32_t)w1;
    } else {
        o[0] = e4m3fn_encode(f[0]) | (e4m3fn_encode(f[1]) << 8) | (e4m3fn_encode(f[2]) << 16) |
               (e4m3fn_encode(f[3]) << 24);
        o[1] = e4m3fn_encode(f[4]) | (e4m3fn_encode(f[5]) << 8) | (e4m3fn_encode(f[6]) << 16) |
               (e4m3fn_encode(f[7]) << 24);
    }
    return o;
}

// ---- fast path: bf16, contiguous columns, cols % 8 == 0, <= CH*512 columns
// W16: a lane takes pairs of neighbouring 16-byte chunks (32 contiguous input bytes), so that its
// eight-byte results pair up into one 16-byte store (rows of a whole number of such pairs)
template <int CH, bool SILU, bool W16 = false>
__global__ __launch_bounds__(256) void quant_rows_bf16_wave(
    const uint16_t* __restrict__ a, int64_t total_rows, int64_t rows, int cols, int64_t a_sb,
    int64_t a_sr, uint8_t* __restrict__ q, int64_t q_sb, int64_t q_sr, float* __restrict__ scale,
    int store_reciprocal) {
    const int lane = lane_id();
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
    if (row >= total_rows) return;
    const int64_t b = row / rows, r = row - b * rows;
    const uint16_t* src = a + b * a_sb + r * a_sr;
    uint8_t* dst = q + b * q_sb + r * q_sr;
    const int chunks = cols >> 3;

    static_assert(!W16 || CH % 2 == 0, "pairs of chunks");
    // chunk held in v[i]
    auto chunk_of = [&](int i) { return W16 ? 2 * (lane + kWave * (i / 2)) + (i & 1) : lane + kWave * i; };
    u32x4 v[CH];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = chunk_of(i);
        v[i] = c < chunks ? *reinterpret_cast<const u32x4*>(src + (int64_t)c * 8) : u32x4{0, 0, 0, 0};
    }
    float m = 0.0f;
    bool nan = false;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float lo = bf16_bits_to_f32(v[i][j] & 0xffffu);
            float hi = __uint_as_float(v[i][j] & 0xffff0000u);
            if (SILU) {
                lo = silu_round_bf16(lo);
                hi = silu_round_bf16(hi);
                v[i][j] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
            }
            m = amax_update(m, lo, nan);
            m = amax_update(m, hi, nan);
        }
    }
    m = finish_amax(m, nan);
    const float s = scale_from_amax<true>(m);   // every element is a bf16 value
    if (lane == 0) scale[row] = store_reciprocal ? 1.0f / s : s;
    const bool special = !(m <= 3.4028234664e38f);   // NaN or inf in the row
    if constexpr (W16) {
#pragma unroll
        for (int i = 0; i < CH; i += 2) {
            const int c = chunk_of(i);
            if (c >= chunks) continue;
            const u32x2 lo = encode8(v[i], s, special), hi = encode8(v[i + 1], s, special);
            *reinterpret_cast<u32x4*>(dst + (int64_t)c * 8) = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    } else {
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            const int c = lane + kWave * i;
            if (c >= chunks) continue;
            const u32x2 o = encode8(v[i], s, special);
            *reinterpret_cast<u32x2*>(dst + (int64_t)c * 8) = o;
        }
    }
}

// ---- long rows (more columns than a wave holds in registers): one block per row, two passes
// with 16-byte loads; the second pass finds most of the row in L2.  The transposed operands of
// the fp8 weight gradient are a few thousand rows of 10^5 columns.
template <bool SILU>
__global__ __launch_bounds__(256) void quant_rows_bf16_block(
    const uint16_t* __restrict__ a, int64_t rows, int64_t cols, int64_t a_sb, int64_t a_sr,
    uint8_t* __restrict__ q, int64_t q_sb, int64_t q_sr, float* __restrict__ scale, int store_reciprocal) {
    __shared__ float s_max[4];
    __shared__ int s_nan[4];
    const int64_t row = blockIdx.x;
    const int64_t b = row / rows, r = row - b * rows;
    const uint16_t* src = a + b * a_sb + r * a_sr;
    uint8_t* dst = q + b * q_sb + r * q_sr;
    const int64_t chunks = cols >> 3;
    auto load = [&](int64_t c) {
        u32x4 v = *reinterpret_cast<const u32x4*>(src + c * 8);
        if (SILU) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float lo = silu_round_bf16(bf16_bits_to_f32(v[j] & 0xffffu));
                const float hi = silu_round_bf16(__uint_as_float(v[j] & 0xffff0000u));
                v[j] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
            }
        }
        return v;
    };
    float m = 0.0f;
    bool nan = false;
    for (int64_t c = threadIdx.x; c < chunks; c += 256) {
        const u32x4 v = load(c);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            m = amax_update(m, bf16_bits_to_f32(v[j] & 0xffffu), nan);
            m = amax_update(m, __uint_as_float(v[j] & 0xffff0000u), nan);
        }
    }
    m = wave_max(m);
    const bool any_nan = __ballot(nan) != 0ull;
    if (lane_id() == 0) {
        s_max[threadIdx.x / kWave] = m;
        s_nan[threadIdx.x / kWave] = any_nan;
    }
    __syncthreads();
    m = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    if (s_nan[0] | s_nan[1] | s_nan[2] | s_nan[3]) m = __uint_as_float(0x7fc00000u);
    const float s = scale_from_amax<true>(m);
    if (threadIdx.x == 0) scale[row] = store_reciprocal ? 1.0f / s : s;
    const bool special = !(m <= 3.4028234664e38f);
    for (int64_t c = threadIdx.x; c < chunks; c += 256)
        *reinterpret_cast<u32x2*>(dst + c * 8) = encode8(load(c), s, special);
}

template <typename T>
__device__ __forceinline__ float load_as_f32(const T* p);
template <>
__device__ __forceinline__ float load_as_f32<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_as_f32<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }

template <typename T, bool SILU>
__device__ __forceinline__ float fetch(const T* p) {
    float v = load_as_f32<T>(p);
    if (SILU) v = sizeof(T) == 2 ? silu_round_bf16(v) : silu_f32(v);
    return v;
}

// ---- generic: one wave per row, lanes stride over the columns, two passes
template <typename T, bool SILU>
__global__ __launch_bounds__(256) void quant_rows_generic_wave(
    const T* __restrict__ a, int64_t total_rows, int64_t rows, int64_t cols, int64_t a_sb, int64_t a_sr,
    int64_t a_sc, uint8_t* __restrict__ q, int64_t q_sb, int64_t q_sr, int64_t q_sc,
    float* __restrict__ scale, int store_reciprocal) {
    const int lane = lane_id();
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
    if (row >= total_rows) return;
    const int64_t b = row / rows, r = row - b * rows;
    const T* src = a + b * a_sb + r * a_sr;
    uint8_t* dst = q + b * q_sb + r * q_sr;
    float m = 0.0f;
    bool nan = false;
    for (int64_t c = lane; c < cols; c += kWave) m = amax_update(m, fetch<T, SILU>(src + c * a_sc), nan);
    m = finish_amax(m, nan);
    const float s = sizeof(T) == 2 ? scale_from_amax<true>(m) : scale_from_amax<false>(m);
    if (lane == 0) scale[row] = store_reciprocal ? 1.0f / s : s;
    for (int64_t c = lane; c < cols; c += kWave)
        dst[c * q_sc] = (uint8_t)e4m3fn_encode(fetch<T, SILU>(src + c * a_sc) * s);
}

// ---- generic, rows adjacent in memory (a_sr == 1): one lane per row so that
// the loads of a wave are contiguous
template <typename T, bool SILU>
__global__ __launch_bounds__(256) void quant_rows_generic_lane(
    const T* __restrict__ a, int64_t total_rows, int64_t rows, int64_t cols, int64_t a_sb, int64_t a_sr,
    int64_t a_sc, uint8_t* __restrict__ q, int64_t q_sb, int64_t q_sr, int64_t q_sc,
    float* __restrict__ scale, int store_reciprocal) {
    const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= total_rows) return;
    const int64_t b = row / rows, r = row - b * rows;
    const T* src = a + b * a_sb + r * a_sr;
    uint8_t* dst = q + b * q_sb + r * q_sr;
    float m = 0.0f;
    bool nan = false;
    for (int64_t c = 0; c < cols; ++c) m = amax_update(m, fetch<T, SILU>(src + c * a_sc), nan);
    if (nan) m = __uint_as_float(0x7fc00000u);
    const float s = sizeof(T) == 2 ? scale_from_amax<true>(m) : scale_from_amax<false>(m);
    scale[row] = store_reciprocal ? 1.0f / s : s;
    for (int64_t c = 0; c < cols; ++c)
        dst[c * q_sc] = (uint8_t)e4m3fn_encode(fetch<T, SILU>(src + c * a_sc) * s);
}

// rows that are whole pairs of chunks, stored 16 bytes at a time
inline bool wide_stores(int64_t cols, const uint8_t* q, int64_t q_sb, int64_t q_sr) {
    return cols % 16 == 0 && (reinterpret_cast<uintptr_t>(q) & 15u) == 0 && q_sb % 16 == 0 && q_sr % 16 == 0;
}

template <int CH>
void launch_fast(bool silu, const uint16_t* a, int64_t total, int64_t rows, int cols, int64_t a_sb,
                 int64_t a_sr, uint8_t* q, int64_t q_sb, int64_t q_sr, float* scale, int recip,
                 hipStream_t stream) {
    const unsigned blocks = (unsigned)((total + 3) / 4);
    if constexpr (CH % 2 == 0) {
        if (wide_stores(cols, q, q_sb, q_sr)) {
            if (silu)
                quant_rows_bf16_wave<CH, true, true><<<blocks, 256, 0, stream>>>(a, total, rows, cols, a_sb, a_sr, q,
                                                                                 q_sb, q_sr, scale, recip);
            else
                quant_rows_bf16_wave<CH, false, true><<<blocks, 256, 0, stream>>>(a, total, rows, cols, a_sb, a_sr, q,
                                                                                  q_sb, q_sr, scale, recip);
            return;
        }
    }
    if (silu)
        quant_rows_bf16_wave<CH, true><<<blocks, 256, 0, stream>>>(a, total, rows, cols, a_sb, a_sr, q,
                                                                   q_sb, q_sr, scale, recip);
    else
        quant_rows_bf16_wave<CH, false><<<blocks, 256, 0, stream>>>(a, total, rows, cols, a_sb, a_sr, q,
                                                                    q_sb, q_sr, scale, recip);
}

template <typename T>
void launch_generic(bool silu, bool lane_per_row, const void* a_, int64_t total, int64_t rows,
                    int64_t cols, int64_t a_sb, int64_t a_sr, int64_t a_sc, uint8_t* q, int64_t q_sb,
                    int64_t q_sr, int64_t q_sc, float* scale, int recip, hipStream_t stream) {
    const T* a = (const T*)a_;
#define FMOE_ARGS a, total, rows, cols, a_sb, a_sr, a_sc, q, q_sb, q_sr, q_sc, scale, recip
    if (lane_per_row) {
        const unsigned blocks = (unsigned)((total + 255) / 256);
        if (silu) quant_rows_generic_lane<T, true><<<blocks, 256, 0, stream>>>(FMOE_ARGS);
        else quant_rows_generic_lane<T, false><<<blocks, 256, 0, stream>>>(FMOE_ARGS);
    } else {
        const unsigned blocks = (unsigned)((total + 3) / 4);
        if (silu) quant_rows_generic_wave<T, true><<<blocks, 256, 0, stream>>>(FMOE_ARGS);
        else quant_rows_generic_wave<T, false><<<blocks, 256, 0, stream>>>(FMOE_ARGS);
    }
#undef FMOE_ARGS
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_quant_rows_e4m3(const void* a, int a_dtype, int64_t batch, int64_t rows, int64_t cols,
                                    int64_t a_sb, int64_t a_sr, int64_t a_sc, int apply_silu, uint8_t* q,
                                    int64_t q_sb, int64_t q_sr, int64_t q_sc, float* scale,
                                    int store_reciprocal, fmoe_stream_t stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    FMOE_REQUIRE(a_dtype == FMOE_BF16 || a_dtype == FMOE_F32,
                 "fmoe_quant_rows_e4m3: input must be bf16 or fp32");
    FMOE_REQUIRE(batch >= 0 && rows >= 0 && cols >= 1,
                 "fmoe_quant_rows_e4m3: need batch, rows >= 0 and cols >= 1 (got %lld, %lld, %lld)",
                 (long long)batch, (long long)rows, (long long)cols);
    const int64_t total = batch * rows;
    if (total == 0) return FMOE_OK;
    FMOE_REQUIRE(total < ((int64_t)1 << 31) * 4, "fmoe_quant_rows_e4m3: too many rows");
    FMOE_REQUIRE(a && q && scale, "fmoe_quant_rows_e4m3: NULL pointer");

    const bool fast = a_dtype == FMOE_BF16 && a_sc == 1 && q_sc == 1 && (cols % 8) == 0 &&
                      cols <= 16 * 512 && aligned16(a) && (a_sb % 8) == 0 && (a_sr % 8) == 0 &&
                      (reinterpret_cast<uintptr_t>(q) & 7u) == 0 && (q_sb % 8) == 0 && (q_sr % 8) == 0;
    if (fast) {
        int ch = (int)((cols / 8 + kWave - 1) / kWave);
        if (wide_stores(cols, q, q_sb, q_sr)) ch = 2 * (int)((cols / 16 + kWave - 1) / kWave);
#define FMOE_FAST(CH)                                                                              \
    launch_fast<CH>(apply_silu != 0, (const uint16_t*)a, total, rows, (int)cols, a_sb, a_sr, q, q_sb, \
                    q_sr, scale, store_reciprocal, stream)
        if (ch <= 1) FMOE_FAST(1);
        else if (ch <= 2) FMOE_FAST(2);
        else if (ch <= 3) FMOE_FAST(3);
        else if (ch <= 4) FMOE_FAST(4);
        else if (ch <= 6) FMOE_FAST(6);
        else if (ch <= 8) FMOE_FAST(8);
        else if (ch <= 12) FMOE_FAST(12);
        else FMOE_FAST(16);
#undef FMOE_FAST
        return check_launch("fmoe_quant_rows_e4m3");
    }
    const bool long_rows = a_dtype == FMOE_BF16 && a_sc == 1 && q_sc == 1 && (cols % 8) == 0 && aligned16(a) &&
                           (a_sb % 8) == 0 && (a_sr % 8) == 0 && (reinterpret_cast<uintptr_t>(q) & 7u) == 0 &&
                           (q_sb % 8) == 0 && (q_sr % 8) == 0 && total < ((int64_t)1 << 31);
    if (long_rows) {
        if (apply_silu)
            quant_rows_bf16_block<true><<<(unsigned)total, 256, 0, stream>>>((const uint16_t*)a, rows, cols, a_sb, a_sr,
                                                                             q, q_sb, q_sr, scale, store_reciprocal);
        else
            quant_rows_bf16_block<false><<<(unsigned)total, 256, 0, stream>>>((const uint16_t*)a, rows, cols, a_sb, a_sr,
                                                                              q, q_sb, q_sr, scale, store_reciprocal);
        return check_launch("fmoe_quant_rows_e4m3");
    }
    const bool lane_per_row = a_sc != 1 && a_sr == 1 && rows >= 16;
    if (a_dtype == FMOE_BF16)
        launch_generic<uint16_t>(apply_silu != 0, lane_per_row, a, total, rows, cols, a_sb, a_sr, a_sc, q,
                                 q_sb, q_sr, q_sc, scale, store_reciprocal, stream);
    else
        launch_generic<float>(apply_silu != 0, lane_per_row, a, total, rows, cols, a_sb, a_sr, a_sc, q,
                              q_sb, q_sr, q_sc, scale, store_reciprocal, stream);
    return check_launch("fmoe_quant_rows_e4m3");
}
