// Shared host/device helpers for the gfx950 kernels of libfastmoe_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/fast_moe_amd.h"

namespace fmoe {

// ---------------------------------------------------------------- host side
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

#define FMOE_REQUIRE(cond, ...)                                   \
    do {                                                          \
        if (!(cond)) return ::fmoe::fail(FMOE_ERR_ARGUMENT, __VA_ARGS__); \
    } while (0)

__host__ __device__ static inline bool aligned16(const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}
__host__ __device__ static inline bool aligned_ok(const void* a, const void* b, const void* c) {
    return aligned16(a) && aligned16(b) && aligned16(c);
}

// -------------------------------------------------------------- device side
constexpr int kWave = 64;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) int i32x8;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even fp32 -> bf16 bit pattern; NaN stays NaN (quiet)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// two fp32 -> two bf16 (round to nearest even) in one v_cvt_pk_bf16_f32, `lo` in the low half: for
// loops that round every element they touch (with the integer sequence above, which also keeps a
// NaN's payload, the rounding is most of such a loop's instructions and the loop is bound by them,
// not by the memory it streams)
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    const bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
    return __builtin_bit_cast(uint32_t, r);
}
// both values rounded to bf16 and back
__device__ __forceinline__ void round_bf16_pair(float& a, float& b) {
    const uint32_t pk = cvt_pk_bf16(a, b);
    a = __uint_as_float(pk << 16);
    b = __uint_as_float(pk & 0xffff0000u);
}

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

// round(silu(x)) to bf16 for a bf16-valued x, equal on every one of the 65536 inputs to what
// x / (1 + exp(-x)) gives when it is evaluated in fp32 with correctly rounded steps and then rounded
// to bf16 (F.silu on a bf16 tensor).  The fp32 evaluation here may be a few units in the last
// place off, which only matters when the result lies next to the midpoint of two bf16 values: those
// (about one input in 4000) are evaluated again in double.  exp(-x) overflows fp32 from x = -88.8
// down and the quotient is -0 there, as in the fp32 formula; such results never take the second path.
__device__ __forceinline__ float silu_round_bf16(float x) {
    float y = x / (1.0f + expf(-x));
    const uint32_t low = __float_as_uint(y) & 0xffffu;
    if (low - 0x7ff0u <= 0x20u) {
        const double xd = (double)x;
        y = (float)(xd / (1.0 + exp(-xd)));
    }
    return round_bf16(y);
}

// SiLU from the hardware exp / reciprocal (about 2 ulp in fp32): for values that
// are rounded to bf16 right afterwards.
__device__ __forceinline__ float fast_silu_f32(float x) {
    // v_exp_f32 and v_rcp_f32 only: a true division costs ten more VALU instructions
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896341f));
}

__device__ __forceinline__ int lane_id() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

template <typename T>
__device__ __forceinline__ T wave_bcast(T v, int src_lane) {
    return __shfl(v, src_lane, kWave);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// inclusive prefix sum over the 64 lanes
__device__ __forceinline__ int wave_inclusive_scan(int v) {
    const int lane = lane_id();
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        int n = __shfl_up(v, o, kWave);
        if (lane >= o) v += n;
    }
    return v;
}
__device__ __forceinline__ long long wave_inclusive_scan(long long v) {
    const int lane = lane_id();
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        long long n = __shfl_up(v, o, kWave);
        if (lane >= o) v += n;
    }
    return v;
}

}  // namespace fmoe
