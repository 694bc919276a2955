// Error reporting, version, and the small element-wise kernel of libfastmoe_hip.so.
#include "common.h"

#include <cstring>

namespace fmoe {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(FMOE_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
    return FMOE_OK;
}

namespace {

// out = round(round(silu(a)) * b), 8 bf16 per thread; without b: out = round(silu(a))
template <bool GATED>
__global__ __launch_bounds__(256) void silu_mul_bf16_kernel(const uint16_t* __restrict__ a,
                                                            const uint16_t* __restrict__ b,
                                                            uint16_t* __restrict__ out, int64_t n) {
    const int64_t i0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i0 + 8 <= n && aligned_ok(a, GATED ? b : a, out)) {
        const u32x4 va = *reinterpret_cast<const u32x4*>(a + i0);
        const u32x4 vb = GATED ? *reinterpret_cast<const u32x4*>(b + i0) : u32x4{0, 0, 0, 0};
        u32x4 vo;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t r = 0;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float x = bf16_bits_to_f32((va[j] >> (16 * h)) & 0xffffu);
                const float y = bf16_bits_to_f32((vb[j] >> (16 * h)) & 0xffffu);
                r |= f32_to_bf16_bits(GATED ? silu_round_bf16(x) * y : silu_round_bf16(x)) << (16 * h);
            }
            vo[j] = r;
        }
        *reinterpret_cast<u32x4*>(out + i0) = vo;
    } else {
        for (int64_t i = i0; i < n && i < i0 + 8; ++i) {
            const float x = bf16_bits_to_f32(a[i]);
            const float y = GATED ? bf16_bits_to_f32(b[i]) : 1.0f;
            out[i] = (uint16_t)f32_to_bf16_bits(GATED ? silu_round_bf16(x) * y : silu_round_bf16(x));
        }
    }
}

template <bool GATED>
__global__ __launch_bounds__(256) void silu_mul_f32_kernel(const float* __restrict__ a,
                                                           const float* __restrict__ b,
                                                           float* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = GATED ? silu_f32(a[i]) * b[i] : silu_f32(a[i]);
}

// 64 x 64 tile transpose through LDS; reads and writes are both row-contiguous
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ src, T* __restrict__ dst,
                                                        int64_t rows, int64_t cols, int64_t sb, int64_t sr) {
    __shared__ T tile[64][64 + 2];
    const int64_t b = blockIdx.z;
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const T* s = src + b * sb;
    T* d = dst + b * rows * cols;
    for (int i = ty; i < 64; i += 4) {
        const int64_t r = r0 + i, c = c0 + tx;
        if (r < rows && c < cols) tile[i][tx] = s[r * sr + c];
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int64_t c = c0 + i, r = r0 + tx;
        if (r < rows && c < cols) d[c * rows + r] = tile[tx][i];
    }
}

// HBM probe: what this part reads and writes per second when nothing else limits a kernel.
// One-shot grid: block b owns piece b of 256 * PER * 16 bytes, lane l the 16-byte words
// l, l + 256, ... of it (every access instruction of a wave covers 1 KB of contiguous memory).
// READ: non-temporal loads folded into a value that is stored only if it takes a value no
// buffer produces in practice (the loads cannot be dropped).  WRITE: 16-byte stores of a
// pattern.  COPY: first half of the buffer to the second.  PER = accesses per lane: reads want
// several in flight, writes are fastest with one store per lane and many short waves.
template <int MODE, int PER>
__global__ __launch_bounds__(256) void hbm_probe_kernel(u32x4* __restrict__ buf, int64_t n16, int64_t half16,
                                                        uint32_t* sink) {
    const int64_t i0 = (int64_t)blockIdx.x * 256 * PER + threadIdx.x;
    u32x4 v[PER];
    if (MODE != 1) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int64_t idx = i0 + (int64_t)i * 256;
            v[i] = idx < n16 ? __builtin_nontemporal_load(buf + idx) : u32x4{0, 0, 0, 0};
        }
    }
    if (MODE == 0) {
        u32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < PER; ++i) acc ^= v[i];
        if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && sink) *sink = acc[0];
    } else {
        const uint32_t x = (uint32_t)blockIdx.x * 2654435761u + threadIdx.x;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int64_t idx = i0 + (int64_t)i * 256;
            if (idx < n16) buf[(MODE == 2 ? half16 : 0) + idx] = MODE == 2 ? v[i] : u32x4{x, x ^ 0x5bd1e995u, x + i, ~x};
        }
    }
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_hbm_probe(void* buf, int64_t bytes, int mode, int per_lane, fmoe_stream_t stream) {
    FMOE_REQUIRE(buf && aligned16(buf), "fmoe_hbm_probe: buf must be a 16-byte aligned device pointer");
    FMOE_REQUIRE(mode >= 0 && mode <= 2, "fmoe_hbm_probe: mode must be 0 (read), 1 (write) or 2 (copy)");
    FMOE_REQUIRE(per_lane == 1 || per_lane == 2 || per_lane == 4 || per_lane == 8,
                 "fmoe_hbm_probe: 1, 2, 4 or 8 accesses per lane");
    FMOE_REQUIRE(bytes >= 32 && bytes % 32 == 0, "fmoe_hbm_probe: bytes must be a multiple of 32");
    const int64_t n16 = (mode == 2 ? bytes / 2 : bytes) / 16;
    const int64_t grid = (n16 + 256 * (int64_t)per_lane - 1) / (256 * (int64_t)per_lane);
    FMOE_REQUIRE(grid < ((int64_t)1 << 31), "fmoe_hbm_probe: buffer too large");
    u32x4* b = (u32x4*)buf;
    hipStream_t s = (hipStream_t)stream;
#define FMOE_PROBE(M, P)                                                                      \
    if (mode == M && per_lane == P) hbm_probe_kernel<M, P><<<(unsigned)grid, 256, 0, s>>>(b, n16, n16, (uint32_t*)buf)
    FMOE_PROBE(0, 1); FMOE_PROBE(0, 2); FMOE_PROBE(0, 4); FMOE_PROBE(0, 8);
    FMOE_PROBE(1, 1); FMOE_PROBE(1, 2); FMOE_PROBE(1, 4); FMOE_PROBE(1, 8);
    FMOE_PROBE(2, 1); FMOE_PROBE(2, 2); FMOE_PROBE(2, 4); FMOE_PROBE(2, 8);
#undef FMOE_PROBE
    return check_launch("fmoe_hbm_probe");
}

extern "C" int fmoe_transpose_last2(const void* src, void* dst, int elem_size, int64_t batch, int64_t rows,
                                    int64_t cols, int64_t src_stride_b, int64_t src_stride_r,
                                    fmoe_stream_t stream) {
    FMOE_REQUIRE(elem_size == 1 || elem_size == 2, "fmoe_transpose_last2: element size must be 1 or 2");
    FMOE_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, "fmoe_transpose_last2: negative extent");
    if (batch == 0 || rows == 0 || cols == 0) return FMOE_OK;
    FMOE_REQUIRE(src && dst, "fmoe_transpose_last2: NULL pointer");
    FMOE_REQUIRE(src_stride_r >= cols, "fmoe_transpose_last2: source row stride %lld < cols %lld",
                 (long long)src_stride_r, (long long)cols);
    FMOE_REQUIRE(batch <= 65535 && (rows + 63) / 64 <= 65535, "fmoe_transpose_last2: grid too large");
    dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64), (unsigned)batch);
    if (elem_size == 2)
        transpose_kernel<uint16_t><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint16_t*)src, (uint16_t*)dst, rows, cols, src_stride_b, src_stride_r);
    else
        transpose_kernel<uint8_t><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint8_t*)src, (uint8_t*)dst, rows, cols, src_stride_b, src_stride_r);
    return check_launch("fmoe_transpose_last2");
}


extern "C" int fmoe_version(void) { return 100; }

extern "C" const char* fmoe_last_error(void) { return g_error; }

extern "C" int fmoe_silu_mul(const void* a, const void* b, void* out, int dtype, int64_t n,
                             fmoe_stream_t stream) {
    FMOE_REQUIRE(dtype == FMOE_BF16 || dtype == FMOE_F32, "fmoe_silu_mul: dtype must be bf16 or fp32");
    FMOE_REQUIRE(n >= 0, "fmoe_silu_mul: n < 0");
    if (n == 0) return FMOE_OK;
    FMOE_REQUIRE(a && out, "fmoe_silu_mul: NULL pointer");
    FMOE_REQUIRE((n + 255) / 256 < ((int64_t)1 << 31), "fmoe_silu_mul: too many elements");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FMOE_F32) {
        const unsigned blocks = (unsigned)((n + 255) / 256);
        if (b) silu_mul_f32_kernel<true><<<blocks, 256, 0, s>>>((const float*)a, (const float*)b, (float*)out, n);
        else silu_mul_f32_kernel<false><<<blocks, 256, 0, s>>>((const float*)a, nullptr, (float*)out, n);
        return check_launch("fmoe_silu_mul");
    }
    const unsigned blocks = (unsigned)(((n + 7) / 8 + 255) / 256);
    if (b) silu_mul_bf16_kernel<true><<<blocks, 256, 0, s>>>((const uint16_t*)a, (const uint16_t*)b, (uint16_t*)out, n);
    else silu_mul_bf16_kernel<false><<<blocks, 256, 0, s>>>((const uint16_t*)a, nullptr, (uint16_t*)out, n);
    return check_launch("fmoe_silu_mul");
}
