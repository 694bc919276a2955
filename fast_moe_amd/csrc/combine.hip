// Weighted merge of the K expert rows of every token (gather form, no atomics):
// each output row is produced by exactly one wavefront that adds its K source
// rows in ascending source-row order, which is the order of a sequential
// index_add and therefore reproducible bit for bit.
#include "common.h"

namespace fmoe {
namespace {

template <typename T>
struct Elem;
template <>
struct Elem<float> {
    static constexpr int kVec = 4;
    __device__ static float load(const float* p) { return *p; }
    __device__ static void store(float* p, float v) { *p = v; }
    __device__ static void unpack(const u32x4& raw, float* f) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(raw[i]);
    }
    __device__ static u32x4 pack(const float* f) {
        return u32x4{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]),
                     __float_as_uint(f[3])};
    }
};
template <>
struct Elem<uint16_t> {
    static constexpr int kVec = 8;
    __device__ static float load(const uint16_t* p) { return bf16_bits_to_f32(*p); }
    __device__ static void store(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
    __device__ static void unpack(const u32x4& raw, float* f) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = bf16_bits_to_f32(raw[i] & 0xffffu);
            f[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
        }
    }
    __device__ static u32x4 pack(const float* f) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = cvt_pk_bf16(f[2 * i], f[2 * i + 1]);
        return r;
    }
};

struct GateView {
    const void* ptr;
    int64_t cols, stride_row, stride_col;
    const int64_t* index;
    int64_t numel;
};

template <typename TG>
__device__ __forceinline__ float gate_of(const GateView& g, int64_t r, bool& ok) {
    int64_t flat = g.index ? g.index[r] : r;
    ok = (uint64_t)flat < (uint64_t)g.numel;
    if (!ok) return 0.0f;
    const int64_t gr = flat / g.cols, gc = flat - gr * g.cols;
    return Elem<TG>::load((const TG*)g.ptr + gr * g.stride_row + gc * g.stride_col);
}

// TV value dtype, TG gate dtype, ROUND_BF16: the product is rounded to bf16
// (both operands bf16); HAS_GATE false = plain segmented sum.
// VECTOR: 16-byte loads; one wave covers CPW * 64 * kVec consecutive columns of one token.
// The K source rows and gates of the token are fetched by lanes 0..K-1 in three parallel
// rounds (reverse_index -> gates_index -> gate) and handed out with readlane; rows are
// loaded in batches of JB with all loads of a batch in flight, then added in order.
template <typename TV, typename TG, typename TO, bool HAS_GATE, bool ROUND_BF16, bool VECTOR, int CPW>
__global__ __launch_bounds__(256) void combine_kernel(const TV* __restrict__ value, int64_t T, int K,
                                                      int64_t D, int64_t stride_row,
                                                      const int64_t* __restrict__ reverse_index,
                                                      GateView gate, TO* __restrict__ out,
                                                      int groups_per_token) {
    constexpr int VEC = VECTOR ? Elem<TV>::kVec : 1;
    constexpr int JB = 8;
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
    const int64_t t = wave / groups_per_token;
    const int group = (int)(wave - t * groups_per_token);
    if (t >= T) return;
    const int64_t R = T * K;

    // lanes 0..K-1 (K <= 64 per pass) own one source row each
    float acc[CPW][VEC];
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[c][i] = 0.0f;
    int64_t col[CPW];
    bool active[CPW];
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
        col[c] = (((int64_t)group * CPW + c) * kWave + lane) * VEC;
        active[c] = col[c] < D;
    }

    for (int k0 = 0; k0 < K; k0 += kWave) {
        const int kn = K - k0 < kWave ? K - k0 : kWave;
        int64_t my_r = -1;
        float my_w = 1.0f;
        if (lane < kn) {
            my_r = reverse_index[t * K + k0 + lane];
            if ((uint64_t)my_r >= (uint64_t)R) my_r = -1;        // malformed index: contributes nothing
            if (HAS_GATE && my_r >= 0) {
                bool ok;
                my_w = gate_of<TG>(gate, my_r, ok);
                if (!ok) my_r = -1;
            }
        }
        for (int j0 = 0; j0 < kn; j0 += JB) {
            u32x4 raw[JB][CPW];
            float sv[JB][CPW];
            int64_t rj[JB];
            float wj[JB];
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) {
                const int j = j0 + jj < kn ? j0 + jj : kn - 1;
                rj[jj] = wave_bcast(my_r, j);
                wj[jj] = wave_bcast(my_w, j);
                if (j0 + jj >= kn) rj[jj] = -1;
#pragma unroll
                for (int c = 0; c < CPW; ++c) {
                    raw[jj][c] = u32x4{0, 0, 0, 0};
                    sv[jj][c] = 0.0f;
                    if (rj[jj] >= 0 && active[c]) {
                        const TV* src = value + rj[jj] * stride_row + col[c];
                        if (VECTOR) raw[jj][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src));
                        else sv[jj][c] = Elem<TV>::load(src);
                    }
                }
            }
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) {
                if (rj[jj] < 0) continue;
#pragma unroll
                for (int c = 0; c < CPW; ++c) {
                    float f[VEC];
                    if (VECTOR) Elem<TV>::unpack(raw[jj][c], f);
                    else f[0] = sv[jj][c];
                    if constexpr (HAS_GATE && ROUND_BF16 && VEC % 2 == 0) {
#pragma unroll
                        for (int i = 0; i < VEC; i += 2) {       // products rounded to bf16 two at a time
                            const uint32_t pk = cvt_pk_bf16(f[i] * wj[jj], f[i + 1] * wj[jj]);
                            acc[c][i] = acc[c][i] + __uint_as_float(pk << 16);
                            acc[c][i + 1] = acc[c][i + 1] + __uint_as_float(pk & 0xffff0000u);
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < VEC; ++i) {
                            float p = HAS_GATE ? f[i] * wj[jj] : f[i];
                            if (HAS_GATE && ROUND_BF16) p = round_bf16(p);
                            acc[c][i] = acc[c][i] + p;
                        }
                    }
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
        if (!active[c]) continue;
        if (VECTOR && sizeof(TO) == sizeof(TV)) {
            *reinterpret_cast<u32x4*>(out + t * D + col[c]) = Elem<TO>::pack(acc[c]);
        } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i) Elem<TO>::store(out + t * D + col[c] + i, acc[c][i]);
        }
    }
}

template <typename TV, typename TG, typename TO, bool HAS_GATE, bool ROUND_BF16>
void launch(const void* value, int64_t T, int K, int64_t D, int64_t stride_row,
            const int64_t* reverse_index, const GateView& gate, void* out, hipStream_t stream) {
    constexpr int vec = Elem<TV>::kVec;
    const bool vector = (D % vec) == 0 && (stride_row % vec) == 0 && aligned16(value) && aligned16(out);
    const int per_chunk = kWave * (vector ? vec : 1);
    const int chunks = (int)((D + per_chunk - 1) / per_chunk);
    const bool wide = vector && chunks >= 2;                 // two 16-byte chunks per lane
    const int groups = wide ? (chunks + 1) / 2 : chunks;
    const int64_t waves = T * groups;
    const unsigned blocks = (unsigned)((waves + 3) / 4);
#define FMOE_COMBINE(VECTOR, CPW)                                                                  \
    combine_kernel<TV, TG, TO, HAS_GATE, ROUND_BF16, VECTOR, CPW><<<blocks, 256, 0, stream>>>(        \
        (const TV*)value, T, K, D, stride_row, reverse_index, gate, (TO*)out, groups)
    if (wide) FMOE_COMBINE(true, 2);
    else if (vector) FMOE_COMBINE(true, 1);
    else FMOE_COMBINE(false, 1);
#undef FMOE_COMBINE
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_combine(const void* value, int value_dtype, int64_t T, int K, int64_t D,
                            int64_t value_stride_row, const int64_t* reverse_index, const void* gates,
                            int gates_dtype, int64_t gates_cols, int64_t gates_stride_row,
                            int64_t gates_stride_col, const int64_t* gates_index, void* out, int out_dtype,
                            fmoe_stream_t stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    FMOE_REQUIRE(T >= 0 && K >= 1 && D >= 1, "fmoe_combine: need T >= 0, K >= 1, D >= 1");
    FMOE_REQUIRE(value_dtype == FMOE_BF16 || value_dtype == FMOE_F32, "fmoe_combine: value must be bf16 or fp32");
    if (T == 0) return FMOE_OK;
    FMOE_REQUIRE(value && reverse_index && out, "fmoe_combine: NULL pointer");
    FMOE_REQUIRE(value_stride_row >= D, "fmoe_combine: value row stride %lld < D %lld",
                 (long long)value_stride_row, (long long)D);
    FMOE_REQUIRE(T * (int64_t)((D + 63) / 64) < ((int64_t)1 << 33), "fmoe_combine: problem too large");
    GateView g{gates, gates_cols, gates_stride_row, gates_stride_col, gates_index, T * (int64_t)K};
    int expect_out = value_dtype;
    if (gates) {
        FMOE_REQUIRE(gates_dtype == FMOE_BF16 || gates_dtype == FMOE_F32, "fmoe_combine: gates must be bf16 or fp32");
        FMOE_REQUIRE(gates_cols >= 1, "fmoe_combine: gates_cols < 1");
        if (gates_dtype == FMOE_F32) expect_out = FMOE_F32;
    }
    FMOE_REQUIRE(out_dtype == expect_out,
                 "fmoe_combine: out dtype must be the promoted dtype of value and gates (%d), got %d",
                 expect_out, out_dtype);
    const bool vb = value_dtype == FMOE_BF16;
    if (!gates) {
        if (vb) launch<uint16_t, float, uint16_t, false, false>(value, T, K, D, value_stride_row, reverse_index, g, out, stream);
        else launch<float, float, float, false, false>(value, T, K, D, value_stride_row, reverse_index, g, out, stream);
    } else if (vb && gates_dtype == FMOE_BF16) {
        launch<uint16_t, uint16_t, uint16_t, true, true>(value, T, K, D, value_stride_row, reverse_index, g, out, stream);
    } else if (vb) {
        launch<uint16_t, float, float, true, false>(value, T, K, D, value_stride_row, reverse_index, g, out, stream);
    } else if (gates_dtype == FMOE_BF16) {
        launch<float, uint16_t, float, true, false>(value, T, K, D, value_stride_row, reverse_index, g, out, stream);
    } else {
        launch<float, float, float, true, false>(value, T, K, D, value_stride_row, reverse_index, g, out, stream);
    }
    return check_launch("fmoe_combine");
}
