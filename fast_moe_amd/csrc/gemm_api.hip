// fmoe_grouped_gemm: argument checks and kernel selection for the jagged GEMM.
#include "gemm_kernel.h"

#include <cstdlib>

using namespace fmoe;

namespace fmoe {
int compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

int lds_per_block() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || n <= 0) n = 65536;
        cached[dev] = n;
    }
    return cached[dev];
}
}  // namespace fmoe

// Checks the descriptor, fills the kernel parameters and picks the kernel.  sel < 0: nothing to do.
static int prepare_gemm(const fmoe_gemm_desc* d, GemmParams& p, int& sel) {
    sel = -1;
    FMOE_REQUIRE(d != nullptr, "fmoe_grouped_gemm: desc is NULL");
    FMOE_REQUIRE(d->num_experts >= 1 && d->n >= 1 && d->k >= 1,
                 "fmoe_grouped_gemm: need E, n, k >= 1 (E=%d n=%d k=%d)", d->num_experts, d->n, d->k);
    FMOE_REQUIRE(d->total_rows >= 0, "fmoe_grouped_gemm: total_rows < 0");
    FMOE_REQUIRE(d->a_dtype == FMOE_BF16 || d->a_dtype == FMOE_E4M3 || d->a_dtype == FMOE_F32,
                 "fmoe_grouped_gemm: operands must be bf16, e4m3 or fp32 (got dtype %d)", d->a_dtype);
    FMOE_REQUIRE(d->out_dtype == (d->a_dtype == FMOE_F32 ? FMOE_F32 : FMOE_BF16),
                 "fmoe_grouped_gemm: output must be bf16 (fp32 for fp32 operands)");
    FMOE_REQUIRE(d->epilogue >= FMOE_EPI_NONE && d->epilogue <= FMOE_EPI_GATED,
                 "fmoe_grouped_gemm: unknown epilogue %d", d->epilogue);
    if (d->total_rows == 0) return FMOE_OK;     // sel stays -1
    FMOE_REQUIRE(d->offsets && d->a && d->b && d->out, "fmoe_grouped_gemm: NULL tensor pointer");
    FMOE_REQUIRE(d->a_rows >= 1, "fmoe_grouped_gemm: a_rows < 1");
    FMOE_REQUIRE(d->index_div >= 1, "fmoe_grouped_gemm: index_div < 1");
    const bool row_indexed = d->a_stride_k > 1;      // A (and B) given with k as the row index
    if (!row_indexed)
        FMOE_REQUIRE(d->a_stride_row >= d->k, "fmoe_grouped_gemm: A row stride %lld < k %d",
                     (long long)d->a_stride_row, d->k);
    FMOE_REQUIRE(d->out_stride_row >= d->n, "fmoe_grouped_gemm: out row stride %lld < n %d",
                 (long long)d->out_stride_row, d->n);
    const bool fp8 = d->a_dtype == FMOE_E4M3;
    const bool f32 = d->a_dtype == FMOE_F32;
    const bool swiglu = d->epilogue == FMOE_EPI_SWIGLU;
    if (swiglu) FMOE_REQUIRE(d->b2 != nullptr, "fmoe_grouped_gemm: SWIGLU needs b2");
    const bool gated = d->epilogue == FMOE_EPI_GATED;
    if (gated) {
        FMOE_REQUIRE(d->aux && !d->aux2, "fmoe_grouped_gemm: GATED reads its gate from aux (aux2 stays NULL)");
        if (d->a_dtype != FMOE_BF16)
            return fmoe::fail(FMOE_ERR_UNSUPPORTED, "fmoe_grouped_gemm: the GATED epilogue is built for bf16 operands");
        FMOE_REQUIRE(!d->a_silu && !d->out2 && !d->a2, "fmoe_grouped_gemm: GATED goes without a_silu, out2 and a2");
    } else {
        FMOE_REQUIRE((d->aux == nullptr) == (d->aux2 == nullptr), "fmoe_grouped_gemm: aux and aux2 come together");
    }
    if (d->aux) {
        FMOE_REQUIRE(swiglu || gated, "fmoe_grouped_gemm: aux outputs are the SWIGLU pre-activations");
        FMOE_REQUIRE(d->aux_stride_row >= d->n, "fmoe_grouped_gemm: aux row stride %lld < n %d",
                     (long long)d->aux_stride_row, d->n);
    }
    const bool two = d->a2 != nullptr;               // out = a * b + a2 * b2
    if (two)
        FMOE_REQUIRE(d->b2 && d->k2 >= 1 && d->epilogue == FMOE_EPI_NONE && !d->k_window && !row_indexed,
                     "fmoe_grouped_gemm: a2 needs b2 and k2, and goes with no epilogue and no k_window");
    if (two) FMOE_REQUIRE(d->k <= (1 << 30) && d->k2 <= (1 << 30), "fmoe_grouped_gemm: k + k2 does not fit 32 bits");
    const int ktot = d->k + (two ? d->k2 : 0);
    if (fp8) {
        FMOE_REQUIRE(d->a_scale && d->b_scale, "fmoe_grouped_gemm: e4m3 operands need a_scale and b_scale");
        if (swiglu) FMOE_REQUIRE(d->b2_scale != nullptr, "fmoe_grouped_gemm: SWIGLU e4m3 needs b2_scale");
        FMOE_REQUIRE(!d->a_silu, "fmoe_grouped_gemm: a_silu is not defined for e4m3 operands");
    }

    p.offsets = d->offsets;
    p.row_index = d->row_index;
    p.E = d->num_experts;
    p.N = d->n;
    p.K = ktot;
    p.out2 = (uint16_t*)d->out2;
    p.out_half = 0;
    if (d->out2) {
        FMOE_REQUIRE(row_indexed && d->total_rows % (2 * (int64_t)d->num_experts) == 0 &&
                         (d->total_rows / (2 * (int64_t)d->num_experts)) % 32 == 0 && aligned16(d->out2),
                     "fmoe_grouped_gemm: out2 goes with a_stride_k and experts of 2 * h output rows each, h a "
                     "multiple of 32 (total_rows=%lld E=%d)", (long long)d->total_rows, d->num_experts);
        p.out_half = d->total_rows / (2 * (int64_t)d->num_experts);
    }
    p.a2 = (const uint8_t*)d->a2;
    p.k_split = d->k;
    p.index_div = d->index_div;
    p.index_shift = -1;
    for (int s = 0; s < 31; ++s)
        if (d->index_div == (1 << s)) p.index_shift = s;
    magic_u31(d->index_div, &p.index_magic, &p.index_magic_shift);     // (read when index_div is no power of two)
    p.total_rows = d->total_rows;
    p.a_rows = d->a_rows;
    p.a = (const uint8_t*)d->a;
    p.a_stride_row = d->a_stride_row;
    p.a_stride_e = d->a_stride_e;
    p.a_sk = row_indexed ? d->a_stride_k : 1;
    p.a_scale = d->a_scale;
    p.b = (const uint8_t*)d->b;
    p.b2 = (const uint8_t*)d->b2;
    p.b_se = d->b_stride_e;
    p.b_sk = d->b_stride_k;
    p.b_sn = d->b_stride_n;
    p.b_scale = d->b_scale;
    p.b2_scale = d->b2_scale;
    p.bias = (const uint16_t*)d->bias;
    p.bias2 = (const uint16_t*)d->bias2;
    p.bias_se = d->bias_stride_e;
    p.out = (uint16_t*)d->out;
    p.out_stride = d->out_stride_row;
    p.n_tiles = 0;
    // 16-byte stores: 8 bf16 (4 fp32) output columns at a time
    const int vec_cols = f32 ? 4 : 8;
    p.k_window = d->k_window;
    p.k_window_multiple = d->k_window ? d->k_window_multiple : 0;
#ifdef FMOE_TRACE
    {   // debug builds only: FMOE_TRACE_PTR=<device address in hex> of a zeroed 2 x [grid][32][2][8] uint64 buffer
        const char* t = getenv("FMOE_TRACE_PTR");
        p.trace = t ? (uint64_t*)strtoull(t, nullptr, 16) : nullptr;
    }
#endif
    p.aux = (uint16_t*)d->aux;
    p.aux2 = (uint16_t*)d->aux2;
    p.aux_stride = d->aux_stride_row;
    // (the vector-store path addresses a row inside a 32-row block with a 32-bit byte offset)
    const int64_t stride_cap = (int64_t)1 << 25;
    p.vec_store = (d->n % vec_cols == 0) && (d->out_stride_row % vec_cols == 0) && aligned16(d->out) &&
                  d->out_stride_row < stride_cap &&
                  (!d->aux || gated || ((d->aux_stride_row % vec_cols == 0) && aligned16(d->aux) && aligned16(d->aux2) &&
                                        d->aux_stride_row < stride_cap));

    p.short_tile_rows = 0;      // (the paired ring's launcher decides)
    p.gate_vec16 = gated && aligned16(d->aux) && d->aux_stride_row % 8 == 0;
    p.gate_vec = gated && (reinterpret_cast<uintptr_t>(d->aux) % 8 == 0) && d->aux_stride_row % 4 == 0;
    p.scale_pow2 = fp8 && d->scale_pow2 != 0;
    p.scale_vec = fp8 && d->n >= 4 && d->n % 4 == 0 && aligned16(d->b_scale) && (!d->b2_scale || aligned16(d->b2_scale));
    const int esize = fp8 ? 1 : (f32 ? 4 : 2);
    const int chunk = 16 / esize;
    const bool fast = d->b_stride_k == 1 && (d->k % chunk) == 0 && aligned16(d->a) && aligned16(d->b) &&
                      (!swiglu || aligned16(d->b2)) && (d->a_stride_row % chunk) == 0 &&
                      (d->a_stride_e % chunk) == 0 && (d->b_stride_n % chunk) == 0 &&
                      (d->b_stride_e % chunk) == 0;
    // rows per expert decide the tile height: tall tiles for prefill-like loads,
    // short ones when the experts see a handful of rows (weight-streaming regime)
    const bool big = d->total_rows / d->num_experts >= 96;
    // the ring kernel moves whole 64-byte K-slices by LDS-DMA and stores 16-byte groups
    const int slice = 64 / esize;
    // ... and addresses rows as a 64-bit base per expert plus a 32-bit byte offset
    const int64_t span32 = ((int64_t)1 << 32) - 4096;
    const bool near = d->a_rows * d->a_stride_row * esize + (int64_t)d->k * esize < span32 &&
                      (int64_t)d->n * d->b_stride_n * esize + (int64_t)d->k * esize < span32;
    const bool ring = fast && big && !f32 && !d->a_silu && (d->k % slice) == 0 && d->k / slice >= 3 &&
                      p.vec_store && d->num_experts <= 1024 && d->total_rows < ((int64_t)1 << 31) * 128 && near;
    // N-contiguous bf16 weights (B[e][k][n], n fastest) are read in place by the paired ring
    const bool ring_tr = !fp8 && !f32 && big && !d->a_silu && !d->k_window && d->b_stride_n == 1 &&
                         d->b_stride_k != 1 && (d->b_stride_k % chunk) == 0 && (d->b_stride_e % chunk) == 0 &&
                         (d->a_stride_row % chunk) == 0 && (d->a_stride_e % chunk) == 0 && aligned16(d->a) &&
                         aligned16(d->b) && (!(swiglu || two) || aligned16(d->b2)) && (d->k % (2 * slice)) == 0 &&
                         (ktot % (2 * slice)) == 0 && (!two || aligned16(d->a2)) &&
                         ktot / slice >= 4 && p.vec_store && d->num_experts <= TileRing5W::kMaxExperts &&
                         d->total_rows < ((int64_t)1 << 31) && lds_per_block() >= TileRing5::LDS_BYTES &&
                         d->a_rows * d->a_stride_row * esize + (int64_t)ktot * esize < span32 &&
                         ((int64_t)ktot * d->b_stride_k + d->n) * esize < span32;
    // the second product exists in that kernel only; a caller that is turned away runs two
    // GEMMs and adds
    if (two)
        FMOE_REQUIRE(ring_tr, "fmoe_grouped_gemm: a2 * b2 is summed in only by the kernel that reads bf16 weights "
                              "B[e][k][n] with n contiguous: k and k2 in multiples of 128, 16-byte alignment, "
                              "96 or more rows per expert on average, E <= 256, a 160 KB LDS");
    // a contraction window is followed by the paired ring only (bf16, no epilogue, whole pairs of
    // slices as promised by the caller, register tables); otherwise by the register-staged kernel
    const bool ring_window = !fp8 && d->epilogue == FMOE_EPI_NONE && (d->k / slice) % 2 == 0 && d->k / slice >= 4 &&
                             d->k_window_multiple >= 2 * slice && d->k_window_multiple % (2 * slice) == 0 &&
                             d->num_experts <= TileRing5W::kMaxExperts && d->total_rows < ((int64_t)1 << 31) &&
                             lds_per_block() >= TileRing5::LDS_BYTES;
    const bool take_ring = ring && (!d->k_window || ring_window);
    if (row_indexed) {
        // the weight gradient from the row-major tensors themselves: paired ring only
        const bool ok = !fp8 && !f32 && d->epilogue == FMOE_EPI_NONE && d->k_window && !d->a_silu &&
                        d->a_stride_row == 1 && d->b_stride_n == 1 && d->a_stride_e == 0 &&
                        (d->a_stride_k % chunk) == 0 && (d->b_stride_k % chunk) == 0 && (d->b_stride_e % chunk) == 0 &&
                        aligned16(d->a) && aligned16(d->b) && (d->total_rows % 8) == 0 && p.vec_store &&
                        d->k_slack_rows >= 4 * slice && d->k >= 4 * slice &&
                        d->num_experts <= TileRing5W::kMaxExperts && d->total_rows < ((int64_t)1 << 31) &&
                        lds_per_block() >= TileRing5::LDS_BYTES &&
                        ((int64_t)2 * slice * d->a_stride_k + d->total_rows) * esize < span32 &&
                        ((int64_t)2 * slice * d->b_stride_k + d->n) * esize < span32;
        FMOE_REQUIRE(ok, "fmoe_grouped_gemm: row-indexed operands (a_stride_k > 1) need bf16, no epilogue, a "
                         "k_window, unit strides along A's rows and B's columns, 16-byte alignment, row counts "
                         "in multiples of 8, k_slack_rows >= 128, E <= 256 and a 160 KB LDS");
        sel = kSelRing;
        return FMOE_OK;
    }
    sel = ring_tr ? kSelRing : !fast ? kSelGeneric : take_ring ? kSelRing : big ? kSelStagedBig : kSelStagedSmall;
    return FMOE_OK;
}

extern "C" int fmoe_grouped_gemm(const fmoe_gemm_desc* d, fmoe_stream_t stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    GemmParams p;
    int sel;
    if (int rc = prepare_gemm(d, p, sel)) return rc;
    if (sel < 0) return FMOE_OK;
    if (d->a_dtype == FMOE_E4M3) return run_gemm_fp8(p, d->epilogue, sel, stream);
    if (d->a_dtype == FMOE_F32) return run_gemm_f32(p, d->epilogue, d->a_silu != 0, sel, stream);
    return run_gemm_bf16(p, d->epilogue, d->a_silu != 0, sel, stream);
}

extern "C" int fmoe_grouped_gemm_plan(const fmoe_gemm_desc* d, int* plan) {
    FMOE_REQUIRE(plan != nullptr, "fmoe_grouped_gemm_plan: plan is NULL");
    GemmParams p;
    int sel;
    if (int rc = prepare_gemm(d, p, sel)) return rc;
    *plan = sel < 0 ? FMOE_PLAN_NONE : sel;
    return FMOE_OK;
}
