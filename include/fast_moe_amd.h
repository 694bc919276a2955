/*
 * fast_moe_amd -- C ABI of libfastmoe_hip.so: the MoE-forward hot path of
 * meta-recsys/fast_moe as hand-written gfx950 (MI355X) HIP kernels.
 *
 * Conventions shared by every entry point
 *   - plain pointers and sizes only; every pointer is a DEVICE pointer unless
 *     stated otherwise; the caller owns all memory, the library allocates none,
 *     keeps no pointer past the call and holds no global state;
 *   - all work is enqueued on `stream` (a hipStream_t passed as void*) and the
 *     call returns without synchronising the host;
 *   - return value 0 = success; non-zero = error, message from fmoe_last_error()
 *     (thread local).  Nothing is launched when an argument check fails;
 *   - index tensors are int64 (what torch.sort / cumsum hand the reference),
 *     row addressing is 64-bit inside.
 *
 * Reference citations are relative to the root of meta-recsys/fast_moe.
 */
#ifndef FAST_MOE_AMD_H
#define FAST_MOE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* fmoe_stream_t; /* hipStream_t */

enum fmoe_dtype {
    FMOE_F32 = 0,
    FMOE_BF16 = 1,
    FMOE_E4M3 = 2 /* OCP float8 e4m3fn bytes + fp32 row scales */
};

enum fmoe_epilogue {
    FMOE_EPI_NONE = 0,  /* out = acc + bias                                  */
    FMOE_EPI_SILU = 1,  /* out = silu(round(acc + bias))                     */
    FMOE_EPI_SWIGLU = 2, /* out = silu(round(acc + bias)) * round(acc2 + bias2) */
    FMOE_EPI_GATED = 3   /* out = round(silu(gate)) * round(acc + bias), gate = the [total_rows, n]
                            bf16 tensor in desc.aux (an input here): the second GEMM of the gating
                            operator whose two GEMMs read different inputs, multiplied into the
                            first one's result where it is produced (the one kernel with two input
                            pointers of kernels/triton/triton_moe.py:2993-3159 as two launches
                            without the product's round trip); bf16 operands only              */
};

enum fmoe_status {
    FMOE_OK = 0,
    FMOE_ERR_ARGUMENT = 1,    /* bad shape / dtype / null pointer / alignment   */
    FMOE_ERR_UNSUPPORTED = 2, /* valid request this build has no kernel for     */
    FMOE_ERR_WORKSPACE = 3,   /* workspace too small                            */
    FMOE_ERR_LAUNCH = 4       /* hipGetLastError() after a launch               */
};

/* Library version (major*10000 + minor*100 + patch). No reference counterpart. */
int fmoe_version(void);

/* Message of the last non-zero return on this thread ("" if none).  No reference counterpart:
 * its errors are Python assert / ValueError / NotImplementedError (kernels/moe.py:277-280,
 * kernels/moe_fp8.py:73-74); the Python layer above this library raises from this message. */
const char* fmoe_last_error(void);

/* ------------------------------------------------------------------ routing */

/* Bytes of scratch fmoe_route_topk / fmoe_route_from_topk need for (T, E, K).  No reference
 * counterpart: its two sorts allocate inside torch (modules/fast_moe_module.py:107-144); here
 * the caller owns every byte. */
size_t fmoe_route_workspace_bytes(int64_t T, int E, int K);

/*
 * Top-k expert selection, L1 gate renormalisation and the jagged routing
 * tensors, from gate probabilities.
 * Replaces FastMoELayer._select_top_k_experts + _compute_routing_metadata
 * (modules/fast_moe_module.py:93-144) including the third-party
 * torch.ops.fbgemm.asynchronous_complete_cumsum call at :131.
 *
 *   scores        [T, E] row-major, FMOE_F32 or FMOE_BF16 (softmax output)
 *   renorm        gate mode.  0: gates = selected scores.
 *                 1: gates = v / max(sum|v|, 1e-12) in the scores' dtype (F.normalize, :103).
 *                 2, 3: `scores` are router LOGITS, the SGMoE router of utils/utils.py:139-164
 *                 (_compute_top_logits): logits L2-normalised over the experts, selection in
 *                 descending stable order, gates = softmax of the normalised logits over all
 *                 experts (2, post_softmax=False) or over the K selected ones (3, post_softmax=True)
 * outputs
 *   topk_idx      [T, K] int64  selected experts; slot order = descending score,
 *                               equal scores -> lower expert id first
 *   gates         [T, K] scores' dtype
 *   lengths       [E]    int64  rows per expert
 *   offsets       [E+1]  int64  exclusive prefix sum of lengths
 *   gate_index    [T*K]  int64  stable argsort of topk_idx.view(-1)      (:122)
 *   token_index   [T*K]  int64  gate_index / K                           (:124)
 *   reverse_index [T, K] int64  stable argsort of token_index            (:132)
 * Limits: 1 <= K <= E <= 512, K <= 64.
 */
int fmoe_route_topk(const void* scores, int score_dtype, int64_t T, int E, int K, int renorm,
                    int64_t* topk_idx, void* gates, int64_t* lengths, int64_t* offsets,
                    int64_t* gate_index, int64_t* token_index, int64_t* reverse_index,
                    void* workspace, size_t workspace_bytes, fmoe_stream_t stream);

/*
 * fmoe_route_topk without a workspace argument and without any allocation: the scratch lives in
 * device memory that is part of the library image (6.3 MiB per GPU the library runs on, held until
 * the process ends).  No counterpart in the reference.  For callers that cannot allocate: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same arguments
 * and results as fmoe_route_topk, bit for bit.
 * Limits: T * K <= FMOE_ROUTE_STATIC_MAX_POSITIONS, E <= FMOE_ROUTE_STATIC_MAX_EXPERTS; larger
 * calls are turned away with FMOE_ERR_ARGUMENT (use fmoe_route_topk with a workspace).
 * Every call on a GPU uses that GPU's one buffer: calls that may overlap on one GPU (two
 * streams, two threads) race; calls on one stream, or ordered by events, do not.  The first call
 * on a device looks the buffer's address up (hipGetSymbolAddress); make that call outside a
 * graph capture.
 */
#define FMOE_ROUTE_STATIC_MAX_POSITIONS (1 << 20)
#define FMOE_ROUTE_STATIC_MAX_EXPERTS 512
int fmoe_route_topk_static(const void* scores, int score_dtype, int64_t T, int E, int K, int renorm,
                           int64_t* topk_idx, void* gates, int64_t* lengths, int64_t* offsets,
                           int64_t* gate_index, int64_t* token_index, int64_t* reverse_index,
                           fmoe_stream_t stream);

/*
 * The same routing tensors for a caller that already holds the selected expert
 * ids (the generator of kernels/tests/moe_test.py:191-197,241: topk -> stable
 * sort -> scatter_add -> complete cumsum).  topk_idx values must lie in [0, E);
 * out-of-range ids are counted into no expert and reported through
 * `bad_count` (device int64, may be NULL); the positions they leave unfilled (the
 * tail of gate_index / token_index behind offsets[E], the last slots of their
 * token's reverse_index row) hold 0.  Limits: E <= 1024, K <= 64.
 */
int fmoe_route_from_topk(const int64_t* topk_idx, int64_t T, int E, int K,
                         int64_t* lengths, int64_t* offsets, int64_t* gate_index,
                         int64_t* token_index, int64_t* reverse_index, int64_t* bad_count,
                         void* workspace, size_t workspace_bytes, fmoe_stream_t stream);

/* ---------------------------------------------------------- FP8 quantisation */

/*
 * Row-wise OCP e4m3fn quantisation with a power-of-two multiplier scale
 * 2^floor(log2(448/amax)) per row.
 * Replaces pytorch_rowwise_quant_fp8 / pytorch_transpose_rowwise_quant_fp8
 * (kernels/pytorch/quant_fp8.py:13-40), pytorch_silu_jagged_fp8 and
 * pytorch_bmm_weight_rowwise_quant_fp8 (kernels/pytorch/moe_fp8.py:17-43),
 * i.e. triton_rowwise_quant_fp8 & co (kernels/triton/triton_quant_fp8.py:130-302).
 *
 *   a      logical [batch, rows, cols] read through element strides a_stride_*;
 *          the amax runs over `cols`.  FMOE_BF16 or FMOE_F32.
 *   q      e4m3fn bytes written through element strides q_stride_*
 *   scale  [batch, rows] fp32, contiguous: the multiplier, or its reciprocal
 *          when store_reciprocal != 0 (the convention of
 *          kernels/triton/triton_quant_fp8.py:273-277)
 *   apply_silu  quantise silu(a) (rounded to a's dtype first) instead of a
 */
int fmoe_quant_rows_e4m3(const void* a, int a_dtype, int64_t batch, int64_t rows, int64_t cols,
                         int64_t a_stride_b, int64_t a_stride_r, int64_t a_stride_c,
                         int apply_silu, uint8_t* q, int64_t q_stride_b, int64_t q_stride_r,
                         int64_t q_stride_c, float* scale, int store_reciprocal,
                         fmoe_stream_t stream);

/* -------------------------------------------------------------- grouped GEMM */

/*
 * One jagged ("grouped") GEMM over expert segments:
 *   for e in [0, E), r in [offsets[e], offsets[e+1]):
 *     src      = row_index ? row_index[r] / index_div : r
 *     acc [n]  = sum_k A [src, k] * B [e, k, n]
 *     acc2[n]  = sum_k A [src, k] * B2[e, k, n]              (SWIGLU only)
 *     out[r,n] = epilogue(acc (+bias[e,n]), acc2 (+bias2[e,n]))
 * With FMOE_E4M3 operands acc is divided by a_scale[src] * b_scale[e, n]
 * (multiplier scales) before the bias, as kernels/pytorch/moe_fp8.py:127-137.
 *
 * Replaces, by choice of fields:
 *   index_select_jagged_bmm          kernels/moe.py:39-68     (row_index, EPI_NONE)
 *   index_select_jagged_bmm_swiglu   kernels/moe.py:156-189   (row_index, EPI_SWIGLU)
 *   index_select_jagged_bmm_3D       kernels/moe.py:118-153   (a_stride_e != 0)
 *   the GEMM half of silu_jagged_bmm_combine kernels/moe.py:236-292
 *                                    (row_index NULL, a_silu = has_silu)
 *   index_select_jagged_bmm(fp8=True) kernels/moe_fp8.py:185-248 (FMOE_E4M3)
 *   the GEMM of silu_jagged_bmm_combine_fp8 kernels/moe_fp8.py:127-182
 * i.e. the Triton kernels kernels/triton/triton_moe.py:184-282, 2526-2671,
 * 3167-3347, kernels/triton/triton_moe_fp8.py:672-884 and
 * kernels/triton/triton_gemm_fp8.py:55-204.
 *
 * All strides are in elements.  B is addressed as B[e*b_stride_e + k*b_stride_k
 * + n*b_stride_n], so both [E,K,N]-contiguous weights and [E,K,N] views of
 * [E,N,K] storage are consumed in place.  No host synchronisation: tile
 * scheduling reads `offsets` on the device; max_seq_len is not needed.
 *
 * With k_window the contraction range differs per expert: this is the weight
 * gradient of the operators above, dW[e] = A_e^T x dOut_e reduced over the rows of
 * expert e (kernels/triton/triton_moe.py:1793-1976, 4030-4108), computed either on the
 * transposed, zero-padded operands fmoe_jagged_transpose writes or, with a_stride_k, on the
 * row-major tensors themselves.
 */
typedef struct fmoe_gemm_desc {
    int32_t num_experts;    /* E                                                  */
    int32_t n;              /* output columns (per B matrix)                      */
    int32_t k;              /* contraction length                                 */
    int32_t index_div;      /* divisor applied to row_index values (>= 1)         */
    int64_t total_rows;     /* rows of `out` (= offsets[E]; host-known upper bound) */
    int64_t a_rows;         /* rows of A (bound for gathered sources)             */
    const int64_t* offsets; /* [E+1]                                              */
    const int64_t* row_index; /* [total_rows] or NULL                             */

    const void* a;          /* [a_rows, k] (or [a_rows, E, k] with a_stride_e)    */
    int32_t a_dtype;        /* FMOE_BF16 | FMOE_E4M3 | FMOE_F32                   */
    int32_t a_silu;         /* apply SiLU to A elements on load (bf16 / fp32)      */
    int64_t a_stride_row;
    int64_t a_stride_e;     /* 0, or per-expert offset for the 3D variant         */
    const float* a_scale;   /* [a_rows] multiplier scales (FMOE_E4M3)             */

    const void* b;          /* same dtype as A                                    */
    const void* b2;         /* second weight (SWIGLU) or NULL                     */
    int64_t b_stride_e, b_stride_k, b_stride_n;
    const float* b_scale;   /* [E, n] multiplier scales (FMOE_E4M3); any 4-byte
                             * alignment works, 16-byte alignment loads 4 at a time */
    const float* b2_scale;

    const void* bias;       /* [E, n] in out_dtype, or NULL                       */
    const void* bias2;
    int64_t bias_stride_e;

    int32_t epilogue;       /* enum fmoe_epilogue                                 */
    int32_t out_dtype;      /* FMOE_BF16; FMOE_F32 iff a_dtype is FMOE_F32        */
    void* out;              /* [total_rows, n]                                    */
    int64_t out_stride_row;
    const int64_t* k_window; /* NULL, or [E+1]: expert e contracts over the k range
                                [k_window[e], k_window[e+1]) of A and B (then `k` is
                                only an upper bound); values multiples of 8          */
    int32_t k_window_multiple; /* 0, or a promise of the caller: every window length is a
                                multiple of this many elements and at least twice it
                                (64 or more lets the LDS-ring kernel take the call; a
                                broken promise gives wrong sums, never an access outside
                                the k columns of A and B)                              */
    int32_t k_slack_rows;   /* with a_stride_k: rows readable behind the last k row of A and of
                                B (128 or more; what they hold does not matter)      */
    void* aux;              /* with FMOE_EPI_GATED: the gate, read (aux2 NULL).  Otherwise
                                NULL, or with FMOE_EPI_SWIGLU [total_rows, n] in out_dtype:  */
    void* aux2;             /* receive A x B + bias (aux) and A x B2 + bias2 (aux2), the
                                two pre-activations the backward pass needs (the ALPHA and
                                BETA outputs of kernels/triton/triton_moe.py:2316-2345) */
    int64_t aux_stride_row;
    int64_t a_stride_k;     /* 0 / 1: A rows are contiguous along k.  > 1: both operands are given
                                with the contraction index as their row index, A[m][k] =
                                a[k*a_stride_k + m] (a_stride_row = 1) and B[k][n] = b[k*b_stride_k
                                + n] (b_stride_n = 1, b_stride_e = 0), and k_window holds arbitrary
                                row ranges: the weight gradient straight from the row gradients
                                [rows, n_out] and the expert-sorted input rows [rows, n_in], with
                                no transposed copies (bf16, FMOE_EPI_NONE, LDS-ring kernel only;
                                row_index is not used; every expert's output row count a multiple
                                of 8)                                                   */
    const void* a2;         /* NULL, or a second product summed into the same output:
                                out = a * b + a2 * b2, with a2 [rows, k2] and b2 [E, k2, n] under
                                the strides of a and b (so k2 = k unless the tensors are views of
                                larger ones).  The input gradient of a SwiGLU layer,
                                d_gate * W_gate + d_up * W_up, in one pass with one output; the
                                reference runs two GEMMs, rounds each and adds
                                (kernels/triton/triton_moe.py:2472-2500), here the sum is rounded
                                once.  bf16, FMOE_EPI_NONE (bias allowed), weights with n
                                contiguous (b_stride_n = 1), k and k2 in multiples of 128; other
                                descriptors with a2 are turned away with FMOE_ERR_ARGUMENT */
    int32_t k2;             /* contraction length of a2 * b2                                */
    int32_t scale_pow2;     /* FMOE_E4M3: non-zero = the caller promises that every value of a_scale,
                                b_scale and b2_scale is an exact power of two (what
                                fmoe_quant_rows_e4m3 writes, the convention of
                                kernels/pytorch/quant_fp8.py:13-24).  The LDS-ring kernel then lets
                                the MFMA instructions divide the scales out (as their E8M0 block
                                scales) instead of its epilogue; same results.  With 0 any fp32
                                scales are accepted.  A broken promise drops the mantissa of the
                                scale, nothing else                                            */
    void* out2;             /* NULL, or (with a_stride_k only) a second output: offsets then
                                describes experts of 2 * h rows each (h a multiple of 32), and
                                rows [h, 2h) of every expert are stored to out2 + (e * h + row - h) *
                                out_stride_row, rows [0, h) to out + (e * h + row) * out_stride_row:
                                the weight gradients of two matrices (SwiGLU's gate and up
                                projection, whose row gradients lie side by side) from one GEMM,
                                each into its own [E, h, n] tensor                          */
} fmoe_gemm_desc;

int fmoe_grouped_gemm(const fmoe_gemm_desc* desc /* host pointer */, fmoe_stream_t stream);

/* Which kernel fmoe_grouped_gemm would run for this descriptor on the current device
 * (no launch).  The Triton reference leaves this choice to its autotuner
 * (kernels/triton/triton_moe.py:146-183); here it is a pure function of the descriptor, so
 * a caller can see beforehand whether its weight layout is read in place by a streaming
 * kernel or only by the element-load kernel, and tests can name the path they cover. */
enum fmoe_gemm_plan {
    FMOE_PLAN_NONE = -1,          /* nothing to do (no rows)                                */
    FMOE_PLAN_RING = 0,           /* persistent LDS-ring kernel, 256 x 256 tiles            */
    FMOE_PLAN_STAGED = 1,         /* register-staged kernel, 256 x 256 tiles                */
    FMOE_PLAN_STAGED_SHORT = 2,   /* 64 x 256 tiles (few rows per expert): the streaming kernel,
                                     or the register-staged one where that does not apply   */
    FMOE_PLAN_ELEMENT = 3         /* element loads: any strides, any alignment              */
};
int fmoe_grouped_gemm_plan(const fmoe_gemm_desc* desc, int* plan);

/* ------------------------------------------------------------------ combine */

/*
 * Weighted, deterministic merge of the K expert rows of each token:
 *   out[t, :] = sum_{j<K} round(value[reverse_index[t,j], :] * w(reverse_index[t,j]))
 * accumulated in fp32 in ascending j (= ascending source row, the order of the
 * reference's CPU index_add), where w(r) = gates_flat[gates_index[r]]
 * (or gates_flat[r] if gates_index is NULL, or 1 if gates is NULL) and the
 * product is rounded to the promoted dtype of (value, gates) before the add.
 * Replaces pytorch_mul_merge_k_add (kernels/pytorch/moe.py:14-37) /
 * _mul_merge_k_add_fwd (kernels/triton/triton_moe.py:864-914), the second half
 * of silu_jagged_bmm_combine (kernels/moe.py:236-292).
 *
 *   value        [T*K, D], FMOE_BF16 or FMOE_F32, row stride value_stride_row
 *   gates        logical [gates_rows, gates_cols] read through strides (the
 *                reference flattens weight.contiguous().view(-1)); dtype
 *                FMOE_BF16 or FMOE_F32; NULL = unweighted
 *   out          [T, D] contiguous; dtype = promoted dtype of value and gates
 */
int fmoe_combine(const void* value, int value_dtype, int64_t T, int K, int64_t D,
                 int64_t value_stride_row, const int64_t* reverse_index, const void* gates,
                 int gates_dtype, int64_t gates_cols, int64_t gates_stride_row,
                 int64_t gates_stride_col, const int64_t* gates_index, void* out, int out_dtype,
                 fmoe_stream_t stream);

/* out[i] = silu(a[i]) * b[i] over n bf16 (or fp32) elements with the reference's rounding
 * points (F.silu(alpha) * beta, kernels/pytorch/moe.py:221): the element-wise
 * tail of index_select_jagged_gating_bmm when its two inputs differ.  b == NULL: out = silu(a)
 * (F.silu in the operand's dtype, kernels/pytorch/moe.py:266), the rows the weight gradient of
 * silu_jagged_bmm_combine(has_silu=True) contracts with. */
int fmoe_silu_mul(const void* a, const void* b, void* out, int dtype, int64_t n,
                  fmoe_stream_t stream);

/*
 * Measurement aid with no counterpart in the reference (bench.py --hbm-ceiling): streams `bytes`
 * of device memory at `buf` with nothing but memory accesses, so that the GB/s of the quantisers and
 * of the merge can be read against what this part delivers to a kernel that only reads
 * (mode 0), only writes (mode 1; the buffer is overwritten) or copies its first half to its second
 * (mode 2).  `per_lane` (1, 2, 4 or 8): 16-byte accesses per lane; the grid follows from it
 * (256 lanes per block).  `bytes`: a multiple of 32.
 */
int fmoe_hbm_probe(void* buf, int64_t bytes, int mode, int per_lane, fmoe_stream_t stream);

/*
 * dst[b, c, r] = src[b, r, c] for 1- or 2-byte elements: turns N-contiguous expert weights
 * [E, K, N] into the K-contiguous [E, N, K] storage the fast GEMM path streams.  The reference
 * has no counterpart (its Triton kernels read either layout through strides,
 * kernels/triton/triton_moe.py:238-242); callers that keep weights N-contiguous transpose once
 * per weight update, or per call as the Python wrapper does.
 *   src  logical [batch, rows, cols], cols contiguous, element strides src_stride_b / src_stride_r
 *   dst  [batch, cols, rows] contiguous
 */
int fmoe_transpose_last2(const void* src, void* dst, int elem_size, int64_t batch, int64_t rows,
                         int64_t cols, int64_t src_stride_b, int64_t src_stride_r, fmoe_stream_t stream);

/* ----------------------------------------------------------------- backward */

/*
 * Transposed, zero-padded copy of jagged rows, the operand layout of the weight-gradient GEMM:
 *   for e in [0, E), j in [0, len_e):  dst[c, pad_offsets[e] + j] = src[src_row(offsets[e] + j), c]
 *   dst[c, p] = 0 for the padding columns p in [pad_offsets[e] + len_e, pad_offsets[e+1])
 * with len_e = offsets[e+1] - offsets[e] and src_row(r) = row_index ? row_index[r] / index_div : r;
 * apply_silu != 0 stores silu(src) (rounded to dtype) instead, for the operator whose GEMM input
 * is silu(jagged) (kernels/pytorch/moe.py:255-275).
 * The reference's jagged x jagged kernels read both operands strided
 * (kernels/triton/triton_moe.py:1793-1976); here the reduction index is made contiguous once.
 *   src          [src_rows, cols], FMOE_BF16 or FMOE_F32, cols contiguous
 *   pad_offsets  [E+1], pad_offsets[e+1] - pad_offsets[e] >= len_e
 *   dst          [cols, dst_stride], columns [0, dst_cols) are written (dst_cols >= pad_offsets[E],
 *                a host-side bound; columns past pad_offsets[E] are zeroed)
 */
int fmoe_jagged_transpose(const void* src, int dtype, int64_t src_rows, int64_t cols,
                          int64_t src_stride_row, const int64_t* row_index, int index_div,
                          const int64_t* offsets, const int64_t* pad_offsets, int num_experts,
                          void* dst, int64_t dst_stride, int64_t dst_cols, int apply_silu,
                          fmoe_stream_t stream);

/*
 * out[e, c] = sum over r in [offsets[e], offsets[e+1]) of src[r, c], fp32 accumulation in a
 * fixed order: the bias gradient of the grouped GEMMs (torch autograd's sum over the rows of
 * each F.linear call in kernels/pytorch/moe.py:75-82).  src / out FMOE_BF16 or FMOE_F32.
 */
/*
 * dst[i, :] = src[index[i] / index_div, :]: the routed rows' inputs in expert order, what the
 * weight-gradient GEMM contracts with (triton_index_select, kernels/triton/triton_general_ops.py:42-129,
 * as called at kernels/triton/triton_moe.py:2451-2453).  Rows are row_bytes long (a multiple of
 * 16, any element type), pitches in bytes; an index outside [0, src_rows) is clamped.
 */
int fmoe_gather_rows(const void* src, int64_t src_rows, int64_t row_bytes, int64_t src_stride_bytes,
                     const int64_t* index, int index_div, int64_t n_out, void* dst,
                     int64_t dst_stride_bytes, fmoe_stream_t stream);

int fmoe_segment_colsum(const void* src, int dtype, int64_t total_rows, int64_t cols,
                        int64_t src_stride_row, const int64_t* offsets, int num_experts, void* out,
                        fmoe_stream_t stream);

/*
 * Element-wise backward of h = silu(g) * u (the SwiGLU epilogue; kernels/triton/triton_moe.py:62-141):
 *   du = dh * silu(g),   dg = (dh * u) * sigmoid(g) * (1 + g * (1 - sigmoid(g)))
 * rounded where torch autograd rounds (silu(g), dh * u and both results in `dtype`).
 * u == NULL: plain SiLU backward, dg = dh * sigmoid(g) * (1 + g * (1 - sigmoid(g))), du unused.
 * g, u, dh are contiguous with n elements.  out_stride_row = 0 (or = cols): so are dg and du.
 * Otherwise the n elements are rows of `cols`, and row i of dg / du starts at element
 * i * out_stride_row: the two halves of one [rows, 2 * cols] buffer (dg = buf, du = buf + cols,
 * pitch 2 * cols), which the next GEMMs then read as one operand (bf16, cols and the pitch in
 * multiples of 8).
 */
int fmoe_swiglu_bwd(const void* g, const void* u, const void* dh, void* dg, void* du, int dtype,
                    int64_t n, int64_t cols, int64_t out_stride_row, fmoe_stream_t stream);

/*
 * Backward of fmoe_combine (kernels/triton/triton_moe.py:922-983): for every routed row r with
 * t = token_index[r] and w(r) as in fmoe_combine,
 *   d_value[r, :]          = round(dy[t, :] * w(r))
 *   d_gates[flat(r)]       = sum_c round(value[r, c] * dy[t, c])      (fp32 sum; skipped if d_gates NULL)
 * flat(r) = gates_index ? gates_index[r] : r.  value / dy / d_value share value_dtype.
 */
int fmoe_combine_bwd(const void* dy, const void* value, int value_dtype, int64_t T, int K, int64_t D,
                     int64_t value_stride_row, const int64_t* token_index, const void* gates,
                     int gates_dtype, int64_t gates_cols, int64_t gates_stride_row,
                     int64_t gates_stride_col, const int64_t* gates_index, void* d_value,
                     float* d_gates, fmoe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FAST_MOE_AMD_H */
