// bf16 instantiations of the jagged GEMM (v_mfma_f32_32x32x16_bf16).
#include "gemm_kernel.h"

namespace fmoe {

int run_gemm_bf16(GemmParams& p, int epilogue, bool a_silu, int sel, hipStream_t stream) {
    if (a_silu) {
        if (epilogue != FMOE_EPI_NONE)
            return fail(FMOE_ERR_UNSUPPORTED, "fmoe_grouped_gemm: a_silu is only built for the plain epilogue");
        return dispatch_tile<kDtBf16, FMOE_EPI_NONE, true>(p, sel, stream);
    }
    switch (epilogue) {
        case FMOE_EPI_NONE: return dispatch_tile<kDtBf16, FMOE_EPI_NONE, false>(p, sel, stream);
        case FMOE_EPI_SILU: return dispatch_tile<kDtBf16, FMOE_EPI_SILU, false>(p, sel, stream);
        case FMOE_EPI_SWIGLU: return dispatch_tile<kDtBf16, FMOE_EPI_SWIGLU, false>(p, sel, stream);
        case FMOE_EPI_GATED: return dispatch_tile<kDtBf16, FMOE_EPI_GATED, false>(p, sel, stream);
    }
    return fail(FMOE_ERR_ARGUMENT, "fmoe_grouped_gemm: unknown epilogue %d", epilogue);
}

}  // namespace fmoe
