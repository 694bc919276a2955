// OCP e4m3 instantiations of the jagged GEMM (v_mfma_scale_f32_32x32x64_f8f6f4, both
// operand formats = e4m3).  Row-wise scales the caller declares to be exact powers of
// two (fmoe_gemm_desc.scale_pow2) are applied by the MFMAs as E8M0 block scales on the
// ring and streaming kernels; any other scales are divided out in the epilogue.
#include "gemm_kernel.h"

namespace fmoe {

int run_gemm_fp8(GemmParams& p, int epilogue, int sel, hipStream_t stream) {
    switch (epilogue) {
        case FMOE_EPI_NONE: return dispatch_tile<kDtE4m3, FMOE_EPI_NONE, false>(p, sel, stream);
        case FMOE_EPI_SILU: return dispatch_tile<kDtE4m3, FMOE_EPI_SILU, false>(p, sel, stream);
        case FMOE_EPI_SWIGLU: return dispatch_tile<kDtE4m3, FMOE_EPI_SWIGLU, false>(p, sel, stream);
    }
    return fail(FMOE_ERR_ARGUMENT, "fmoe_grouped_gemm: unknown epilogue %d", epilogue);
}

}  // namespace fmoe
