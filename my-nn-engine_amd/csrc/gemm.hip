// DequantMatMul for M > 1: kernel choice of the reference (src/codegen/cuda.rs:1518-1652).
#include "mynn_common.h"

namespace mynn {
int dequant_gemv_dispatch(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N, int K,
                          int act_dtype, int out_dtype, hipStream_t s);
}

extern "C" int mynn_dequant_matmul(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N,
                                   int K, int act_dtype, int out_dtype, mynn_stream s) {
    using namespace mynn;
    MYNN_REQUIRE(M >= 1, MYNN_ERR_INVALID, "dequant_matmul: M=%d", M);
    const bool sixteen = act_dtype != MYNN_F32 && out_dtype != MYNN_F32;
    if (M >= 16 && sixteen && K % 8 == 0)
        return fail(MYNN_ERR_UNSUPPORTED, "dequant_matmul: matrix-core GEMM not built yet");
    return dequant_gemv_dispatch(out, act, wq, scale, M, N, K, act_dtype, out_dtype, as_stream(s));
}

namespace mynn {
int dequant_gemm_mfma(void *, const void *, const int8_t *, const void *, int, int, int, int, hipStream_t) {
    return fail(MYNN_ERR_UNSUPPORTED, "dequant_matmul: matrix-core GEMM not built yet");
}
}  // namespace mynn
