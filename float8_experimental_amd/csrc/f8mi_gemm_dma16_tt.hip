// The 16x16x128 LDS-DMA GEMM with both operands given transposed (grad_weight: dY^T x with dY and x as the other GEMMs hold them).
#include "f8mi_gemm_dma16_impl.h"

namespace f8mi {

int launch_gemm_dma16_tt(int a_fmt, int b_fmt, int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                         const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb,
                         void* C, int64_t ldc, const void* bias, int tiles_m, int tiles_n, int c_vec_ok) {
    return launch_gemm_dma16_t<true, true>(a_fmt, b_fmt, c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C,
                                             ldc, bias, tiles_m, tiles_n, c_vec_ok);
}

}  // namespace f8mi
