// K3, fastest path: the LDS-DMA GEMM of f8mi_gemm_dma.hip on v_mfma_f32_16x16x128_f8f6f4.
//
// This GPU runs the fp8 matrix cores against its power limit, not its clock: on random
// data the 16x16x128 MFMA sustains about 18 % more flop/s than the 32x32x64 one (half
// the accumulator traffic per flop), so the same tile (256 x 256 per workgroup, 128 x 128
// per wave, 256 accumulator registers = 8 x 8 tiles of 16 x 16) is multiplied in steps of
// 128 k: 64 MFMAs per step and wave.
//
// LDS (160 KB) = five slabs of 32 KB, each one operand's 256 rows x 128 k of one step,
// stored as two halves of 256 rows x 64 B (the 64-deep units of the k-blocked / row-major
// DMA addressing, with the same 16-byte swizzle as f8mi_gemm_dma.hip).  Three slabs rotate
// through A, two through Bt:
//   * the eight Bt fragments of step t+1 are read into registers during the last quarter of
//     step t, so a Bt slab is free again at the step boundary;
//   * the A fragments are read one 8-MFMA group ahead, all through step t.
// Two barriers per step: Q (after 6 of 8 groups; before it a wave waits until its own DMAs
// of step t+1 have landed, after it everybody's have) and S (step boundary; everybody is done
// reading A of step t and Bt of step t+1; during step t+1 those two slabs are refilled with
// step t+3's A and Bt -- 16 DMAs per wave, issued one per four MFMAs through the step, 1 to
// 1.75 steps ahead of their first use).
// Requirements checked by the host: 16-byte aligned operands and strides, K % 128 == 0,
// K >= 384.
#include "f8mi_gemm_dma16_impl.h"

namespace f8mi {

int launch_gemm_dma16(int a_fmt, int b_fmt, int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                      const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb,
                      void* C, int64_t ldc, const void* bias, int tiles_m, int tiles_n, int c_vec_ok) {
    return launch_gemm_dma16_t<false, false>(a_fmt, b_fmt, c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc,
                                             bias, tiles_m, tiles_n, c_vec_ok);
}

}  // namespace f8mi
