// K3 for few rows (m <= 256): C[m][n] = sum_k A[m][k] * Bt[n][k] where reading Bt once from HBM is all the
// work there is (a decode step of an inference linear: A is a handful of tokens, Bt the weight).
//
// The 256 x 256 tile kernels would put n / 256 workgroups on 256 CUs and walk the whole k on each, which is
// 70 us for k = n = 8192 whatever m is.  Here a workgroup of eight waves owns 32 columns of C (two 16-row tiles
// of Bt) and all rows of A (of its block of A, past 64 rows); the waves split k among themselves, eight ways, and
// each streams its part of Bt straight from memory into MFMA operands: a lane's operand of
// v_mfma_f32_16x16x128_f8f6f4 is 32 consecutive k bytes of one row, two 16-byte loads, no LDS on the way.  With up
// to 32 rows of A four steps of 128 k are loaded back to back before the first is multiplied (16 loads of 16
// bytes per lane in flight for Bt alone), with more rows two or one.  The A fragments come the same
// way (A is small and stays in the L2).  At the end the eight partial sums meet in LDS, are added in a
// fixed order, scaled, biased, converted and stored.
//
// Operands are addressed as (row stride, stride of a 64-deep k block): row-major (ld, 64) or k-blocked
// (64, rows * 64).  Needs k % 128 == 0 and 16-byte aligned operands and strides; any n.  Up to 64 rows of A go
// through one workgroup per 32 columns in tiles of 16, 32 or 64 rows; more rows in blocks of 128 (second grid
// dimension: one pass over Bt per block, one step in flight per wave), which still beats the tile kernels'
// latency up to 256 rows (k-blocked operands; row-major ones break even there).
#include "f8mi_gemm_util.h"

namespace f8mi {

typedef float v4f_s __attribute__((ext_vector_type(4)));

constexpr int SK_WAVES = 8;
constexpr int SK_THREADS = SK_WAVES * 64;
constexpr int SK_NT = 2;     // 16-column tiles per workgroup
// 128-deep steps loaded before the first is multiplied: four where the A fragments leave registers for it
constexpr int sk_depth(int mt) { return mt <= 2 ? 4 : mt <= 4 ? 2 : 1; }

__device__ __forceinline__ v8i load_frag_global(const uint8_t* p) {
    const uint4 lo = *(const uint4*)p;
    const uint4 hi = *(const uint4*)(p + 16);
    return (v8i){(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
}

template <int AF, int BF, int C_DT, int MT>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(
    const uint8_t* __restrict__ A, int64_t lda, int64_t a_unit, const uint8_t* __restrict__ Bt, int64_t ldb, int64_t b_unit,
    int M_all, int N, int K, const float* __restrict__ sa_dev, const float* __restrict__ sb_dev, void* __restrict__ C_all,
    int64_t ldc, const void* __restrict__ bias) {
    constexpr int SK_DEPTH = sk_depth(MT);
    // blockIdx.y: which block of 16 * MT rows of A (and C) this workgroup multiplies
    // 1 / (sa * sb) for the epilogue: fetched first, so that the round trip to memory is over long before it is needed
    const float inv = __fdiv_rn(1.0f, *sa_dev) * __fdiv_rn(1.0f, *sb_dev);
    const int m_base = blockIdx.y * (16 * MT);
    const int M = min(M_all - m_base, 16 * MT);
    A += (int64_t)m_base * lda;
    void* C = (uint8_t*)C_all + (int64_t)m_base * ldc * (C_DT == F8MI_FP32 ? 4 : 2);
    __shared__ float4 part[SK_WAVES / 2][MT * SK_NT][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lm = lane & 15, lq = lane >> 4;
    const int n0 = blockIdx.x * (16 * SK_NT);
    const int steps = K / 128;
    const int s0 = steps * wave / SK_WAVES, s1 = steps * (wave + 1) / SK_WAVES;

    // a lane's 32 bytes of step s: row * ld + (2s + lq / 2) * unit + 32 * (lq % 2); rows past the end re-read the last one
    const uint8_t* pa[MT];
    const uint8_t* pb[SK_NT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) pa[mt] = A + (int64_t)min(mt * 16 + lm, M - 1) * lda + (lq >> 1) * a_unit + (lq & 1) * 32;
#pragma unroll
    for (int nt = 0; nt < SK_NT; nt++) pb[nt] = Bt + (int64_t)min(n0 + nt * 16 + lm, N - 1) * ldb + (lq >> 1) * b_unit + (lq & 1) * 32;

    v4f_s acc[MT][SK_NT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < SK_NT; nt++) acc[mt][nt] = (v4f_s){0.f, 0.f, 0.f, 0.f};

    for (int s = s0; s < s1; s += SK_DEPTH) {
        v8i fa[SK_DEPTH][MT], fb[SK_DEPTH][SK_NT];
#pragma unroll
        for (int d = 0; d < SK_DEPTH; d++) {
            const int sd = min(s + d, s1 - 1);  // past the wave's range: a valid address, the product is skipped
#pragma unroll
            for (int nt = 0; nt < SK_NT; nt++) fb[d][nt] = load_frag_global(pb[nt] + 2 * (int64_t)sd * b_unit);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) fa[d][mt] = load_frag_global(pa[mt] + 2 * (int64_t)sd * a_unit);
        }
#pragma unroll
        for (int d = 0; d < SK_DEPTH; d++) {
            if (s + d < s1) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int nt = 0; nt < SK_NT; nt++)
                        acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[d][nt], fa[d][mt], acc[mt][nt], BF, AF, 0, 0, 0, 0);
            }
        }
    }

    // the eight partial sums of every output meet in LDS: waves 4..7 hand theirs to waves 0..3, then the four
    // sums are added in a fixed order
    if (wave >= SK_WAVES / 2) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int nt = 0; nt < SK_NT; nt++)
                part[wave - SK_WAVES / 2][mt * SK_NT + nt][lane] = make_float4(acc[mt][nt][0], acc[mt][nt][1], acc[mt][nt][2], acc[mt][nt][3]);
    }
    __syncthreads();
    if (wave < SK_WAVES / 2) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int nt = 0; nt < SK_NT; nt++) {
                const float4 p = part[wave][mt * SK_NT + nt][lane];
                part[wave][mt * SK_NT + nt][lane] = make_float4(acc[mt][nt][0] + p.x, acc[mt][nt][1] + p.y, acc[mt][nt][2] + p.z, acc[mt][nt][3] + p.w);
            }
    }
    __syncthreads();

    for (int item = threadIdx.x; item < MT * SK_NT * 64; item += SK_THREADS) {
        const int tile = item >> 6, l = item & 63;
        float4 sum = part[0][tile][l];
#pragma unroll
        for (int w = 1; w < SK_WAVES / 2; w++) {
            const float4 p = part[w][tile][l];
            sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
        }
        // MFMA(first = Bt rows, second = A rows): lane l holds row l % 16 of A's tile and columns 4 * (l / 16) + e
        const int row = (tile / SK_NT) * 16 + (l & 15);
        const int col = n0 + (tile % SK_NT) * 16 + 4 * (l >> 4);
        if (row >= M || col >= N) continue;
        const float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (col + e >= N) break;
            const float r = v[e] * inv + (bias ? load_bias<C_DT>(bias, col + e) : 0.f);
            const int64_t at = (int64_t)row * ldc + col + e;
            if constexpr (C_DT == F8MI_FP32) ((float*)C)[at] = r;
            else ((uint16_t*)C)[at] = (uint16_t)(pack2<C_DT>(r, 0.f) & 0xffffu);
        }
    }
}

template <int AF, int BF, int C_DT>
static int launch_skinny3(dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt, int64_t ldb,
                          int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc,
                          const void* bias) {
    const dim3 b(SK_THREADS);
    if (M > 64) {  // blocks of 128 rows: Bt is read once per block (second grid dimension)
        g.y = (unsigned)((M + 127) / 128);
        hipLaunchKernelGGL((gemm_skinny_kernel<AF, BF, C_DT, 8>), g, b, 0, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
        return check_hip(hipGetLastError(), "skinny gemm kernel launch");
    }
    if (M <= 16) hipLaunchKernelGGL((gemm_skinny_kernel<AF, BF, C_DT, 1>), g, b, 0, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
    else if (M <= 32) hipLaunchKernelGGL((gemm_skinny_kernel<AF, BF, C_DT, 2>), g, b, 0, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
    else hipLaunchKernelGGL((gemm_skinny_kernel<AF, BF, C_DT, 4>), g, b, 0, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
    return check_hip(hipGetLastError(), "skinny gemm kernel launch");
}

template <int AF, int BF>
static int launch_skinny2(int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt,
                          int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc,
                          const void* bias) {
    if (c_dtype == F8MI_BF16) return launch_skinny3<AF, BF, F8MI_BF16>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
    if (c_dtype == F8MI_FP16) return launch_skinny3<AF, BF, F8MI_FP16>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
    return launch_skinny3<AF, BF, F8MI_FP32>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
}

// Host side has checked: 1 <= M <= SKINNY_MAX_M, K % 128 == 0, K >= 128, 16-byte aligned operands and strides.
int launch_gemm_skinny(int a_fmt, int b_fmt, int c_dtype, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                       const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C,
                       int64_t ldc, const void* bias) {
    const dim3 g((unsigned)((N + 16 * SK_NT - 1) / (16 * SK_NT)));
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E4M3FN) return launch_skinny2<0, 0>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
    if (a_fmt == F8MI_E5M2 && b_fmt == F8MI_E4M3FN) return launch_skinny2<1, 0>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E5M2) return launch_skinny2<0, 1>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
    return launch_skinny2<1, 1>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias);
}

}  // namespace f8mi
