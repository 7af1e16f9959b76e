// K3: scaled fp8 GEMM  C[m][n] = (sum_k A[m][k] * Bt[n][k]) / (sa * sb)  on the
// gfx950 matrix cores (v_mfma_f32_32x32x64_f8f6f4, fp32 accumulate), MFMA-bound.
//
// Workgroup = 256 lanes (4 waves, 2 x 2), macro tile 256 x 256, K step 128 bytes.
// Each wave owns 128 x 128 of C = 4 x 4 MFMA tiles of 32 x 32 (256 accumulator
// registers).  Operand tiles are staged HBM -> registers -> LDS (two stages, 64 KB
// each) as 16-byte pieces; piece c of tile row r lives at r*128 + ((c ^ (r & 7)) * 16),
// which makes both the 16-byte LDS writes and the per-lane 2 x 16-byte fragment
// reads (lane = tile row, 32 consecutive k per lane) bank-conflict free.
// Workgroup ids are first re-dealt so that each of the 8 XCDs (which receive
// consecutive ids round-robin) works on one contiguous band of tiles, then
// walked in groups of 8 tile rows so the tiles in flight share A and B panels
// in that XCD's L2.
#include "f8mi_common.h"

namespace f8mi {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int GEMM_THREADS = 256;
constexpr int STAGE_BYTES = (BM + BN) * BK;  // 64 KB
constexpr int GEMM_LDS = 2 * STAGE_BYTES;    // 128 KB
constexpr int GROUP_M = 8;
constexpr int NUM_XCD = 8;

// 16 bytes of one operand row; bytes at k >= klimit read as zero.
template <bool ALIGNED, bool GUARD>
__device__ __forceinline__ uint4 load_piece(const uint8_t* __restrict__ p, int valid) {
    if (!GUARD) {
        if (ALIGNED) return *(const uint4*)p;
        uint4 v;
        __builtin_memcpy(&v, p, 16);
        return v;
    }
    uint4 v = make_uint4(0, 0, 0, 0);
    if (valid >= 16) {
        if (ALIGNED) v = *(const uint4*)p;
        else __builtin_memcpy(&v, p, 16);
    } else if (valid > 0) {
        uint32_t w[4] = {0, 0, 0, 0};
        for (int i = 0; i < valid; i++) w[i >> 2] |= (uint32_t)p[i] << (8 * (i & 3));
        v = make_uint4(w[0], w[1], w[2], w[3]);
    }
    return v;
}

template <int AF, int BF, bool ALIGNED>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_nt_kernel(
    const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ Bt, int64_t ldb, int M, int N, int K,
    const float* __restrict__ sa_dev, const float* __restrict__ sb_dev, void* __restrict__ C, int c_dtype,
    int64_t ldc, const void* __restrict__ bias, int tiles_m, int tiles_n) {
    extern __shared__ __align__(16) uint8_t smem[];

    // ---- which tile
    int lid = blockIdx.x;
    const int npid = gridDim.x;
    if (npid % NUM_XCD == 0) lid = (lid % NUM_XCD) * (npid / NUM_XCD) + lid / NUM_XCD;
    const int width = GROUP_M * tiles_n;
    const int group = lid / width;
    const int first_m = group * GROUP_M;
    const int gsz = min(tiles_m - first_m, GROUP_M);
    const int tm = first_m + (lid % width) % gsz;
    const int tn = (lid % width) / gsz;
    const int m0 = tm * BM, n0 = tn * BN;

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- global -> register staging: piece (row = i*32 + t/8, c = t%8), i = 0..7, per operand
    const int lrow = t >> 3, lc = t & 7;
    const uint8_t* a_base = A + (int64_t)m0 * lda;
    const uint8_t* b_base = Bt + (int64_t)n0 * ldb;
    uint32_t a_off[8], b_off[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int r = i * 32 + lrow;
        a_off[i] = (uint32_t)(min(r, M - 1 - m0) * lda) + lc * 16;  // rows past the edge re-read the last row
        b_off[i] = (uint32_t)(min(r, N - 1 - n0) * ldb) + lc * 16;
    }
    const int st_off = lrow * BK + ((lc ^ (lrow & 7)) << 4);  // + i*32*BK

    const int nk_full = K / BK;
    const int nk = (K + BK - 1) / BK;

    uint4 ra[8], rb[8];
    auto gload = [&](int kb) {
        const int k0 = kb * BK;
        if (ALIGNED && kb < nk_full) {
#pragma unroll
            for (int i = 0; i < 8; i++) ra[i] = load_piece<ALIGNED, false>(a_base + a_off[i] + k0, 16);
#pragma unroll
            for (int i = 0; i < 8; i++) rb[i] = load_piece<ALIGNED, false>(b_base + b_off[i] + k0, 16);
        } else {
            const int valid = K - k0 - lc * 16;
#pragma unroll
            for (int i = 0; i < 8; i++) ra[i] = load_piece<ALIGNED, true>(a_base + a_off[i] + k0, valid);
#pragma unroll
            for (int i = 0; i < 8; i++) rb[i] = load_piece<ALIGNED, true>(b_base + b_off[i] + k0, valid);
        }
    };
    auto lstore = [&](int stage) {
        uint8_t* as = smem + stage * STAGE_BYTES;
        uint8_t* bs = as + BM * BK;
#pragma unroll
        for (int i = 0; i < 8; i++) *(uint4*)(as + st_off + i * 32 * BK) = ra[i];
#pragma unroll
        for (int i = 0; i < 8; i++) *(uint4*)(bs + st_off + i * 32 * BK) = rb[i];
    };

    // ---- fragment addressing: lane -> tile row (lane % 32), k half (lane / 32)
    const int frow = lane & 31, fh = lane >> 5;
    const int fsw = frow & 7;
    int f_off[2][2];  // [ks][j]: byte offset of piece (ks*4 + fh*2 + j) of row frow
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int j = 0; j < 2; j++) f_off[ks][j] = frow * BK + (((ks * 4 + fh * 2 + j) ^ fsw) << 4);
    const int a_frag_base = (wm * 128) * BK;
    const int b_frag_base = BM * BK + (wn * 128) * BK;

    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    if (nk > 0) {
        gload(0);
        lstore(0);
        if (nk > 1) gload(1);
    }
    __syncthreads();

    for (int kb = 0; kb < nk; kb++) {
        const uint8_t* st = smem + (kb & 1) * STAGE_BYTES;
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            v8i af[4], bf[4];
#pragma unroll
            for (int ti = 0; ti < 4; ti++) {
                const uint4 lo = *(const uint4*)(st + a_frag_base + ti * 32 * BK + f_off[ks][0]);
                const uint4 hi = *(const uint4*)(st + a_frag_base + ti * 32 * BK + f_off[ks][1]);
                af[ti] = (v8i){(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            }
#pragma unroll
            for (int tj = 0; tj < 4; tj++) {
                const uint4 lo = *(const uint4*)(st + b_frag_base + tj * 32 * BK + f_off[ks][0]);
                const uint4 hi = *(const uint4*)(st + b_frag_base + tj * 32 * BK + f_off[ks][1]);
                bf[tj] = (v8i){(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            }
#pragma unroll
            for (int ti = 0; ti < 4; ti++)
#pragma unroll
                for (int tj = 0; tj < 4; tj++)
                    acc[ti][tj] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[ti], bf[tj], acc[ti][tj], AF, BF,
                                                                                 0, 0, 0, 0);
        }
        if (kb + 1 < nk) {
            lstore((kb + 1) & 1);
            if (kb + 2 < nk) gload(kb + 2);
        }
        __syncthreads();
    }

    // ---- epilogue: scale, (+bias), convert, store.  acc[ti][tj][e] of lane l is
    // C[row = 8*(e/4) + 4*(l/32) + e%4][col = l%32] of its 32 x 32 tile.
    const float inv = __fdiv_rn(1.0f, *sa_dev) * __fdiv_rn(1.0f, *sb_dev);
#pragma unroll
    for (int tj = 0; tj < 4; tj++) {
        const int col = n0 + wn * 128 + tj * 32 + (lane & 31);
        if (col >= N) continue;
        float bv = 0.0f;
        if (bias) {
            if (c_dtype == F8MI_BF16) bv = bf16_bits_to_float(((const uint16_t*)bias)[col]);
            else if (c_dtype == F8MI_FP16) bv = fp16_bits_to_float(((const uint16_t*)bias)[col]);
            else bv = ((const float*)bias)[col];
        }
#pragma unroll
        for (int ti = 0; ti < 4; ti++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int row = m0 + wm * 128 + ti * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (row >= M) continue;
                const float v = acc[ti][tj][e] * inv + bv;
                const int64_t idx = (int64_t)row * ldc + col;
                if (c_dtype == F8MI_BF16) ((uint16_t*)C)[idx] = (uint16_t)float_to_bf16_bits(v);
                else if (c_dtype == F8MI_FP16) ((__half*)C)[idx] = __float2half_rn(v);
                else ((float*)C)[idx] = v;
            }
        }
    }
}

template <int AF, int BF>
static int launch_gemm(bool aligned, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, const uint8_t* Bt,
                       int64_t ldb, int M, int N, int K, const float* sa, const float* sb, void* C, int c_dtype,
                       int64_t ldc, const void* bias, int tiles_m, int tiles_n) {
    static bool attr_done[2] = {false, false};
    auto ka = gemm_nt_kernel<AF, BF, true>;
    auto ku = gemm_nt_kernel<AF, BF, false>;
    if (!attr_done[aligned ? 1 : 0]) {
        hipError_t e = hipFuncSetAttribute(aligned ? (const void*)ka : (const void*)ku,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS);
        if (e != hipSuccess) return check_hip(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
        attr_done[aligned ? 1 : 0] = true;
    }
    if (aligned) hipLaunchKernelGGL(ka, g, dim3(GEMM_THREADS), GEMM_LDS, stream, A, lda, Bt, ldb, M, N, K, sa, sb, C, c_dtype, ldc, bias, tiles_m, tiles_n);
    else hipLaunchKernelGGL(ku, g, dim3(GEMM_THREADS), GEMM_LDS, stream, A, lda, Bt, ldb, M, N, K, sa, sb, C, c_dtype, ldc, bias, tiles_m, tiles_n);
    return check_hip(hipGetLastError(), "gemm kernel launch");
}

}  // namespace f8mi

using namespace f8mi;

extern "C" int f8mi_gemm_nt(const void* a, int a_fmt, int64_t lda, const void* bt, int b_fmt, int64_t ldb, int64_t m,
                            int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c,
                            int c_dtype, int64_t ldc, const void* bias_dev, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (m < 0 || n < 0 || k < 0 || lda < k || ldb < k || ldc < n) { set_error("f8mi_gemm_nt: bad shape m=%lld n=%lld k=%lld lda=%lld ldb=%lld ldc=%lld", (long long)m, (long long)n, (long long)k, (long long)lda, (long long)ldb, (long long)ldc); return F8MI_ERR_INVALID_ARG; }
    if (a_fmt < 0 || a_fmt > 1 || b_fmt < 0 || b_fmt > 1 || c_dtype < 0 || c_dtype > 2) { set_error("f8mi_gemm_nt: unknown format/dtype code"); return F8MI_ERR_INVALID_ARG; }
    if (m == 0 || n == 0) return F8MI_OK;
    if (!c || !scale_a_dev || !scale_b_dev || (k > 0 && (!a || !bt))) { set_error("f8mi_gemm_nt: null pointer"); return F8MI_ERR_INVALID_ARG; }
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff - BK) { set_error("f8mi_gemm_nt: dimension over 2^31"); return F8MI_ERR_UNSUPPORTED; }
    // the kernel addresses rows inside a tile with 32-bit offsets
    if (lda * (BM - 1) + k + BK > 0x7fffffffLL || ldb * (BN - 1) + k + BK > 0x7fffffffLL) { set_error("f8mi_gemm_nt: row stride too large (lda=%lld ldb=%lld)", (long long)lda, (long long)ldb); return F8MI_ERR_UNSUPPORTED; }
    const int64_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7fffffff) { set_error("f8mi_gemm_nt: too many tiles"); return F8MI_ERR_UNSUPPORTED; }
    const bool aligned = ((uintptr_t)a % 16 == 0) && ((uintptr_t)bt % 16 == 0) && (lda % 16 == 0) && (ldb % 16 == 0);
    dim3 g((unsigned)(tiles_m * tiles_n));
    ProfScope prof(F8MI_K_GEMM, 2.0 * (double)m * (double)n * (double)k, stream);
    const uint8_t* A = (const uint8_t*)a;
    const uint8_t* B = (const uint8_t*)bt;
    const int M = (int)m, N = (int)n, K = (int)k;
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E4M3FN) return launch_gemm<0, 0>(aligned, g, stream, A, lda, B, ldb, M, N, K, scale_a_dev, scale_b_dev, c, c_dtype, ldc, bias_dev, (int)tiles_m, (int)tiles_n);
    if (a_fmt == F8MI_E5M2 && b_fmt == F8MI_E4M3FN) return launch_gemm<1, 0>(aligned, g, stream, A, lda, B, ldb, M, N, K, scale_a_dev, scale_b_dev, c, c_dtype, ldc, bias_dev, (int)tiles_m, (int)tiles_n);
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E5M2) return launch_gemm<0, 1>(aligned, g, stream, A, lda, B, ldb, M, N, K, scale_a_dev, scale_b_dev, c, c_dtype, ldc, bias_dev, (int)tiles_m, (int)tiles_n);
    return launch_gemm<1, 1>(aligned, g, stream, A, lda, B, ldb, M, N, K, scale_a_dev, scale_b_dev, c, c_dtype, ldc, bias_dev, (int)tiles_m, (int)tiles_n);
}
