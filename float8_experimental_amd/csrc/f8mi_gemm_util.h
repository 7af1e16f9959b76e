// Pieces shared by the two fp8 GEMM kernels (register-staged and LDS-DMA): tile constants,
// fragment reads, output conversion and the C epilogue.
#pragma once
#include <atomic>
#include <type_traits>

#include "f8mi_common.h"

namespace f8mi {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int GEMM_THREADS = 256;
constexpr int STAGE_BYTES = (BM + BN) * BK;  // 64 KB
constexpr int EPI_PITCH = 128 * 2 + 16;      // bytes per row of a wave's 128 x 128 2-byte output tile in LDS
constexpr int EPI_BYTES = 4 * 128 * EPI_PITCH;
constexpr int GEMM_LDS = 2 * STAGE_BYTES > EPI_BYTES ? 2 * STAGE_BYTES : EPI_BYTES;
constexpr int GROUP_M = 8;
constexpr int NUM_XCD = 8;

// Consecutive workgroup ids go to the 8 XCDs round-robin.  Re-deals them so that XCD x (ids x, x+8, ...) works on
// a contiguous run of the tile order -- whatever the grid size: the first `grid % 8` XCDs get one workgroup more.
__device__ __forceinline__ int xcd_contiguous_id(int bid, int grid) {
    const int x = bid % NUM_XCD, q = grid / NUM_XCD, r = grid % NUM_XCD;
    return x * q + min(x, r) + bid / NUM_XCD;
}

#define F8MI_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

__device__ __forceinline__ v8i read_frag(const uint8_t* p0, const uint8_t* p1) {
    const uint4 lo = *(const uint4*)p0;
    const uint4 hi = *(const uint4*)p1;
    return (v8i){(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
}

template <int C_DT>
__device__ __forceinline__ float load_bias(const void* bias, int col) {
    if constexpr (C_DT == F8MI_BF16) return bf16_bits_to_float(((const uint16_t*)bias)[col]);
    else if constexpr (C_DT == F8MI_FP16) return fp16_bits_to_float(((const uint16_t*)bias)[col]);
    else return ((const float*)bias)[col];
}

// two fp32 -> two packed 2-byte outputs (round to nearest even)
template <int C_DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    if constexpr (C_DT == F8MI_BF16) {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        typedef float f2 __attribute__((ext_vector_type(2)));
        bf2 r = __builtin_convertvector((f2){a, b}, bf2);
        return __builtin_bit_cast(uint32_t, r);
    } else {
        return (uint32_t)__half_as_ushort(__float2half_rn(a)) | ((uint32_t)__half_as_ushort(__float2half_rn(b)) << 16);
    }
}

// Scales a workgroup's 256 x 256 accumulators by 1 / (sa * sb), adds the bias, converts and writes C.
// acc[tj][ti] is the 32 x 32 tile (row block ti, column block tj) of this wave's 128 x 128 quarter
// as left by MFMA(first = Bt rows, second = A rows): lane holds row lane%32 and columns
// 8*(e/4) + 4*(lane/32) + e%4.  2-byte outputs go through a padded LDS tile per wave so that C is
// written with 16-byte stores; `smem` must be free for that (EPI_BYTES) when every wave arrives.
template <int C_DT>
__device__ __forceinline__ void store_c_tile(v16f (&acc)[4][4], uint8_t* smem, int m0, int n0, int M, int N,
                                             const float* __restrict__ sa_dev, const float* __restrict__ sb_dev,
                                             void* __restrict__ C, int64_t ldc, const void* __restrict__ bias,
                                             int c_vec_ok) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const float inv = __fdiv_rn(1.0f, *sa_dev) * __fdiv_rn(1.0f, *sb_dev);
    const int lm = lane & 31, lh = lane >> 5;
    const int wrow0 = m0 + wm * 128, wcol0 = n0 + wn * 128;

    if constexpr (C_DT == F8MI_FP32) {
        // 4 consecutive columns per lane = one 16-byte store
        float* Cf = (float*)C;
#pragma unroll
        for (int ti = 0; ti < 4; ti++) {
            const int row = wrow0 + ti * 32 + lm;
#pragma unroll
            for (int tj = 0; tj < 4; tj++) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int col = wcol0 + tj * 32 + 8 * g + 4 * lh;
                    if (row >= M || col >= N) continue;
                    float v[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        v[r] = acc[tj][ti][4 * g + r] * inv;
                        if (bias && col + r < N) v[r] += load_bias<C_DT>(bias, col + r);
                    }
                    float* dst = Cf + (int64_t)row * ldc + col;
                    if (c_vec_ok && col + 4 <= N) {
                        store16_any(dst, make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])));
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (col + r < N) dst[r] = v[r];
                    }
                }
            }
        }
    } else {
        // all waves are done with the operand stages before they become the output staging area
        lds_barrier();
        uint8_t* ep = smem + wave * (128 * EPI_PITCH);
#pragma unroll
        for (int tj = 0; tj < 4; tj++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int cl = tj * 32 + 8 * g + 4 * lh;  // column inside the wave's 128
                float bv[4] = {0.f, 0.f, 0.f, 0.f};
                if (bias) {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (wcol0 + cl + r < N) bv[r] = load_bias<C_DT>(bias, wcol0 + cl + r);
                }
#pragma unroll
                for (int ti = 0; ti < 4; ti++) {
                    const float v0 = acc[tj][ti][4 * g + 0] * inv + bv[0];
                    const float v1 = acc[tj][ti][4 * g + 1] * inv + bv[1];
                    const float v2 = acc[tj][ti][4 * g + 2] * inv + bv[2];
                    const float v3 = acc[tj][ti][4 * g + 3] * inv + bv[3];
                    *(uint2*)(ep + (ti * 32 + lm) * EPI_PITCH + cl * 2) = make_uint2(pack2<C_DT>(v0, v1), pack2<C_DT>(v2, v3));
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own wave's tile only: no workgroup barrier needed
        uint16_t* Ch = (uint16_t*)C;
        const int chunk = lane & 15, rsub = lane >> 4;
        const int col = wcol0 + chunk * 8;
#pragma unroll 4
        for (int it = 0; it < 32; it++) {
            const int rl = it * 4 + rsub;
            const int row = wrow0 + rl;
            const uint4 v = *(const uint4*)(ep + rl * EPI_PITCH + chunk * 16);
            if (row < M && col < N) {
                uint16_t* dst = Ch + (int64_t)row * ldc + col;
                if (c_vec_ok && col + 8 <= N) {
                    store16_any(dst, v);
                } else {
                    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int i = 0; i < 8; i++)
                        if (col + i < N) dst[i] = (uint16_t)((w[i >> 1] >> (16 * (i & 1))) & 0xffffu);
                }
            }
        }
    }
}

// Raises a kernel's dynamic LDS limit once per device (the attribute is per device, calls may come from any
// host thread: a repeated call is harmless, a missing one is not).
template <typename K>
static int allow_big_lds(K kern, int bytes, std::atomic<uint64_t>& done_mask) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return check_hip(e, "hipGetDevice");
    const uint64_t bit = 1ull << (dev & 63);
    if (done_mask.load(std::memory_order_acquire) & bit) return 0;
    e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return check_hip(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    done_mask.fetch_or(bit, std::memory_order_release);
    return 0;
}

// The 16x16x128 kernel with Bt (nt) or both operands (tt) given transposed: memory holds [contraction][rows];
// lda / ldb = bytes between contraction rows, a_unit / b_unit = bytes between blocks of 64 rows.
// 128-row-tile kernels (f8mi_gemm_mid.hip) for outputs of few 256 x 256 tiles: K % 128 == 0, aligned operands.
// wide = false: 128 x 128 tiles, true: 128 x 256.
int launch_gemm_mid(int a_fmt, int b_fmt, int c_dtype, bool wide, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                    const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C,
                    int64_t ldc, const void* bias, int c_vec_ok);
// They take over while their own tiles number at most one per CU (with more, the large tiles win again: measured):
// 128 x 128 tiles while at most 256 of them cover the output, else 128 x 256 tiles while 256 of those do.
// Returns 0: large tiles, 1: 128 x 128, 2: 128 x 256.
inline int use_mid_tiles(int64_t m, int64_t n, int64_t k) {
    if (k % 128 != 0 || k < 128) return 0;
    const int64_t row_tiles = (m + 127) / 128;
    if (row_tiles * ((n + 127) / 128) <= 256) return 1;
    if (row_tiles * ((n + 255) / 256) <= 256) return 2;
    return 0;
}
// few-row kernel (f8mi_gemm_skinny.hip): m <= SKINNY_MAX_M, K % 128 == 0, aligned operands.
constexpr int SKINNY_MAX_M = 256;
// Time estimates in us behind the choice between the few-row kernel, a round of 128-row tiles, and the same tiles
// with k split over workgroups -- fitted to measurements (rows, n x k: few-row / tiles): 128, 8192 x 8192: 27 / 37;
// 128, 28672 x 8192: 83 / 37; 64, 28672 x 8192: 53 / 37; 64, 4096 x 14336: 27 / 63; 144 - 256, 4096 x 4096: 14 / 20;
// 4096 x 14336: 36 / 60; 8192 x 8192: 41 - 48 / 37; 14336 x 4096: 39 - 47 / 22; 28672 x 8192: 119 - 143 / 59.
// They depend on the shape only, so the row-major and the k-blocked entry point decide alike.
//
// Few-row kernel: Bt at 6.5 TB/s from memory plus A (n / 32 workgroups x 16 row_tiles x k bytes) at 20 TB/s from L2,
// once per 128 rows; slower when its n / 32 workgroups per pass leave CUs idle.
inline double skinny_time_us(int64_t m, int64_t n, int64_t k) {
    const double passes = (double)((m + 127) / 128);
    const double row_tiles = m > 128 ? 8.0 : (double)((m + 15) / 16);  // 16-row tiles of A per pass
    const double wgs = passes * (double)((n + 31) / 32);
    const double idle = wgs < 256.0 ? __builtin_sqrt(256.0 / wgs) : 1.0;
    return passes * (2.0 + (double)n * (double)k * (0.154 + 0.025 * row_tiles) * 1e-6 * idle);
}
// Tiles: a round of 128 x 128 tiles takes 4.4 ns per unit of k, of 128 x 256 tiles 7.8 ns, of 256 x 256 tiles 10.6 ns,
// for 1 row or 128.
inline double tiles_time_us(int64_t m, int64_t n, int64_t k) {
    const int64_t rt = (m + 127) / 128;
    if (rt * ((n + 127) / 128) <= 256) return 4.4e-3 * (double)k;
    if (rt * ((n + 255) / 256) <= 256) return 7.8e-3 * (double)k;
    return 10.6e-3 * (double)k * (double)((((m + 255) / 256) * ((n + 255) / 256) + 255) / 256);
}
// Up to 16 rows the few-row kernel always runs: it streams Bt once at memory speed.
inline bool use_skinny(int64_t m, int64_t n, int64_t k) {
    if (m > SKINNY_MAX_M || k <= 0 || k % 128 != 0) return false;
    if (m <= 16) return true;
    return skinny_time_us(m, n, k) <= tiles_time_us(m, n, k);
}
// An output of at most 128 of the 128-row tiles and a long k: with `ws_bytes` of scratch for the partial sums, k is
// split 2, 4 or 8 ways so that (nearly) every CU gets a part, and a second kernel adds the parts in a fixed order.
// Returns the number of parts, 0 for no split.  Cost of the split: the parts written and read once (5 TB/s) and a launch.
inline int pick_k_splits(int64_t m, int64_t n, int64_t k, int64_t ws_bytes) {
    const int mode = use_mid_tiles(m, n, k);
    if (!mode || n % 4 != 0 || m <= 16 || ws_bytes <= 0) return 0;
    const int64_t tiles = ((m + 127) / 128) * ((n + (mode == 1 ? 127 : 255)) / (mode == 1 ? 128 : 256));
    if (tiles > 128) return 0;
    const double t_round = (mode == 1 ? 4.4e-3 : 7.8e-3) * (double)k;
    const double t_skinny = m <= SKINNY_MAX_M ? skinny_time_us(m, n, k) : 1e30;
    const double t_other = t_skinny < t_round ? t_skinny : t_round;
    int best = 0;
    double t_best = 0.9 * t_other;  // the estimates are not better than that
    for (int s = 2; s <= 8; s *= 2) {
        if (tiles * s > 256 || k % (128 * s) != 0 || k / s < 1024 || (int64_t)s * m * n * 4 > ws_bytes) break;
        const double t = t_round / s + 3.0 + (double)s * (double)m * (double)n * 8.0 / 5e6 + 4.0;
        if (t < t_best) { t_best = t; best = s; }
    }
    return best;
}
int launch_gemm_mid_splitk(int a_fmt, int b_fmt, int c_dtype, bool wide, int k_splits, float* partial, hipStream_t stream, const uint8_t* A,
                           int64_t lda, int64_t a_unit, const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa,
                           const float* sb, void* C, int64_t ldc, const void* bias, int c_vec_ok);
int launch_gemm_skinny(int a_fmt, int b_fmt, int c_dtype, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                       const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C,
                       int64_t ldc, const void* bias);
int launch_gemm_dma16_nt(int a_fmt, int b_fmt, int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                         const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb,
                         void* C, int64_t ldc, const void* bias, int tiles_m, int tiles_n, int c_vec_ok);
int launch_gemm_dma16_tt(int a_fmt, int b_fmt, int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                         const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb,
                         void* C, int64_t ldc, const void* bias, int tiles_m, int tiles_n, int c_vec_ok);

// LDS-DMA kernel (f8mi_gemm_dma.hip).  Needs 16-byte aligned operands and strides and K % 64 == 0, K >= 384.
// lda / ldb: bytes between operand rows, a_unit / b_unit: bytes between 64-deep units of one row
// (row-major: (row stride, 64); k-blocked [K/64][rows][64]: (64, rows * 64)).
int launch_gemm_dma(int a_fmt, int b_fmt, int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                    const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb,
                    void* C, int64_t ldc, const void* bias, int tiles_m, int tiles_n, int c_vec_ok);
// The same on the 16x16x128 MFMA (f8mi_gemm_dma16.hip); additionally needs K % 128 == 0.
int launch_gemm_dma16(int a_fmt, int b_fmt, int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                      const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb,
                      void* C, int64_t ldc, const void* bias, int tiles_m, int tiles_n, int c_vec_ok);

}  // namespace f8mi
