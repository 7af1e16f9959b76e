// K3 for outputs of few 256 x 256 tiles: the same 16x16x128 MFMA, LDS-DMA and LDS layout as
// f8mi_gemm_dma16_impl.h on tiles of 128 rows, so that two or four times as many workgroups share the CUs.
//
// The large-tile kernel is built for the regime where every CU has tiles queued: one workgroup owns a CU
// (160 KB of LDS, 512 registers per lane) and walks all of k in 1.1 us steps -- 70 us for k = 8192 however
// few tiles there are.  With 512 rows and 8192 columns that is 64 workgroups on 256 CUs.  Here a workgroup
// (4 waves as 2 x 2) takes a tile of 128 x 128 (64 x 64 per wave, 16 accumulator tiles, four LDS stages of
// (128 + 128 rows) x 128 k) or 128 x 256 (64 x 128 per wave, three stages of (128 + 256 rows) x 128 k): 256
// workgroups for that output with the former, and one round of workgroups instead of two for outputs of 65 to 128
// large tiles with the latter.  The DMAs of the step NSTAGE-1 ahead are issued during a step, one after every
// second MFMA (a step is 0.4 - 0.7 us, less than the latency of a DMA); the rest of the schedule is left to the
// compiler: per step and wave a wait for the current step's DMAs, the fragment reads, 16 or 32 MFMAs, two barriers.
//
// A wave's accumulation order over k is that of the large-tile kernels (128-deep steps in sequence, the same
// 32 contraction bytes per lane), so the results are the same bits.
// Host side guarantees: K % 128 == 0, K >= 128, 16-byte aligned operands and strides.
#include "f8mi_gemm_util.h"

namespace f8mi {

typedef float v4f_m __attribute__((ext_vector_type(4)));

constexpr int MID_TILE_M = 128;
constexpr int MID_A_UNIT = MID_TILE_M * 64;  // A, one 64-deep unit of a stage: 8 KB

// TJ = 16-column tiles per wave: 4 -> 128 x 128 workgroup tiles, four stages of 32 KB;
//                                8 -> 128 x 256, three stages of 48 KB.
template <int TJ>
struct MidCfg {
    static constexpr int TILE_N = 32 * TJ;
    static constexpr int B_UNIT = TILE_N * 64;
    static constexpr int STAGE = 2 * MID_A_UNIT + 2 * B_UNIT;
    static constexpr int NSTAGE = TJ == 4 ? 4 : 3;
    static constexpr int LDS = NSTAGE * STAGE;  // 128 KB / 144 KB
    static constexpr int BI = TJ / 2;           // Bt row groups (16 rows) per wave and unit
    static constexpr int NDMA = 4 + 2 * BI;     // DMAs per wave and step
};

__device__ __forceinline__ void dma_mid(const uint8_t* base, uint32_t voff, uint32_t lds_addr) {
    // M0 carries the LDS address; one wait state between the scalar write of M0 and its use
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds_addr) : "memory");
}

template <int AF, int BF, int C_DT, int TJ>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_mid_kernel(
    const uint8_t* __restrict__ A, int64_t lda, int64_t a_unit, const uint8_t* __restrict__ Bt, int64_t ldb, int64_t b_unit,
    int M, int N, int K, const float* __restrict__ sa_dev, const float* __restrict__ sb_dev, void* __restrict__ C,
    int64_t ldc, const void* __restrict__ bias, int tiles_m, int c_vec_ok, int k_splits) {
    using Cfg = MidCfg<TJ>;
    extern __shared__ __align__(16) uint8_t smem[];
    // consecutive workgroup ids go to the 8 XCDs round-robin; re-deal them so that one XCD (one L2) gets a
    // contiguous run of the tile order (rows fastest): the workgroups that share a block of Bt sit behind the same L2
    int lid = blockIdx.x;
    lid = xcd_contiguous_id(lid, gridDim.x);
    const int tm = lid % tiles_m, tn = lid / tiles_m;
    const int m0 = tm * MID_TILE_M, n0 = tn * Cfg::TILE_N;
    // 1 / (sa * sb) for the epilogue, fetched before the main loop and kept in a scalar register
    // k_splits > 1 (host: fp32 output, no bias): blockIdx.y takes the y-th part of k and writes its partial sums,
    // unscaled, to the y-th M x ldc slab of C; a second kernel adds the slabs in a fixed order.
    const int split = blockIdx.y;
    const int K_part = K / k_splits;
    const float inv = k_splits > 1 ? 1.0f : __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(
        int, __fdiv_rn(1.0f, *sa_dev) * __fdiv_rn(1.0f, *sb_dev))));
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- DMA: one instruction = 16 rows x 64 B of one unit, landing as 1 KB of consecutive LDS; lane l fetches
    // row l/4 of the sixteen, piece (l%4) ^ (l/32) (the slot swizzle, applied on the global side).  Wave w
    // brings row groups 2w, 2w+1 of both units of A and BI*w .. BI*w+BI-1 of both units of Bt.
    const uint32_t lds_u32 = (uint32_t)(uintptr_t)smem;
    uint32_t a_voff[2], b_voff[Cfg::BI];
    const uint32_t piece = (uint32_t)(((lane & 3) ^ (lane >> 5)) << 4);
#pragma unroll
    for (int i = 0; i < 2; i++)
        a_voff[i] = (uint32_t)(min((wave * 2 + i) * 16 + (lane >> 2), M - 1 - m0) * lda) + piece;  // rows past the edge re-read the last row
#pragma unroll
    for (int i = 0; i < Cfg::BI; i++)
        b_voff[i] = (uint32_t)(min((wave * Cfg::BI + i) * 16 + (lane >> 2), N - 1 - n0) * ldb) + piece;
    const uint8_t* a_ptr = A + (int64_t)m0 * lda + (int64_t)split * (K_part / 64) * a_unit;
    const uint8_t* b_ptr = Bt + (int64_t)n0 * ldb + (int64_t)split * (K_part / 64) * b_unit;
    // DMA d = 0..NDMA-1 of this wave's share of a step (4 of A, then Bt); the pointers move on after the last
    auto issue1 = [&](int stage, int d) __attribute__((always_inline)) {
        const uint32_t base = lds_u32 + stage * Cfg::STAGE;
        if (d < 4) {
            const int h = d >> 1, i = d & 1;
            dma_mid(a_ptr + h * a_unit, a_voff[i], base + h * MID_A_UNIT + (wave * 2 + i) * 1024);
        } else {
            const int h = (d - 4) / Cfg::BI, i = (d - 4) % Cfg::BI;
            dma_mid(b_ptr + h * b_unit, b_voff[i], base + 2 * MID_A_UNIT + h * Cfg::B_UNIT + (wave * Cfg::BI + i) * 1024);
        }
        if (d == Cfg::NDMA - 1) {
            a_ptr += 2 * a_unit;
            b_ptr += 2 * b_unit;
        }
    };

    // ---- fragments: lane -> tile row lane % 16, k quarter lane / 16 (32 bytes = two 16-byte pieces of one unit)
    const int frow = lane & 15, fq = lane >> 4;
    const int fsw = (frow >> 3) & 1;
    const int f_row0 = frow * 64 + ((((fq & 1) * 2 + 0) ^ fsw) << 4);
    const int f_row1 = frow * 64 + ((((fq & 1) * 2 + 1) ^ fsw) << 4);
    const int fa_off = (fq >> 1) * MID_A_UNIT + wm * 64 * 64;
    const int fb_off = 2 * MID_A_UNIT + (fq >> 1) * Cfg::B_UNIT + wn * (TJ * 16) * 64;

    v4f_m acc[TJ][4];  // [tj][ti]
#pragma unroll
    for (int tj = 0; tj < TJ; tj++)
#pragma unroll
        for (int ti = 0; ti < 4; ti++) acc[tj][ti] = (v4f_m){0.f, 0.f, 0.f, 0.f};

    const int steps = K_part / 128;
    constexpr int LEAD = Cfg::NSTAGE - 1;  // steps of data in flight
#pragma unroll
    for (int p = 0; p < LEAD; p++)
        if (p < steps) {
#pragma unroll
            for (int d = 0; d < Cfg::NDMA; d++) issue1(p, d);
        }
    int cur = 0;  // stage of step s
    for (int s = 0; s < steps; s++) {
        const uint8_t* st = smem + cur * Cfg::STAGE;
        // wait until this wave's DMAs of step s have landed: everything issued after them may still be in flight
        const int later = min(LEAD - 1, steps - 1 - s);
        if constexpr (TJ == 4) {
            if (later == 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
            else if (later == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            if (later == 1) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        asm volatile("s_barrier" ::: "memory");  // ... and so have everybody's
        v8i fa[4], fb[TJ];
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint8_t* pa = st + fa_off + t * 16 * 64;
            fa[t] = read_frag(pa + f_row0, pa + f_row1);
        }
#pragma unroll
        for (int t = 0; t < TJ; t++) {
            const uint8_t* pb = st + fb_off + t * 16 * 64;
            fb[t] = read_frag(pb + f_row0, pb + f_row1);
        }
        // the stage read in step s-1 (the barrier at its end has been passed) is refilled with step s+LEAD, one DMA
        // after every second MFMA: a burst of them would hold up all four waves at the CU's one load unit
        const bool more = s + LEAD < steps;
        const int refill = cur == 0 ? Cfg::NSTAGE - 1 : cur - 1;
#pragma unroll
        for (int ti = 0; ti < 4; ti++)
#pragma unroll
            for (int tj = 0; tj < TJ; tj++) {
                acc[tj][ti] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[tj], fa[ti], acc[tj][ti], BF, AF, 0, 0, 0, 0);
                if (tj & 1) {
                    const int d = (ti * TJ + tj) >> 1;
                    F8MI_SCHED_FENCE();
                    if (d < Cfg::NDMA && more) issue1(refill, d);
                    F8MI_SCHED_FENCE();
                }
            }
        lds_barrier();  // everybody is done reading this stage before step s+1 refills it
        cur = cur + 1 == Cfg::NSTAGE ? 0 : cur + 1;
    }

    // ---- epilogue: MFMA(first = Bt rows, second = A rows) leaves lane l with row ti*16 + l%16 and the four
    // columns tj*16 + 4*(l/16) + e of the wave's 64 x (16 TJ)
    const int lm = lane & 15, lq = lane >> 4;
    const int wcol0 = n0 + wn * (TJ * 16);
    if constexpr (C_DT == F8MI_FP32) {
#pragma unroll
        for (int tj = 0; tj < TJ; tj++) {
            const int col = wcol0 + tj * 16 + 4 * lq;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (col + e < N) bv[e] = load_bias<C_DT>(bias, col + e);
            }
#pragma unroll
            for (int ti = 0; ti < 4; ti++) {
                const int row = m0 + wm * 64 + ti * 16 + lm;
                if (row >= M || col >= N) continue;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[tj][ti][e] * inv + bv[e];
                float* dst = (float*)C + ((int64_t)split * M + row) * ldc + col;
                if (c_vec_ok && col + 4 <= N) {
                    store16_any(dst, make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (col + e < N) dst[e] = v[e];
                }
            }
        }
    } else {
        // 2-byte outputs: v_permlane16_swap between the accumulator tiles 2p and 2p + 1 trades the odd 16-lane rows of
        // the first for the even ones of the second, which turns a lane's 4 + 4 columns of two tiles into 8
        // neighbouring columns of one (lq even: columns 4 lq .. + 7 of tile 2p, lq odd: 4 (lq - 1) .. + 7 of tile
        // 2p + 1): one 16-byte store per lane, 64 contiguous bytes per row and instruction.
        float bv[TJ][4];
#pragma unroll
        for (int tj = 0; tj < TJ; tj++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int col = wcol0 + tj * 16 + 4 * lq + e;
                bv[tj][e] = (bias && col < N) ? load_bias<C_DT>(bias, col) : 0.f;
            }
        }
        const int col_l = (lq & 1) * 16 + (lq >> 1) * 8;
#pragma unroll
        for (int ti = 0; ti < 4; ti++) {
            const int row = m0 + wm * 64 + ti * 16 + lm;
#pragma unroll
            for (int tp = 0; tp < TJ / 2; tp++) {
                const int te = 2 * tp, to = 2 * tp + 1;
                const uint32_t x0 = pack2<C_DT>(acc[te][ti][0] * inv + bv[te][0], acc[te][ti][1] * inv + bv[te][1]);
                const uint32_t x1 = pack2<C_DT>(acc[te][ti][2] * inv + bv[te][2], acc[te][ti][3] * inv + bv[te][3]);
                const uint32_t y0 = pack2<C_DT>(acc[to][ti][0] * inv + bv[to][0], acc[to][ti][1] * inv + bv[to][1]);
                const uint32_t y1 = pack2<C_DT>(acc[to][ti][2] * inv + bv[to][2], acc[to][ti][3] * inv + bv[to][3]);
                const auto s0 = __builtin_amdgcn_permlane16_swap(x0, y0, false, false);  // every lane takes part
                const auto s1 = __builtin_amdgcn_permlane16_swap(x1, y1, false, false);
                const int col = wcol0 + tp * 32 + col_l;
                if (row < M && col < N) {
                    uint16_t* dst = (uint16_t*)C + (int64_t)row * ldc + col;
                    if (c_vec_ok && col + 8 <= N) {
                        store16_any(dst, make_uint4(s0[0], s1[0], s0[1], s1[1]));
                    } else {
                        const uint32_t w[4] = {s0[0], s1[0], s0[1], s1[1]};
#pragma unroll
                        for (int e = 0; e < 8; e++)
                            if (col + e < N) dst[e] = (uint16_t)((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
                    }
                }
            }
        }
    }
}

template <int AF, int BF, int C_DT, int TJ>
static int launch_mid4(hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt, int64_t ldb,
                       int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc, const void* bias,
                       int c_vec_ok, int k_splits) {
    static std::atomic<uint64_t> lds_allowed{0};
    auto kern = gemm_mid_kernel<AF, BF, C_DT, TJ>;
    if (int rc = allow_big_lds(kern, MidCfg<TJ>::LDS, lds_allowed)) return rc;
    const int tiles_m = (M + MID_TILE_M - 1) / MID_TILE_M, tiles_n = (N + MidCfg<TJ>::TILE_N - 1) / MidCfg<TJ>::TILE_N;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), (unsigned)k_splits), dim3(GEMM_THREADS), MidCfg<TJ>::LDS, stream, A, lda, a_unit,
                       Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok, k_splits);
    return check_hip(hipGetLastError(), "gemm (128-row tiles) kernel launch");
}

template <int AF, int BF, int C_DT>
static int launch_mid3(bool wide, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt, int64_t ldb,
                       int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc, const void* bias,
                       int c_vec_ok, int k_splits) {
    if (wide) return launch_mid4<AF, BF, C_DT, 8>(stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
    return launch_mid4<AF, BF, C_DT, 4>(stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
}

template <int AF, int BF>
static int launch_mid2(int c_dtype, bool wide, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt,
                       int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc,
                       const void* bias, int c_vec_ok, int k_splits) {
    if (c_dtype == F8MI_BF16) return launch_mid3<AF, BF, F8MI_BF16>(wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
    if (c_dtype == F8MI_FP16) return launch_mid3<AF, BF, F8MI_FP16>(wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
    return launch_mid3<AF, BF, F8MI_FP32>(wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
}

static int launch_mid1(int a_fmt, int b_fmt, int c_dtype, bool wide, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                       const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C,
                       int64_t ldc, const void* bias, int c_vec_ok, int k_splits) {
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E4M3FN) return launch_mid2<0, 0>(c_dtype, wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
    if (a_fmt == F8MI_E5M2 && b_fmt == F8MI_E4M3FN) return launch_mid2<1, 0>(c_dtype, wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E5M2) return launch_mid2<0, 1>(c_dtype, wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
    return launch_mid2<1, 1>(c_dtype, wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, k_splits);
}

// wide: 128 x 256 tiles instead of 128 x 128
int launch_gemm_mid(int a_fmt, int b_fmt, int c_dtype, bool wide, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                    const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C,
                    int64_t ldc, const void* bias, int c_vec_ok) {
    return launch_mid1(a_fmt, b_fmt, c_dtype, wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, c_vec_ok, 1);
}

// C = (partial[0] + partial[1] + ... in this order) / (sa * sb) + bias: four neighbouring columns per lane (N % 4 == 0)
template <int C_DT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int k_splits, int M, int N,
                                                            const float* __restrict__ sa_dev, const float* __restrict__ sb_dev,
                                                            void* __restrict__ C, int64_t ldc, const void* __restrict__ bias, int c_vec_ok) {
    const int64_t quads = (int64_t)N / 4;
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= (int64_t)M * quads) return;
    const int64_t row = q / quads;
    const int col = (int)(q % quads) * 4;
    const float inv = __fdiv_rn(1.0f, *sa_dev) * __fdiv_rn(1.0f, *sb_dev);
    const int64_t slab = (int64_t)M * N;
    float4 sum = *(const float4*)(partial + row * N + col);
    for (int s = 1; s < k_splits; s++) {
        const float4 p = *(const float4*)(partial + s * slab + row * N + col);
        sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
    }
    float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = v[e] * inv + (bias ? load_bias<C_DT>(bias, col + e) : 0.f);
    if constexpr (C_DT == F8MI_FP32) {
        float* dst = (float*)C + row * ldc + col;
        if (c_vec_ok) {
            store16_any(dst, make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])));
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) dst[e] = v[e];
        }
    } else {
        uint16_t* dst = (uint16_t*)C + row * ldc + col;
        const uint32_t p0 = pack2<C_DT>(v[0], v[1]), p1 = pack2<C_DT>(v[2], v[3]);
        if (c_vec_ok) {  // one 8-byte store at element alignment
            store8_any(dst, p0, p1);
        } else {
            dst[0] = (uint16_t)(p0 & 0xffffu); dst[1] = (uint16_t)(p0 >> 16);
            dst[2] = (uint16_t)(p1 & 0xffffu); dst[3] = (uint16_t)(p1 >> 16);
        }
    }
}

// The contraction split k_splits ways over workgroups (outputs of few tiles and a long k: every CU gets a part).
// `partial` holds k_splits x M x N floats (16-byte aligned); host side has checked K % (128 * k_splits) == 0, N % 4 == 0.
int launch_gemm_mid_splitk(int a_fmt, int b_fmt, int c_dtype, bool wide, int k_splits, float* partial, hipStream_t stream, const uint8_t* A,
                           int64_t lda, int64_t a_unit, const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa,
                           const float* sb, void* C, int64_t ldc, const void* bias, int c_vec_ok) {
    if (int rc = launch_mid1(a_fmt, b_fmt, F8MI_FP32, wide, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, partial, N, nullptr, 1, k_splits))
        return rc;
    const int64_t quads = (int64_t)M * (N / 4);
    const dim3 grid((unsigned)((quads + 255) / 256));
    if (c_dtype == F8MI_BF16) hipLaunchKernelGGL(splitk_reduce_kernel<F8MI_BF16>, grid, dim3(256), 0, stream, partial, k_splits, M, N, sa, sb, C, ldc, bias, c_vec_ok);
    else if (c_dtype == F8MI_FP16) hipLaunchKernelGGL(splitk_reduce_kernel<F8MI_FP16>, grid, dim3(256), 0, stream, partial, k_splits, M, N, sa, sb, C, ldc, bias, c_vec_ok);
    else hipLaunchKernelGGL(splitk_reduce_kernel<F8MI_FP32>, grid, dim3(256), 0, stream, partial, k_splits, M, N, sa, sb, C, ldc, bias, c_vec_ok);
    return check_hip(hipGetLastError(), "gemm split-k reduction kernel launch");
}

}  // namespace f8mi
