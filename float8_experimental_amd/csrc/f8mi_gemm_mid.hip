// K3 for outputs of few 256 x 256 tiles: the same 16x16x128 MFMA, LDS-DMA and LDS layout as
// f8mi_gemm_dma16_impl.h on 128 x 128 tiles, so that four times as many workgroups share the CUs.
//
// The large-tile kernel is built for the regime where every CU has tiles queued: one workgroup owns a CU
// (160 KB of LDS, 512 registers per lane) and walks all of k in 1.1 us steps -- 70 us for k = 8192 however
// few tiles there are.  With 512 rows and 8192 columns that is 64 workgroups on 256 CUs.  Here a workgroup
// (4 waves as 2 x 2, 64 x 64 outputs each = 16 accumulator tiles) takes a 128 x 128 tile: 256 workgroups for the
// same output.  LDS holds four stages of (128 + 128 rows) x 128 k; the DMAs of step s+3 are issued during step s,
// one after every second MFMA (a step is 0.4 us, less than the latency of a DMA), the rest of the schedule is left
// to the compiler: per step and wave a wait for the current step's 8 DMAs, 16 fragment reads, 16 MFMAs, two
// barriers.
//
// A wave's accumulation order over k is that of the large-tile kernels (128-deep steps in sequence, the same
// 32 contraction bytes per lane), so the results are the same bits.
// Host side guarantees: K % 128 == 0, K >= 128, 16-byte aligned operands and strides.
#include "f8mi_gemm_util.h"

namespace f8mi {

typedef float v4f_m __attribute__((ext_vector_type(4)));

constexpr int MID_TILE = 128;
constexpr int MID_HALF = MID_TILE * 64;           // one operand, one 64-deep unit: 8 KB
constexpr int MID_STAGE = 4 * MID_HALF;           // A (2 units) + Bt (2 units): 32 KB
constexpr int MID_NSTAGE = 4;
constexpr int MID_LDS = MID_NSTAGE * MID_STAGE;   // 128 KB

__device__ __forceinline__ void dma_mid(const uint8_t* base, uint32_t voff, uint32_t lds_addr) {
    // M0 carries the LDS address; one wait state between the scalar write of M0 and its use
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds_addr) : "memory");
}

template <int AF, int BF, int C_DT>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_mid_kernel(
    const uint8_t* __restrict__ A, int64_t lda, int64_t a_unit, const uint8_t* __restrict__ Bt, int64_t ldb, int64_t b_unit,
    int M, int N, int K, const float* __restrict__ sa_dev, const float* __restrict__ sb_dev, void* __restrict__ C,
    int64_t ldc, const void* __restrict__ bias, int tiles_m, int c_vec_ok) {
    extern __shared__ __align__(16) uint8_t smem[];
    // consecutive workgroup ids go to the 8 XCDs round-robin; re-deal them so that one XCD (one L2) gets a
    // contiguous run of the tile order (rows fastest): the workgroups that share a block of Bt sit behind the same L2
    int lid = blockIdx.x;
    if (gridDim.x % NUM_XCD == 0) lid = (lid % NUM_XCD) * (gridDim.x / NUM_XCD) + lid / NUM_XCD;
    const int tm = lid % tiles_m, tn = lid / tiles_m;
    const int m0 = tm * MID_TILE, n0 = tn * MID_TILE;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- DMA: one instruction = 16 rows x 64 B of one unit, landing as 1 KB of consecutive LDS; lane l fetches
    // row l/4 of the sixteen, piece (l%4) ^ (l/32) (the slot swizzle, applied on the global side).  Wave w
    // brings row groups 2w and 2w+1 of both units of A and of Bt: 8 instructions per step.
    const uint32_t lds_u32 = (uint32_t)(uintptr_t)smem;
    uint32_t a_voff[2], b_voff[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int r = (wave * 2 + i) * 16 + (lane >> 2);
        const uint32_t piece = (uint32_t)(((lane & 3) ^ (lane >> 5)) << 4);
        a_voff[i] = (uint32_t)(min(r, M - 1 - m0) * lda) + piece;  // rows past the edge re-read the last row
        b_voff[i] = (uint32_t)(min(r, N - 1 - n0) * ldb) + piece;
    }
    const uint8_t* a_ptr = A + (int64_t)m0 * lda;
    const uint8_t* b_ptr = Bt + (int64_t)n0 * ldb;
    // DMA d = 0..7 of this wave's share of a step (A and Bt alternating); the pointers move on after the last
    auto issue1 = [&](int stage, int d) __attribute__((always_inline)) {
        const uint32_t dst = lds_u32 + stage * MID_STAGE + wave * 2048;
        const int h = d >> 2, i = (d >> 1) & 1;
        if ((d & 1) == 0) dma_mid(a_ptr + h * a_unit, a_voff[i], dst + h * MID_HALF + i * 1024);
        else dma_mid(b_ptr + h * b_unit, b_voff[i], dst + (2 + h) * MID_HALF + i * 1024);
        if (d == 7) {
            a_ptr += 2 * a_unit;
            b_ptr += 2 * b_unit;
        }
    };
    auto issue = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int d = 0; d < 8; d++) issue1(stage, d);
    };

    // ---- fragments: lane -> tile row lane % 16, k quarter lane / 16 (32 bytes = two 16-byte pieces of one unit)
    const int frow = lane & 15, fq = lane >> 4;
    const int fsw = (frow >> 3) & 1;
    const int f_off0 = (fq >> 1) * MID_HALF + frow * 64 + ((((fq & 1) * 2 + 0) ^ fsw) << 4);
    const int f_off1 = (fq >> 1) * MID_HALF + frow * 64 + ((((fq & 1) * 2 + 1) ^ fsw) << 4);

    v4f_m acc[4][4];  // [tj][ti]
#pragma unroll
    for (int tj = 0; tj < 4; tj++)
#pragma unroll
        for (int ti = 0; ti < 4; ti++) acc[tj][ti] = (v4f_m){0.f, 0.f, 0.f, 0.f};

    const int steps = K / 128;
    constexpr int LEAD = MID_NSTAGE - 1;  // steps of data in flight
#pragma unroll
    for (int p = 0; p < LEAD; p++)
        if (p < steps) issue(p);
    for (int s = 0; s < steps; s++) {
        const uint8_t* st = smem + (s & (MID_NSTAGE - 1)) * MID_STAGE;
        // wait until this wave's 8 DMAs of step s have landed: everything issued after them may still be in flight
        const int later = min(LEAD - 1, steps - 1 - s);
        if (later == 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else if (later == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        asm volatile("s_barrier" ::: "memory");  // ... and so have everybody's
        v8i fa[4], fb[4];
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint8_t* pa = st + (wm * 64 + t * 16) * 64;
            const uint8_t* pb = st + 2 * MID_HALF + (wn * 64 + t * 16) * 64;
            fa[t] = read_frag(pa + f_off0, pa + f_off1);
            fb[t] = read_frag(pb + f_off0, pb + f_off1);
        }
        // the stage read in step s-1 (the barrier at its end has been passed) is refilled with step s+LEAD, one DMA
        // after every second MFMA: a burst of them would hold up all four waves at the CU's one load unit
        const bool more = s + LEAD < steps;
        const int refill = (s + LEAD) & (MID_NSTAGE - 1);
#pragma unroll
        for (int ti = 0; ti < 4; ti++)
#pragma unroll
            for (int tj = 0; tj < 4; tj++) {
                acc[tj][ti] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[tj], fa[ti], acc[tj][ti], BF, AF, 0, 0, 0, 0);
                if (tj & 1) {
                    F8MI_SCHED_FENCE();
                    if (more) issue1(refill, ti * 2 + (tj >> 1));
                    F8MI_SCHED_FENCE();
                }
            }
        lds_barrier();  // everybody is done reading this stage before step s+1 refills it
    }

    // ---- epilogue: MFMA(first = Bt rows, second = A rows) leaves lane l with row ti*16 + l%16 and the four
    // columns tj*16 + 4*(l/16) + e of the wave's 64 x 64
    const float inv = __fdiv_rn(1.0f, *sa_dev) * __fdiv_rn(1.0f, *sb_dev);
    const int lm = lane & 15, lq = lane >> 4;
#pragma unroll
    for (int tj = 0; tj < 4; tj++) {
        const int col = n0 + wn * 64 + tj * 16 + 4 * lq;
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
            if constexpr (C_DT == F8MI_FP32) {
                float* dst = (float*)C + (int64_t)row * ldc + col;
                if (c_vec_ok && col + 4 <= N) {
                    *(float4*)dst = make_float4(v[0], v[1], v[2], v[3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (col + e < N) dst[e] = v[e];
                }
            } else {
                uint16_t* dst = (uint16_t*)C + (int64_t)row * ldc + col;
                const uint32_t p0 = pack2<C_DT>(v[0], v[1]), p1 = pack2<C_DT>(v[2], v[3]);
                if (c_vec_ok && col + 4 <= N) {
                    *(uint2*)dst = make_uint2(p0, p1);
                } else {
                    const uint32_t w[2] = {p0, p1};
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (col + e < N) dst[e] = (uint16_t)((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
                }
            }
        }
    }
}

template <int AF, int BF, int C_DT>
static int launch_mid3(dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt, int64_t ldb,
                       int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc, const void* bias,
                       int tiles_m, int c_vec_ok) {
    static std::atomic<uint64_t> lds_allowed{0};
    auto kern = gemm_mid_kernel<AF, BF, C_DT>;
    if (int rc = allow_big_lds(kern, MID_LDS, lds_allowed)) return rc;
    hipLaunchKernelGGL(kern, g, dim3(GEMM_THREADS), MID_LDS, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok);
    return check_hip(hipGetLastError(), "gemm (128 x 128 tiles) kernel launch");
}

template <int AF, int BF>
static int launch_mid2(int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt,
                       int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc,
                       const void* bias, int tiles_m, int c_vec_ok) {
    if (c_dtype == F8MI_BF16) return launch_mid3<AF, BF, F8MI_BF16>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok);
    if (c_dtype == F8MI_FP16) return launch_mid3<AF, BF, F8MI_FP16>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok);
    return launch_mid3<AF, BF, F8MI_FP32>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok);
}

int launch_gemm_mid(int a_fmt, int b_fmt, int c_dtype, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                    const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C,
                    int64_t ldc, const void* bias, int c_vec_ok) {
    const int tiles_m = (M + MID_TILE - 1) / MID_TILE, tiles_n = (N + MID_TILE - 1) / MID_TILE;
    const dim3 g((unsigned)(tiles_m * tiles_n));
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E4M3FN) return launch_mid2<0, 0>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok);
    if (a_fmt == F8MI_E5M2 && b_fmt == F8MI_E4M3FN) return launch_mid2<1, 0>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok);
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E5M2) return launch_mid2<0, 1>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok);
    return launch_mid2<1, 1>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, c_vec_ok);
}

}  // namespace f8mi
