// K3, LDS-DMA path on 32x32x64 MFMAs (takes K % 128 == 64; K % 128 == 0 goes to
// f8mi_gemm_dma16.hip): the scaled fp8 GEMM of f8mi_gemm.hip with the operands moved
// HBM -> LDS by the load unit itself (global_load_lds_dwordx4: every lane names 16
// bytes of global memory, the wave's 64 pieces land in 1 KB of consecutive LDS
// starting at M0), no staging registers and no LDS writes by the waves.
//
// Same macro tile (256 x 256, 4 waves of 128 x 128, 256 accumulator registers) and
// the same MFMA / fragment scheme; what changes is the pipeline:
//   * K is consumed in units of 64 bytes (one MFMA depth).  The LDS is a ring of
//     5 slots of 32 KB = [A: 256 rows x 64 B][Bt: 256 rows x 64 B], all 160 KB.
//   * 16-byte piece c of tile row r of a slot lives at r*64 + ((c ^ ((r >> 2) & 3)) * 16):
//     16 consecutive rows of one piece cover all 64 banks, so fragment reads run
//     at the LDS's full rate.  The swizzle is applied on the global side: lane l
//     of DMA instruction j fetches row 16j + l/4, piece (l%4) ^ ((l/16) % 4).
//   * per unit and wave: 8 DMA instructions (4 for A, 4 for Bt), issued one at a time
//     between MFMAs after the barrier that ends all reads of the slot they refill,
//     5 units ahead of the multiply (about two full K steps of latency cover).
//   * one barrier per unit, after the second MFMA group: before it a wave has
//     fetched all its A fragments of the unit and waits until its own DMAs of the
//     next unit have landed (vmcnt); after it every wave's have, and the Bt
//     fragments of the next unit are read between the remaining MFMAs.
// Requirements checked by the host: 16-byte aligned operands and row strides, K a
// multiple of 64 and at least 384.  Everything else runs the register-staged kernel.
#include "f8mi_gemm_util.h"

namespace f8mi {

constexpr int UK = 64;                        // K bytes per unit
constexpr int SLOT_BYTES = (BM + BN) * UK;    // 32 KB
constexpr int NSLOT = 5;
constexpr int DMA_LDS = NSLOT * SLOT_BYTES;   // 160 KB
static_assert(DMA_LDS >= EPI_BYTES, "the C staging tile reuses the ring");

// One DMA instruction: lane's 16 bytes at base + voff -> LDS[lds_addr + lane*16].
// M0 carries the LDS address; the s_nop covers the one wait state the load unit needs
// between a scalar write of M0 and reading it.
__device__ __forceinline__ void dma16(const uint8_t* base, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds_addr) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_dma() {
    if constexpr (N >= 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else if constexpr (N == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if constexpr (N == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int AF, int BF, int C_DT, bool ODD>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_nt_dma_kernel(
    const uint8_t* __restrict__ A, int64_t lda, int64_t a_unit, const uint8_t* __restrict__ Bt, int64_t ldb, int64_t b_unit,
    int M, int N, int K, const float* __restrict__ sa_dev, const float* __restrict__ sb_dev, void* __restrict__ C,
    int64_t ldc, const void* __restrict__ bias, int tiles_m, int tiles_n, int c_vec_ok) {
    extern __shared__ __align__(16) uint8_t smem[];
    // lda / ldb: bytes from one operand row to the next; a_unit / b_unit: bytes from one 64-deep unit
    // to the next.  Row-major operands: (row stride, 64); k-blocked [K/64][rows][64]: (64, rows*64).

    // ---- which tile (same walk as the register-staged kernel)
    int lid = blockIdx.x;
    const int npid = gridDim.x;
    lid = xcd_contiguous_id(lid, npid);
    const int width = GROUP_M * tiles_n;
    const int group = lid / width;
    const int first_m = group * GROUP_M;
    const int gsz = min(tiles_m - first_m, GROUP_M);
    const int tm = first_m + (lid % width) % gsz;
    const int tn = (lid % width) / gsz;
    const int m0 = tm * BM, n0 = tn * BN;

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- DMA addressing.  Instruction j = wave*4 + i of a slot half covers tile rows 16j .. 16j+15.
    const int drow = lane >> 2;
    const int dpiece = (lane & 3) ^ ((lane >> 4) & 3);
    uint32_t a_voff[4], b_voff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = (wave * 4 + i) * 16 + drow;
        a_voff[i] = (uint32_t)(min(r, M - 1 - m0) * lda) + dpiece * 16;  // rows past the edge re-read the last row
        b_voff[i] = (uint32_t)(min(r, N - 1 - n0) * ldb) + dpiece * 16;
    }
    const uint8_t* a_ptr = A + (int64_t)m0 * lda;  // advanced by one unit per issued unit
    const uint8_t* b_ptr = Bt + (int64_t)n0 * ldb;
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t dma_lds = lds0 + wave * 4096;  // + slot*SLOT_BYTES + (Bt ? BM*UK : 0) + i*1024
    // A unit's 8 DMAs (d = 0..3: A rows, 4..7: Bt rows) are issued one at a time between MFMAs, two per
    // MFMA group, waves 0,1 after the group's 1st and 3rd MFMA and waves 2,3 after its 2nd and 4th: a
    // burst would hold the wave (and its MFMAs) until the load unit, which the four waves share, has
    // taken them all.
    uint32_t refill_dst = 0;  // LDS address of this wave's part of the slot being refilled
    const bool late = wave >= 2;
    auto issue_one = [&](int d) __attribute__((always_inline)) {
        if (d < 4) dma16(a_ptr, a_voff[d], refill_dst + d * 1024);
        else dma16(b_ptr, b_voff[d - 4], refill_dst + BM * UK + (d - 4) * 1024);
        if (d == 7) {
            a_ptr += a_unit;
            b_ptr += b_unit;
        }
    };

    // ---- fragment addressing: lane -> tile row (lane % 32), k half (lane / 32)
    const int frow = lane & 31, fh = lane >> 5;
    const int fsw = (frow >> 2) & 3;
    const int f_off0 = frow * UK + (((fh * 2 + 0) ^ fsw) << 4);
    const int f_off1 = frow * UK + (((fh * 2 + 1) ^ fsw) << 4);
    const int a_frag_base = (wm * 128) * UK;
    const int b_frag_base = BM * UK + (wn * 128) * UK;
    auto frag_a = [&](const uint8_t* slot, int ti) __attribute__((always_inline)) {
        const uint8_t* p = slot + a_frag_base + ti * 32 * UK;
        return read_frag(p + f_off0, p + f_off1);
    };
    auto frag_b = [&](const uint8_t* slot, int tj) __attribute__((always_inline)) {
        const uint8_t* p = slot + b_frag_base + tj * 32 * UK;
        return read_frag(p + f_off0, p + f_off1);
    };

    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    v8i fb[2][4];  // [unit parity][n tile]
    v8i fa[4];     // the unit's four A fragments; fa[0] is refilled for the next unit during the last group

    // ---- prologue: units 0..3 and the A half of unit 4 (its Bt half is issued by unit 0, like every
    // later refill), wait for unit 0 (this wave's oldest 8 of 36 DMAs), first fragments
#pragma unroll
    for (int x = 0; x < NSLOT; x++) {
        refill_dst = dma_lds + x * SLOT_BYTES;
#pragma unroll
        for (int d = 0; d < (x < NSLOT - 1 ? 8 : 4); d++) issue_one(d);
    }
    asm volatile("s_waitcnt vmcnt(28)" ::: "memory");
    lds_barrier();
#pragma unroll
    for (int x = 0; x < 4; x++) fb[0][x] = frag_b(smem, x);
    fa[0] = frag_a(smem, 0);

    // One unit u = 4 groups of 4 MFMAs.  P: parity of u.  MODE: 0 = steady (finishes the refill begun by
    // unit u-1, refills its own slot with unit u+5); 1..5 = the last five units of the tile, which
    // refill nothing (1 still finishes unit u-1's); 5 = last unit, nothing follows.
    int slot = 0;
    auto unit = [&](auto parity, auto mode) __attribute__((always_inline)) {
        constexpr int P = decltype(parity)::value;
        constexpr int MODE = decltype(mode)::value;
        constexpr bool PENDING = MODE <= 1, REFILL = MODE == 0, HAS_NEXT = MODE < 5;
        const int next_slot = slot + 1 == NSLOT ? 0 : slot + 1;
        const uint8_t* cur = smem + slot * SLOT_BYTES;
        const uint8_t* nxt = smem + next_slot * SLOT_BYTES;

#pragma unroll
        for (int g = 0; g < 4; g++) {
            if (g == 0) fa[1] = frag_a(cur, 1);
            if (g == 1) { fa[2] = frag_a(cur, 2); fa[3] = frag_a(cur, 3); }
            if (g == 2) {
                // this wave's DMAs of unit u+1 have landed (those of units u+2 .. u+4 may be in flight)
                wait_dma<MODE <= 1 ? 24 : MODE == 2 ? 16 : MODE == 3 ? 8 : 0>();
                lds_barrier();  // everybody's have, and everybody is done reading this unit's slot
                if (REFILL) refill_dst = dma_lds + slot * SLOT_BYTES;
                if (HAS_NEXT) { fb[P ^ 1][0] = frag_b(nxt, 0); fb[P ^ 1][1] = frag_b(nxt, 1); fb[P ^ 1][2] = frag_b(nxt, 2); }
            }
            if (g == 3 && HAS_NEXT) { fb[P ^ 1][3] = frag_b(nxt, 3); fa[0] = frag_a(nxt, 0); }
            const bool dma_here = g < 2 ? PENDING : REFILL;
            const int d0 = g < 2 ? 4 + 2 * g : 2 * (g - 2);  // groups 0,1 finish the refill in progress, 2,3 start the new one
#pragma unroll
            for (int tj = 0; tj < 4; tj++) {
                acc[tj][g] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[P][tj], fa[g], acc[tj][g], BF, AF, 0, 0, 0, 0);
                F8MI_SCHED_FENCE();
                if (dma_here) {
                    if (late == (bool)(tj & 1)) issue_one(d0 + (tj >> 1));
                    F8MI_SCHED_FENCE();
                }
            }
        }
        slot = next_slot;
    };

    constexpr std::integral_constant<int, 0> c0{};
    constexpr std::integral_constant<int, 1> c1{};
    constexpr std::integral_constant<int, 2> c2{};
    constexpr std::integral_constant<int, 3> c3{};
    constexpr std::integral_constant<int, 4> c4{};
    constexpr std::integral_constant<int, 5> c5{};

    // ODD (from the host): K/64 - 5, the number of refilling units (>= 1), is odd.  Known at compile
    // time so that the whole tile is one loop of unit pairs between straight-line code.
    const int n_steady = K / UK - NSLOT;
    if constexpr (ODD) {
        unit(c0, c0);
        for (int u = 1; u < n_steady; u += 2) {
            unit(c1, c0);
            unit(c0, c0);
        }
        unit(c1, c1); unit(c0, c2); unit(c1, c3); unit(c0, c4); unit(c1, c5);
    } else {
        for (int u = 0; u < n_steady; u += 2) {
            unit(c0, c0);
            unit(c1, c0);
        }
        unit(c0, c1); unit(c1, c2); unit(c0, c3); unit(c1, c4); unit(c0, c5);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    store_c_tile<C_DT>(acc, smem, m0, n0, M, N, sa_dev, sb_dev, C, ldc, bias, c_vec_ok);
}

template <int AF, int BF, int C_DT, bool ODD>
static int launch_dma4(dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt, int64_t ldb,
                       int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc, const void* bias,
                       int tiles_m, int tiles_n, int c_vec_ok) {
    static std::atomic<uint64_t> lds_allowed{0};
    auto kern = gemm_nt_dma_kernel<AF, BF, C_DT, ODD>;
    if (int rc = allow_big_lds(kern, DMA_LDS, lds_allowed)) return rc;
    hipLaunchKernelGGL(kern, g, dim3(GEMM_THREADS), DMA_LDS, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias,
                       tiles_m, tiles_n, c_vec_ok);
    return check_hip(hipGetLastError(), "gemm (LDS-DMA) kernel launch");
}

template <int AF, int BF, int C_DT>
static int launch_dma3(dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt, int64_t ldb,
                       int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc, const void* bias,
                       int tiles_m, int tiles_n, int c_vec_ok) {
    if ((K / UK - NSLOT) & 1) return launch_dma4<AF, BF, C_DT, true>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    return launch_dma4<AF, BF, C_DT, false>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
}

template <int AF, int BF>
static int launch_dma2(int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit, const uint8_t* Bt,
                       int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc,
                       const void* bias, int tiles_m, int tiles_n, int c_vec_ok) {
    if (c_dtype == F8MI_BF16) return launch_dma3<AF, BF, F8MI_BF16>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    if (c_dtype == F8MI_FP16) return launch_dma3<AF, BF, F8MI_FP16>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    return launch_dma3<AF, BF, F8MI_FP32>(g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
}

int launch_gemm_dma(int a_fmt, int b_fmt, int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, int64_t a_unit,
                    const uint8_t* Bt, int64_t ldb, int64_t b_unit, int M, int N, int K, const float* sa, const float* sb, void* C,
                    int64_t ldc, const void* bias, int tiles_m, int tiles_n, int c_vec_ok) {
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E4M3FN) return launch_dma2<0, 0>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    if (a_fmt == F8MI_E5M2 && b_fmt == F8MI_E4M3FN) return launch_dma2<1, 0>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E5M2) return launch_dma2<0, 1>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    return launch_dma2<1, 1>(c_dtype, g, stream, A, lda, a_unit, Bt, ldb, b_unit, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
}

}  // namespace f8mi
