// K3: scaled fp8 GEMM  C[m][n] = (sum_k A[m][k] * Bt[n][k]) / (sa * sb)  on the
// gfx950 matrix cores (v_mfma_f32_32x32x64_f8f6f4, fp32 accumulate), MFMA-bound.
//
// Workgroup = 256 lanes (4 waves, 2 x 2), macro tile 256 x 256, K step 128 bytes.
// Each wave owns 128 x 128 of C = 4 x 4 MFMA tiles of 32 x 32 (256 accumulator
// registers), so there is one wave per SIMD and nothing hides latency for it:
// the loop is software-pipelined by hand.
//   * HBM -> registers -> LDS, two LDS stages of 64 KB.  The loads of K step
//     kb+2 are in flight while step kb is multiplied; they are written to the
//     free stage one iteration later, in small groups between MFMAs.
//   * LDS -> registers: every lane needs 32 consecutive k of one tile row per
//     MFMA (2 x 16-byte reads).  Fragments are double-buffered in registers: the
//     reads for the next 64-deep half step are issued between the MFMAs of the
//     current one.
//   * 16-byte piece c of tile row r lives at r*128 + ((c ^ ((r >> 1) & 7)) * 16): the
//     fragment reads run at the LDS's full 256 bytes per clock (64 banks).
//   * one s_barrier per K step, waiting on LDS traffic only (never on the HBM
//     loads in flight).
// The MFMA is issued with the Bt rows as its first operand, so a lane ends up
// holding 4 consecutive columns of one row of C: the epilogue scales, converts
// (v_cvt_pk_bf16_f32), packs 8 bytes per lane into a padded LDS tile and writes C
// with 16-byte stores, 256 contiguous bytes per row and wave.
// Workgroup ids are first re-dealt so that each of the 8 XCDs (which receive
// consecutive ids round-robin) works on one contiguous band of tiles, then
// walked in groups of 8 tile rows so the tiles in flight share A and B panels
// in that XCD's L2.
#include <cstdlib>
#include <cstring>

#include "f8mi_gemm_util.h"

namespace f8mi {

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

template <int AF, int BF, bool ALIGNED, int C_DT>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_nt_kernel(
    const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ Bt, int64_t ldb, int M, int N, int K,
    const float* __restrict__ sa_dev, const float* __restrict__ sb_dev, void* __restrict__ C, int64_t ldc,
    const void* __restrict__ bias, int tiles_m, int tiles_n, int c_vec_ok) {
    extern __shared__ __align__(16) uint8_t smem[];

    // ---- which tile
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
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- global -> register staging.  Lane t moves, per operand, rows i*64 + t/4 (i = 0..3) and of each
    // row the 16-byte pieces t%4 (first 64-deep half step) and t%4 + 4 (second half step).
    const int lrow = t >> 2, lc = t & 3;
    const uint8_t* a_base = A + (int64_t)m0 * lda;
    const uint8_t* b_base = Bt + (int64_t)n0 * ldb;
    uint32_t a_off[4], b_off[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = i * 64 + lrow;
        a_off[i] = (uint32_t)(min(r, M - 1 - m0) * lda) + lc * 16;  // rows past the edge re-read the last row
        b_off[i] = (uint32_t)(min(r, N - 1 - n0) * ldb) + lc * 16;
    }
    // piece c of tile row r sits at r*128 + ((c ^ swz(r)) * 16), swz(r) = (r >> 1) & 7: the LDS has 64
    // banks (256 bytes per clock), so the 16 lanes served together by a 16-byte read -- 16 consecutive
    // rows, same piece -- must land in 16 different 16-byte columns of a 256-byte span: the row parity
    // picks the 128-byte half, the swizzle the column inside it
    const int lsw = (lrow >> 1) & 7;
    const int st_off0 = lrow * BK + ((lc ^ lsw) << 4);        // + i*64*BK, half step 0 piece
    const int st_off1 = lrow * BK + (((lc + 4) ^ lsw) << 4);  // half step 1 piece

    const int nk_full = K / BK;
    const int nk = (K + BK - 1) / BK;

    uint4 ra[4][2], rb[4][2];  // staging registers [row slot][half]
    // GUARD = false: K step kb lies completely inside [0, K) and rows are 16-byte aligned
    auto gload = [&](int kb, int i, int h, auto guard) __attribute__((always_inline)) {
        const int k0 = kb * BK + h * 64;
        const uint8_t* pa = a_base + k0;
        const uint8_t* pb = b_base + k0;
        if constexpr (!decltype(guard)::value) {
            ra[i][h] = load_piece<ALIGNED, false>(pa + a_off[i], 16);
            rb[i][h] = load_piece<ALIGNED, false>(pb + b_off[i], 16);
        } else {
            ra[i][h] = load_piece<ALIGNED, true>(pa + a_off[i], K - k0 - lc * 16);
            rb[i][h] = load_piece<ALIGNED, true>(pb + b_off[i], K - k0 - lc * 16);
        }
    };
    auto lstore = [&](uint8_t* stage, int i, int h) __attribute__((always_inline)) {
        const int off = (h ? st_off1 : st_off0) + i * 64 * BK;
        *(uint4*)(stage + off) = ra[i][h];
        *(uint4*)(stage + BM * BK + off) = rb[i][h];
    };

    // ---- fragment addressing: lane -> tile row (lane % 32), k half (lane / 32)
    const int frow = lane & 31, fh = lane >> 5;
    const int fsw = (frow >> 1) & 7;
    int f_off[2][2];  // [ks][j]: byte offset of piece (ks*4 + fh*2 + j) of row frow
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int j = 0; j < 2; j++) f_off[ks][j] = frow * BK + (((ks * 4 + fh * 2 + j) ^ fsw) << 4);
    const int a_frag_base = (wm * 128) * BK;
    const int b_frag_base = BM * BK + (wn * 128) * BK;
    auto frag_a = [&](const uint8_t* stage, int ks, int ti) __attribute__((always_inline)) {
        return read_frag(stage + a_frag_base + ti * 32 * BK + f_off[ks][0], stage + a_frag_base + ti * 32 * BK + f_off[ks][1]);
    };
    auto frag_b = [&](const uint8_t* stage, int ks, int tj) __attribute__((always_inline)) {
        return read_frag(stage + b_frag_base + tj * 32 * BK + f_off[ks][0], stage + b_frag_base + tj * 32 * BK + f_off[ks][1]);
    };

    // acc[tj][ti]: MFMA(first = Bt rows (n), second = A rows (m)) -> lane holds m = lane%32,
    // n = 8*(e/4) + 4*(lane/32) + e%4 of its 32 x 32 tile
    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // Fragment registers.  The four Bt fragments of a half step are all live during it while the next
    // half step's four are being fetched; the A fragment is needed one 4-MFMA group at a time.
    v8i fb[2][4];  // [half-step parity][n tile]
    v8i fa[2];     // rolling: group g multiplies fa[g & 1] while fa[(g + 1) & 1] is being fetched

    constexpr std::true_type yes{};
    constexpr std::false_type no{};

    // Fills stage 0 with K step 0, starts the loads of K step 1 and fetches the first fragments.
    // The loads of K step 1 are issued in the loop's own order (and pinned there) so that the
    // compiler's count of loads in flight at the loop head is exact; a pessimistic count would make
    // every iteration wait for loads it has only just issued.
    auto prologue = [&](auto guard) __attribute__((always_inline)) {
        constexpr bool G = decltype(guard)::value;
#pragma unroll
        for (int i = 0; i < 4; i++) { gload(0, i, 0, guard); gload(0, i, 1, guard); }
#pragma unroll
        for (int i = 0; i < 4; i++) { lstore(smem, i, 0); lstore(smem, i, 1); }
        if (!G || nk > 1) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    F8MI_SCHED_FENCE();
                    gload(1, i, h, guard);
                }
        }
        F8MI_SCHED_FENCE();
        lds_barrier();
#pragma unroll
        for (int x = 0; x < 4; x++) fb[0][x] = frag_b(smem, 0, x);
        fa[0] = frag_a(smem, 0, 0);
    };

    // One K step = two half steps of 4 groups of 4 MFMAs.  Slotted in between the MFMAs, evenly spread:
    // the fragment reads for the next group / half step, the 16-byte LDS writes of K step kb+1 (first
    // its half-step-0 pieces, after the middle barrier its half-step-1 pieces) into the other stage, and
    // the loads of K step kb+2 into the registers just written out.
    // STEADY = true: K steps kb+1 and kb+2 exist and kb+2 needs no guards, so the body is
    // straight-line code; the (at most three) last steps of a tile run the general version.
    auto k_step = [&](int kb, auto steady) __attribute__((always_inline)) {
        constexpr bool STEADY = decltype(steady)::value;
        uint8_t* cur = smem + (kb & 1) * STAGE_BYTES;
        uint8_t* nxt = smem + ((kb + 1) & 1) * STAGE_BYTES;
        const bool has1 = STEADY || kb + 1 < nk, has2 = STEADY || kb + 2 < nk;

#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                if (h == 0) {
                    fa[(g + 1) & 1] = g < 3 ? frag_a(cur, 0, g + 1) : frag_a(cur, 1, 0);
                    fb[1][g] = frag_b(cur, 1, g);
                } else {
                    if (g < 3) fa[(g + 1) & 1] = frag_a(cur, 1, g + 1);
                    else if (has1) fa[0] = frag_a(nxt, 0, 0);
                    if (has1) fb[0][g] = frag_b(nxt, 0, g);
                }
                if (has1) lstore(nxt, g, h);
                if (has2) {
                    if constexpr (STEADY) gload(kb + 2, g, h, no);
                    else gload(kb + 2, g, h, yes);
                }
#pragma unroll
                for (int tj = 0; tj < 4; tj++)
                    acc[tj][g] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[h][tj], fa[g & 1], acc[tj][g], BF, AF, 0, 0, 0, 0);
                // A wave cannot run ahead of an MFMA it has not issued yet, so everything else has to be
                // slotted in between the MFMAs (each keeps the matrix core busy for 64 cycles) rather than
                // after them: MFMA, 2 LDS reads, MFMA, LDS write + load, twice.
#pragma unroll
                for (int rep = 0; rep < 2; rep++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // LDS read
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // LDS write
                    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // global load
                }
                F8MI_SCHED_FENCE();
            }
            // h = 0: the half-step-0 pieces of K step kb+1 are in place for everybody;
            // h = 1: its half-step-1 pieces are, and every wave is done reading `cur`.
            lds_barrier();
        }
    };

    const int n_steady = ALIGNED ? max(nk_full - 2, 0) : 0;
    if (n_steady > 0) {  // at least three full, aligned K steps
        prologue(no);
        int kb = 0;
        for (; kb < n_steady; kb++) k_step(kb, yes);
        for (; kb < nk; kb++) k_step(kb, no);
    } else if (nk > 0) {
        prologue(yes);
        for (int kb = 0; kb < nk; kb++) k_step(kb, no);
    }

    store_c_tile<C_DT>(acc, smem, m0, n0, M, N, sa_dev, sb_dev, C, ldc, bias, c_vec_ok);
}

template <int AF, int BF, bool ALIGNED, int C_DT>
static int launch_gemm3(dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, const uint8_t* Bt, int64_t ldb, int M,
                        int N, int K, const float* sa, const float* sb, void* C, int64_t ldc, const void* bias,
                        int tiles_m, int tiles_n, int c_vec_ok) {
    static std::atomic<uint64_t> lds_allowed{0};
    auto kern = gemm_nt_kernel<AF, BF, ALIGNED, C_DT>;
    if (int rc = allow_big_lds(kern, GEMM_LDS, lds_allowed)) return rc;
    hipLaunchKernelGGL(kern, g, dim3(GEMM_THREADS), GEMM_LDS, stream, A, lda, Bt, ldb, M, N, K, sa, sb, C, ldc, bias,
                       tiles_m, tiles_n, c_vec_ok);
    return check_hip(hipGetLastError(), "gemm kernel launch");
}

template <int AF, int BF, bool ALIGNED>
static int launch_gemm2(int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda, const uint8_t* Bt,
                        int64_t ldb, int M, int N, int K, const float* sa, const float* sb, void* C, int64_t ldc,
                        const void* bias, int tiles_m, int tiles_n, int c_vec_ok) {
    if (c_dtype == F8MI_BF16) return launch_gemm3<AF, BF, ALIGNED, F8MI_BF16>(g, stream, A, lda, Bt, ldb, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    if (c_dtype == F8MI_FP16) return launch_gemm3<AF, BF, ALIGNED, F8MI_FP16>(g, stream, A, lda, Bt, ldb, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    return launch_gemm3<AF, BF, ALIGNED, F8MI_FP32>(g, stream, A, lda, Bt, ldb, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
}

template <int AF, int BF>
static int launch_gemm1(bool aligned, int c_dtype, dim3 g, hipStream_t stream, const uint8_t* A, int64_t lda,
                        const uint8_t* Bt, int64_t ldb, int M, int N, int K, const float* sa, const float* sb, void* C,
                        int64_t ldc, const void* bias, int tiles_m, int tiles_n, int c_vec_ok) {
    if (aligned) return launch_gemm2<AF, BF, true>(c_dtype, g, stream, A, lda, Bt, ldb, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
    return launch_gemm2<AF, BF, false>(c_dtype, g, stream, A, lda, Bt, ldb, M, N, K, sa, sb, C, ldc, bias, tiles_m, tiles_n, c_vec_ok);
}

}  // namespace f8mi

using namespace f8mi;

// An output whose last round of 256 x 256 tiles would leave most CUs idle (at most 128 tiles in it) is split by
// rows: the tile rows that fill whole rounds go to the large-tile kernel, the rest to a 128-row-tile kernel that
// spreads them over all CUs (same accumulation order, so no output bit depends on the split).  Returns the number
// of tile rows for the large tiles (0: no split) and which 128-row tile takes the rest.
struct RowSplit { int64_t rows_large; int mid; };
static RowSplit split_last_round(int64_t tiles_m, int64_t tiles_n, int64_t k) {
    const int64_t tiles = tiles_m * tiles_n, per_round = 256;
    if (tiles <= per_round || tiles % per_round == 0) return {0, 0};
    const int64_t rows_large = (tiles / per_round) * per_round / tiles_n;
    if (rows_large < 1 || rows_large >= tiles_m) return {0, 0};
    const int mid = use_mid_tiles((tiles_m - rows_large) * BM, tiles_n * BN, k);
    if (!mid) return {0, 0};
    // in rounds of the large-tile kernel: a round of 128 x 128 tiles takes about 0.5, one of 128 x 256 tiles 0.8 (measured)
    const double cost = (double)((rows_large * tiles_n + per_round - 1) / per_round) + (mid == 1 ? 0.5 : 0.8);
    if (cost > (double)((tiles + per_round - 1) / per_round) - 0.1) return {0, 0};
    return {rows_large, mid};
}

// Which kernel computes an m x n x k product (codes: include/f8mi.h, F8MI_PLAN_*).  One function for both entry points,
// so that row-major and k-blocked operands of one shape always take the same kernel and give the same bits.
//   aligned, K % 128 == 0:  few 128-row tiles, a long k and a workspace (pick_k_splits) -> those tiles with k split over workgroups
//                           up to 16 rows, or up to 256 and a narrow Bt (use_skinny)
//                                                     -> few-row kernel (Bt streamed once per 128 rows, k split over waves)
//                           up to 256 tiles of 128 x 128 / 128 x 256 -> those
//                           K >= 384                  -> 256 x 256 tiles, 16x16x128 MFMA, LDS-DMA (the tile rows of a
//                                                        sparse last round: 128-row tiles, see split_last_round)
//   aligned, K % 64 == 0, K >= 384                    -> 256 x 256 tiles, 32x32x64 MFMA, LDS-DMA
//   anything else (ragged K, unaligned, short K)      -> 256 x 256 tiles, register-staged
struct GemmPlan { int kind; int parts; int mid; RowSplit split; };
static GemmPlan gemm_plan(int64_t m, int64_t n, int64_t k, bool aligned, int64_t ws_bytes) {
    GemmPlan p{F8MI_PLAN_STAGED, 0, 0, {0, 0}};
    if (aligned) {
        if (const int parts = pick_k_splits(m, n, k, ws_bytes)) {
            p.kind = F8MI_PLAN_TILES128_SPLIT_K; p.parts = parts; p.mid = use_mid_tiles(m, n, k);
            return p;
        }
        if (use_skinny(m, n, k)) { p.kind = F8MI_PLAN_FEW_ROWS; return p; }
        if (const int mid = use_mid_tiles(m, n, k)) { p.kind = F8MI_PLAN_TILES128; p.mid = mid; return p; }
    }
    if (aligned && k >= 384 && k % 64 == 0) {
        if (k % 128 == 0) {
            const int64_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
            p.split = split_last_round(tiles_m, tiles_n, k);
            p.kind = p.split.rows_large ? F8MI_PLAN_TILES256_AND_128 : F8MI_PLAN_TILES256;
            p.mid = p.split.mid;
            return p;
        }
        p.kind = F8MI_PLAN_TILES256_MFMA32;
    }
    return p;
}

extern "C" int f8mi_gemm_plan(int64_t m, int64_t n, int64_t k, int aligned, int64_t workspace_bytes) {
    if (m <= 0 || n <= 0 || k < 0) return 0;
    const GemmPlan p = gemm_plan(m, n, k, aligned != 0, workspace_bytes);
    return p.kind | (p.parts << 8) | (p.mid << 16);
}

extern "C" int f8mi_gemm_nt(const void* a, int a_fmt, int64_t lda, const void* bt, int b_fmt, int64_t ldb, int64_t m,
                            int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c,
                            int c_dtype, int64_t ldc, const void* bias_dev, void* stream_) {
    return f8mi_gemm_nt_ws(a, a_fmt, lda, bt, b_fmt, ldb, m, n, k, scale_a_dev, scale_b_dev, c, c_dtype, ldc, bias_dev, nullptr, 0, stream_);
}

extern "C" int f8mi_gemm_nt_ws(const void* a, int a_fmt, int64_t lda, const void* bt, int b_fmt, int64_t ldb, int64_t m,
                               int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c,
                               int c_dtype, int64_t ldc, const void* bias_dev, void* workspace, int64_t workspace_bytes,
                               void* stream_) {
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
    const int64_t csz = c_dtype == F8MI_FP32 ? 4 : 2;
    const int c_vec_ok = (uintptr_t)c % csz == 0;  // 16-byte stores at element alignment: any row pitch will do
    dim3 g((unsigned)(tiles_m * tiles_n));
    ProfScope prof(F8MI_K_GEMM, 2.0 * (double)m * (double)n * (double)k, stream);
    const uint8_t* A = (const uint8_t*)a;
    const uint8_t* B = (const uint8_t*)bt;
    const int M = (int)m, N = (int)n, K = (int)k;
    const bool ws_ok = workspace && (uintptr_t)workspace % 16 == 0;
    const GemmPlan plan = gemm_plan(m, n, k, aligned, ws_ok ? workspace_bytes : 0);
    switch (plan.kind) {
        case F8MI_PLAN_TILES128_SPLIT_K:
            return launch_gemm_mid_splitk(a_fmt, b_fmt, c_dtype, plan.mid == 2, plan.parts, (float*)workspace, stream, A, lda, 64, B, ldb, 64, M, N, K,
                                          scale_a_dev, scale_b_dev, c, ldc, bias_dev, c_vec_ok);
        case F8MI_PLAN_FEW_ROWS:
            return launch_gemm_skinny(a_fmt, b_fmt, c_dtype, stream, A, lda, 64, B, ldb, 64, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev);
        case F8MI_PLAN_TILES128:
            return launch_gemm_mid(a_fmt, b_fmt, c_dtype, plan.mid == 2, stream, A, lda, 64, B, ldb, 64, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, c_vec_ok);
        case F8MI_PLAN_TILES256_AND_128: {
            const int m1 = (int)(plan.split.rows_large * BM);
            if (int rc = launch_gemm_dma16(a_fmt, b_fmt, c_dtype, dim3((unsigned)(plan.split.rows_large * tiles_n)), stream, A, lda, 64, B, ldb, 64, m1, N, K,
                                           scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)plan.split.rows_large, (int)tiles_n, c_vec_ok))
                return rc;
            return launch_gemm_mid(a_fmt, b_fmt, c_dtype, plan.mid == 2, stream, A + (int64_t)m1 * lda, lda, 64, B, ldb, 64, M - m1, N, K, scale_a_dev,
                                   scale_b_dev, (uint8_t*)c + (int64_t)m1 * ldc * csz, ldc, bias_dev, c_vec_ok);
        }
        case F8MI_PLAN_TILES256:
            return launch_gemm_dma16(a_fmt, b_fmt, c_dtype, g, stream, A, lda, 64, B, ldb, 64, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
        case F8MI_PLAN_TILES256_MFMA32:
            return launch_gemm_dma(a_fmt, b_fmt, c_dtype, g, stream, A, lda, 64, B, ldb, 64, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
        default: break;  // F8MI_PLAN_STAGED
    }
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E4M3FN) return launch_gemm1<0, 0>(aligned, c_dtype, g, stream, A, lda, B, ldb, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
    if (a_fmt == F8MI_E5M2 && b_fmt == F8MI_E4M3FN) return launch_gemm1<1, 0>(aligned, c_dtype, g, stream, A, lda, B, ldb, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
    if (a_fmt == F8MI_E4M3FN && b_fmt == F8MI_E5M2) return launch_gemm1<0, 1>(aligned, c_dtype, g, stream, A, lda, B, ldb, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
    return launch_gemm1<1, 1>(aligned, c_dtype, g, stream, A, lda, B, ldb, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
}

extern "C" int f8mi_gemm_nt_kb(const void* a, int a_fmt, const void* bt, int b_fmt, int64_t m, int64_t n, int64_t k,
                               const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype, int64_t ldc,
                               const void* bias_dev, void* stream_) {
    return f8mi_gemm_nt_kb_ws(a, a_fmt, bt, b_fmt, m, n, k, scale_a_dev, scale_b_dev, c, c_dtype, ldc, bias_dev, nullptr, 0, stream_);
}

extern "C" int f8mi_gemm_nt_kb_ws(const void* a, int a_fmt, const void* bt, int b_fmt, int64_t m, int64_t n, int64_t k,
                                  const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype, int64_t ldc,
                                  const void* bias_dev, void* workspace, int64_t workspace_bytes, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (m < 0 || n < 0 || k < 0 || ldc < n) { set_error("f8mi_gemm_nt_kb: bad shape m=%lld n=%lld k=%lld ldc=%lld", (long long)m, (long long)n, (long long)k, (long long)ldc); return F8MI_ERR_INVALID_ARG; }
    if (a_fmt < 0 || a_fmt > 1 || b_fmt < 0 || b_fmt > 1 || c_dtype < 0 || c_dtype > 2) { set_error("f8mi_gemm_nt_kb: unknown format/dtype code"); return F8MI_ERR_INVALID_ARG; }
    if (k % 64 != 0 || k < 384) { set_error("f8mi_gemm_nt_kb: k-blocked operands need k %% 64 == 0 and k >= 384 (k=%lld)", (long long)k); return F8MI_ERR_UNSUPPORTED; }
    if (m == 0 || n == 0) return F8MI_OK;
    if (!a || !bt || !c || !scale_a_dev || !scale_b_dev) { set_error("f8mi_gemm_nt_kb: null pointer"); return F8MI_ERR_INVALID_ARG; }
    if ((uintptr_t)a % 16 != 0 || (uintptr_t)bt % 16 != 0) { set_error("f8mi_gemm_nt_kb: operands must be 16-byte aligned"); return F8MI_ERR_UNSUPPORTED; }
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff - BK) { set_error("f8mi_gemm_nt_kb: dimension over 2^31"); return F8MI_ERR_UNSUPPORTED; }
    const int64_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7fffffff) { set_error("f8mi_gemm_nt_kb: too many tiles"); return F8MI_ERR_UNSUPPORTED; }
    const int64_t csz = c_dtype == F8MI_FP32 ? 4 : 2;
    const int c_vec_ok = (uintptr_t)c % csz == 0;  // 16-byte stores at element alignment: any row pitch will do
    dim3 g((unsigned)(tiles_m * tiles_n));
    ProfScope prof(F8MI_K_GEMM, 2.0 * (double)m * (double)n * (double)k, stream);
    const uint8_t* A = (const uint8_t*)a;
    const uint8_t* B = (const uint8_t*)bt;
    const int M = (int)m, N = (int)n, K = (int)k;
    const int64_t a_unit = m * 64, b_unit = n * 64;  // bytes between 64-deep blocks
    const bool ws_ok = workspace && (uintptr_t)workspace % 16 == 0;
    const GemmPlan plan = gemm_plan(m, n, k, true, ws_ok ? workspace_bytes : 0);
    switch (plan.kind) {
        case F8MI_PLAN_TILES128_SPLIT_K:
            return launch_gemm_mid_splitk(a_fmt, b_fmt, c_dtype, plan.mid == 2, plan.parts, (float*)workspace, stream, A, 64, a_unit, B, 64, b_unit, M, N, K,
                                          scale_a_dev, scale_b_dev, c, ldc, bias_dev, c_vec_ok);
        case F8MI_PLAN_FEW_ROWS:
            return launch_gemm_skinny(a_fmt, b_fmt, c_dtype, stream, A, 64, a_unit, B, 64, b_unit, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev);
        case F8MI_PLAN_TILES128:
            return launch_gemm_mid(a_fmt, b_fmt, c_dtype, plan.mid == 2, stream, A, 64, a_unit, B, 64, b_unit, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, c_vec_ok);
        case F8MI_PLAN_TILES256_AND_128: {
            // rows m1 .. m of a k-blocked operand start m1 * 64 bytes in; the distance between 64-deep blocks stays m * 64
            const int64_t m1 = plan.split.rows_large * BM;
            if (int rc = launch_gemm_dma16(a_fmt, b_fmt, c_dtype, dim3((unsigned)(plan.split.rows_large * tiles_n)), stream, A, 64, a_unit, B, 64, b_unit,
                                           (int)m1, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)plan.split.rows_large, (int)tiles_n, c_vec_ok))
                return rc;
            return launch_gemm_mid(a_fmt, b_fmt, c_dtype, plan.mid == 2, stream, A + m1 * 64, 64, a_unit, B, 64, b_unit, (int)(m - m1), N, K, scale_a_dev,
                                   scale_b_dev, (uint8_t*)c + m1 * ldc * csz, ldc, bias_dev, c_vec_ok);
        }
        default: break;
    }
    // whole output on 256 x 256 tiles (there is no register-staged kernel for k-blocked operands)
    if (k % 128 == 0)
        return launch_gemm_dma16(a_fmt, b_fmt, c_dtype, g, stream, A, 64, a_unit, B, 64, b_unit, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev,
                                 (int)tiles_m, (int)tiles_n, c_vec_ok);
    return launch_gemm_dma(a_fmt, b_fmt, c_dtype, g, stream, A, 64, a_unit, B, 64, b_unit, M, N, K, scale_a_dev, scale_b_dev, c, ldc, bias_dev,
                           (int)tiles_m, (int)tiles_n, c_vec_ok);
}

extern "C" int f8mi_gemm_kb_ex(const void* a, int a_fmt, int a_transposed, const void* bt, int b_fmt, int b_transposed,
                               int64_t m, int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c,
                               int c_dtype, int64_t ldc, const void* bias_dev, void* stream_) {
    if (!a_transposed && !b_transposed)
        return f8mi_gemm_nt_kb(a, a_fmt, bt, b_fmt, m, n, k, scale_a_dev, scale_b_dev, c, c_dtype, ldc, bias_dev, stream_);
    hipStream_t stream = (hipStream_t)stream_;
    if (a_transposed && !b_transposed) { set_error("f8mi_gemm_kb_ex: a transposed with bt not transposed is not built (swap the operands and transpose c)"); return F8MI_ERR_UNSUPPORTED; }
    if (m < 0 || n < 0 || k < 0 || ldc < n) { set_error("f8mi_gemm_kb_ex: bad shape m=%lld n=%lld k=%lld ldc=%lld", (long long)m, (long long)n, (long long)k, (long long)ldc); return F8MI_ERR_INVALID_ARG; }
    if (a_fmt < 0 || a_fmt > 1 || b_fmt < 0 || b_fmt > 1 || c_dtype < 0 || c_dtype > 2) { set_error("f8mi_gemm_kb_ex: unknown format/dtype code"); return F8MI_ERR_INVALID_ARG; }
    if (k % 128 != 0 || k < 384) { set_error("f8mi_gemm_kb_ex: transposed operands need k %% 128 == 0 and k >= 384 (k=%lld)", (long long)k); return F8MI_ERR_UNSUPPORTED; }
    if (n % 64 != 0 || (a_transposed && m % 64 != 0)) { set_error("f8mi_gemm_kb_ex: a transposed operand needs its row count to be a multiple of 64 (m=%lld n=%lld)", (long long)m, (long long)n); return F8MI_ERR_UNSUPPORTED; }
    if (m == 0 || n == 0) return F8MI_OK;
    if (!a || !bt || !c || !scale_a_dev || !scale_b_dev) { set_error("f8mi_gemm_kb_ex: null pointer"); return F8MI_ERR_INVALID_ARG; }
    if ((uintptr_t)a % 16 != 0 || (uintptr_t)bt % 16 != 0) { set_error("f8mi_gemm_kb_ex: operands must be 16-byte aligned"); return F8MI_ERR_UNSUPPORTED; }
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff - BK || k * 64 * 4 > 0x7fffffffLL) { set_error("f8mi_gemm_kb_ex: dimension too large"); return F8MI_ERR_UNSUPPORTED; }
    const int64_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7fffffff) { set_error("f8mi_gemm_kb_ex: too many tiles"); return F8MI_ERR_UNSUPPORTED; }
    const int64_t csz = c_dtype == F8MI_FP32 ? 4 : 2;
    const int c_vec_ok = (uintptr_t)c % csz == 0;  // 16-byte stores at element alignment: any row pitch will do
    dim3 g((unsigned)(tiles_m * tiles_n));
    ProfScope prof(F8MI_K_GEMM, 2.0 * (double)m * (double)n * (double)k, stream);
    // a transposed operand: 64 bytes between contraction rows, k * 64 between blocks of 64 rows
    if (a_transposed)
        return launch_gemm_dma16_tt(a_fmt, b_fmt, c_dtype, g, stream, (const uint8_t*)a, 64, k * 64, (const uint8_t*)bt, 64, k * 64, (int)m, (int)n,
                                    (int)k, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
    return launch_gemm_dma16_nt(a_fmt, b_fmt, c_dtype, g, stream, (const uint8_t*)a, 64, m * 64, (const uint8_t*)bt, 64, k * 64, (int)m, (int)n,
                                (int)k, scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
}

extern "C" int f8mi_gemm_ex(const void* a, int a_fmt, int a_transposed, int64_t lda, const void* bt, int b_fmt, int b_transposed, int64_t ldb,
                            int64_t m, int64_t n, int64_t k, const float* scale_a_dev, const float* scale_b_dev, void* c, int c_dtype,
                            int64_t ldc, const void* bias_dev, void* stream_) {
    if (!a_transposed && !b_transposed)
        return f8mi_gemm_nt(a, a_fmt, lda, bt, b_fmt, ldb, m, n, k, scale_a_dev, scale_b_dev, c, c_dtype, ldc, bias_dev, stream_);
    hipStream_t stream = (hipStream_t)stream_;
    if (a_transposed && !b_transposed) { set_error("f8mi_gemm_ex: a transposed with bt not transposed is not built (copy a, or swap the operands and transpose c)"); return F8MI_ERR_UNSUPPORTED; }
    if (m < 0 || n < 0 || k < 0 || ldc < n || lda < (a_transposed ? m : k) || ldb < n) { set_error("f8mi_gemm_ex: bad shape m=%lld n=%lld k=%lld lda=%lld ldb=%lld ldc=%lld", (long long)m, (long long)n, (long long)k, (long long)lda, (long long)ldb, (long long)ldc); return F8MI_ERR_INVALID_ARG; }
    if (a_fmt < 0 || a_fmt > 1 || b_fmt < 0 || b_fmt > 1 || c_dtype < 0 || c_dtype > 2) { set_error("f8mi_gemm_ex: unknown format/dtype code"); return F8MI_ERR_INVALID_ARG; }
    if (m == 0 || n == 0) return F8MI_OK;
    if (!a || !bt || !c || !scale_a_dev || !scale_b_dev) { set_error("f8mi_gemm_ex: null pointer"); return F8MI_ERR_INVALID_ARG; }
    // what the kernels that read an operand transposed need; anything else is for the caller to copy
    if (k % 128 != 0 || k < 384) { set_error("f8mi_gemm_ex: transposed operands need k %% 128 == 0 and k >= 384 (k=%lld)", (long long)k); return F8MI_ERR_UNSUPPORTED; }
    if (n % 64 != 0 || (a_transposed && m % 64 != 0)) { set_error("f8mi_gemm_ex: a transposed operand needs its row count to be a multiple of 64 (m=%lld n=%lld)", (long long)m, (long long)n); return F8MI_ERR_UNSUPPORTED; }
    if ((uintptr_t)a % 16 != 0 || (uintptr_t)bt % 16 != 0 || lda % 16 != 0 || ldb % 16 != 0) { set_error("f8mi_gemm_ex: transposed operands need 16-byte aligned addresses and row strides"); return F8MI_ERR_UNSUPPORTED; }
    if (((m + 127) / 128) * ((n + 127) / 128) <= 256) { set_error("f8mi_gemm_ex: an output of at most 256 tiles of 128 x 128 is faster from transposed copies (128-row tiles read no operand transposed)"); return F8MI_ERR_UNSUPPORTED; }
    // 32-bit offsets inside a step: 128 contraction rows of a transposed operand, 256 rows of a normal one
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff - BK || 128 * ldb + 256 > 0x7fffffffLL || (a_transposed ? 128 * lda + 256 : lda * (BM - 1) + k + BK) > 0x7fffffffLL) { set_error("f8mi_gemm_ex: dimension or row stride too large"); return F8MI_ERR_UNSUPPORTED; }
    const int64_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7fffffff) { set_error("f8mi_gemm_ex: too many tiles"); return F8MI_ERR_UNSUPPORTED; }
    const int64_t csz = c_dtype == F8MI_FP32 ? 4 : 2;
    const int c_vec_ok = (uintptr_t)c % csz == 0;
    dim3 g((unsigned)(tiles_m * tiles_n));
    ProfScope prof(F8MI_K_GEMM, 2.0 * (double)m * (double)n * (double)k, stream);
    // a row-major matrix read transposed: row stride between contraction rows, 64 bytes between blocks of 64 rows
    if (a_transposed)
        return launch_gemm_dma16_tt(a_fmt, b_fmt, c_dtype, g, stream, (const uint8_t*)a, lda, 64, (const uint8_t*)bt, ldb, 64, (int)m, (int)n, (int)k,
                                    scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
    return launch_gemm_dma16_nt(a_fmt, b_fmt, c_dtype, g, stream, (const uint8_t*)a, lda, 64, (const uint8_t*)bt, ldb, 64, (int)m, (int)n, (int)k,
                                scale_a_dev, scale_b_dev, c, ldc, bias_dev, (int)tiles_m, (int)tiles_n, c_vec_ok);
}
