// K2 / K2d: saturated fp8 cast, with the transposed copy and (optionally) the
// tensor's amax fused into the same pass.  HBM-bound: reads sizeof(T) bytes and
// writes 1 byte per element and per fp8 output.
//
// A workgroup of 256 lanes owns a 128 x 128 tile.  Lane t covers columns
// 8*(t%16) .. +7 of rows 64*h + 4*(t/16) .. +3 for h = 0, 1: eight 16-byte loads
// (bf16/fp16; sixteen for fp32), all issued before the first use.  The row-major
// fp8 tile goes out straight from registers as 8-byte stores (16 lanes = one
// 128-byte row segment).  For the transposed copy each lane transposes its
// 4 x 8 byte block in registers (v_perm), parks the 4-row dwords in a
// 128 x 128-byte LDS tile whose dword index is XOR-swizzled by the column group
// (so the 64 lanes of a store hit 32 banks twice: the floor for 256 bytes), and
// the tile is read back as 16-byte row pieces: 8 lanes = one 128-byte segment of
// a row of the transposed output.
#include <atomic>

#include "f8mi_common.h"

namespace f8mi {

// The fp8 bytes leave as 8-byte (row-major copy) and 16-byte (transposed copy) stores at whatever alignment the
// output's row pitch gives them.
__device__ __forceinline__ void store8(uint8_t* p, uint32_t lo, uint32_t hi) {
#if F8MI_CAST_NT_STORES
    __builtin_nontemporal_store((u32x2){lo, hi}, (u32x2_any*)p);
#else
    store8_any(p, lo, hi);
#endif
}
__device__ __forceinline__ void store16(uint8_t* p, uint4 v) {
#if F8MI_CAST_NT_STORES
    __builtin_nontemporal_store((u32x4){v.x, v.y, v.z, v.w}, (u32x4_any*)p);
#else
    store16_any(p, v);
#endif
}

constexpr int CAST_THREADS = 256;
constexpr int SPREAD_WORDS = 1024;  // words of the delayed-scaling workspace (f8mi_delayed_workspace_bytes)
constexpr int CAST_TILE = 128;
constexpr int CAST_GROUP = 8;

// Fused amax of the cast kernel, without a workspace: *amax_out was zeroed by a tiny kernel launched just before, and holds the
// running maximum as an fp32 bit pattern (non-negative floats and NaNs order like unsigned integers).
// No ticket and, for all but a handful of blocks, no atomic at all: the value only grows, so a block whose
// maximum is not above a (possibly stale) read of it has nothing to add.  (Reducing and reading the word early, right
// after the loads, so that the round trip overlaps the conversion, was 20 % slower: the barrier it needs in the
// middle of the block makes all four waves wait for the slowest one's loads before any of them converts.)
__device__ __forceinline__ void publish_amax_cast(uint32_t blockmax, float* amax_out, int in_dt) {
    if (threadIdx.x == 0) {
        const uint32_t bits = __float_as_uint(abs_bits_to_float(blockmax, in_dt));
        uint32_t* dst = (uint32_t*)amax_out;
        if (bits > __atomic_load_n(dst, __ATOMIC_RELAXED)) atomicMax(dst, bits);
    }
}

// clamp to [-fmax, fmax], NaN kept (v_med3_f32 drops it, so it is put back)
__device__ __forceinline__ float clamp_keep_nan(float y, float fmax) {
    const float c = __builtin_amdgcn_fmed3f(y, -fmax, fmax);
    return (y != y) ? y : c;
}

// Two adjacent elements: x*scale rounded to PROD, clamped, as fp32 ready for conversion.
template <int PROD>
__device__ __forceinline__ void scale_clamp2(float x0, float x1, float scale, float fmax, float& y0, float& y1) {
    float p0 = __fmul_rn(x0, scale), p1 = __fmul_rn(x1, scale);
    if constexpr (PROD == F8MI_BF16) {
        const uint32_t w = pack_bf16x2(p0, p1);
        p0 = __uint_as_float(w << 16);
        p1 = __uint_as_float(w & 0xffff0000u);
    } else if constexpr (PROD == F8MI_FP16) {
        p0 = round_to_fp16(p0);
        p1 = round_to_fp16(p1);
    }
    y0 = clamp_keep_nan(p0, fmax);
    y1 = clamp_keep_nan(p1, fmax);
}

// 4 dwords (rows 0..3, 4 bytes each = columns 0..3) -> 4 dwords (column c: rows 0..3)
__device__ __forceinline__ void transpose4x4_bytes(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t& c0,
                                                   uint32_t& c1, uint32_t& c2, uint32_t& c3) {
    // v_perm_b32(hi, lo, sel): byte i of the result = byte sel[i] of the 8-byte {hi,lo} (lo = bytes 0..3)
    uint32_t a = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
    uint32_t b = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
    uint32_t c = __builtin_amdgcn_perm(r3, r2, 0x05010400u);  // r2.b0 r3.b0 r2.b1 r3.b1
    uint32_t d = __builtin_amdgcn_perm(r3, r2, 0x07030602u);  // r2.b2 r3.b2 r2.b3 r3.b3
    c0 = __builtin_amdgcn_perm(c, a, 0x05040100u);            // a.b0 a.b1 c.b0 c.b1
    c1 = __builtin_amdgcn_perm(c, a, 0x07060302u);            // a.b2 a.b3 c.b2 c.b3
    c2 = __builtin_amdgcn_perm(d, b, 0x05040100u);
    c3 = __builtin_amdgcn_perm(d, b, 0x07060302u);
}

template <int DT>
struct Row8 {  // eight consecutive elements of one row, widened to fp32 on demand
    uint32_t w[DT == F8MI_FP32 ? 8 : 4];
};

template <int DT>
__device__ __forceinline__ float elem(const Row8<DT>& r, int i) {
    if constexpr (DT == F8MI_FP32) return __uint_as_float(r.w[i]);
    else {
        uint32_t h = (i & 1) ? (r.w[i >> 1] >> 16) : (r.w[i >> 1] & 0xffffu);
        if constexpr (DT == F8MI_BF16) return bf16_bits_to_float(h);
        else return fp16_bits_to_float(h);
    }
}

// Folds the eight elements of a row into a running maximum.  16-bit types: `m` holds two 16-bit maxima side by side
// (see absmax16x2); absmax_done merges them.
template <int DT>
__device__ __forceinline__ uint32_t absmax_row(const Row8<DT>& r, uint32_t m) {
    if constexpr (DT == F8MI_FP32) {
#pragma unroll
        for (int i = 0; i < 8; i++) { uint32_t a = r.w[i] & 0x7fffffffu; m = m > a ? m : a; }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) m = absmax16x2(r.w[i], m);
    }
    return m;
}
template <int DT>
__device__ __forceinline__ uint32_t absmax_done(uint32_t m) {
    if constexpr (DT == F8MI_FP32) return m;
    else return fold16(m);
}

// Loads 8 elements of row `row` starting at column `col`; out-of-range elements read as +0.  Eight elements inside the
// row are one 16-byte load (two for fp32) whatever the row pitch: a row only has to start at a multiple of the
// element size.
template <int DT>
__device__ __forceinline__ void load_row8(Row8<DT>& r, const void* x, int64_t row, int64_t col, int64_t rows,
                                          int64_t cols, int64_t ld) {
    constexpr int ESZ = DT == F8MI_FP32 ? 4 : 2;
    constexpr int NW = DT == F8MI_FP32 ? 8 : 4;
#pragma unroll
    for (int i = 0; i < NW; i++) r.w[i] = 0u;
    if (row >= rows || col >= cols) return;
    const char* p = (const char*)x + (row * ld + col) * ESZ;
    if (col + 8 <= cols) {
        uint4 v0 = load_nt16_any(p);
        r.w[0] = v0.x; r.w[1] = v0.y; r.w[2] = v0.z; r.w[3] = v0.w;
        if constexpr (DT == F8MI_FP32) {
            uint4 v1 = load_nt16_any(p + 16);
            r.w[4] = v1.x; r.w[5] = v1.y; r.w[6] = v1.z; r.w[7] = v1.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (col + i < cols) {
                if constexpr (DT == F8MI_FP32) r.w[i] = ((const uint32_t*)p)[i];
                else r.w[i >> 1] |= (uint32_t)((const uint16_t*)p)[i] << ((i & 1) * 16);
            }
        }
    }
}

// out_kb / out_t_kb: F8MI_LAYOUT_* code of the respective output.
template <int DT, int PROD, int FMT>
__global__ __launch_bounds__(CAST_THREADS) void cast_kernel(const void* __restrict__ x, int64_t rows, int64_t cols,
                                                            int64_t ld, const float* __restrict__ scale_dev,
                                                            uint8_t* __restrict__ out, uint8_t* __restrict__ out_t,
                                                            float* amax_out, int64_t tiles_x, int64_t tiles_y,
                                                            int out_kb, int out_t_kb, const uint32_t* __restrict__ amax_ws,
                                                            int amax_nblocks, float* scale_out, uint32_t* amax_spread) {
    __shared__ uint32_t tileT[CAST_TILE * CAST_TILE / 4];  // [column][row/4] dwords, swizzled
    __shared__ uint32_t red[CAST_THREADS / 64];

    const int t = threadIdx.x;
    const int a = t & 15;   // column group: columns 8a .. 8a+7 of the tile
    const int b = t >> 4;   // row group: rows 4b .. 4b+3 of each 64-row half
    // Tiles are walked in bands of CAST_GROUP tile rows and, inside a band, in groups of CAST_GROUP tile
    // columns: the blocks in flight then read 2 KB runs of each input row and write 1 KB runs of each
    // transposed row, instead of one of the two walking through memory with a huge stride.
    int ty, tx;
    {
        // Consecutive workgroup ids go to the 8 XCDs round-robin; re-deal them so that one XCD (one L2) gets whole
        // groups of 64 neighbouring tiles (an 8 x 8 supertile where the tile grid divides evenly) and can merge
        // their adjacent output segments, while consecutive groups go to consecutive XCDs: the workgroups in flight
        // on the whole chip then cover ONE contiguous stretch of the tensor that advances through memory.  (Giving
        // each XCD its own eighth of the tensor instead, eight fronts far apart, measured 5 % slower in the
        // benchmark step: 5.36 -> 5.63 TB/s; up to 20 % on tensors below 300 MB.)
        int64_t bid = blockIdx.x;
        const int64_t nb = gridDim.x, nb_full = nb - nb % 512;  // ids past the last whole round of 8 groups stay
        if (bid < nb_full) {
            const int64_t xcd = bid % 8, j = bid / 8;
            bid = ((j / 64) * 8 + xcd) * 64 + (j % 64);
        }
#if F8MI_CAST_REVERSE_WALK  // measurement builds only: last tiles first, the reverse of the order the amax pass read in
        bid = nb - 1 - bid;
#endif
        const int64_t band = bid / ((int64_t)CAST_GROUP * tiles_x);
        const int64_t rem = bid - band * CAST_GROUP * tiles_x;
        const int rows_in_band = (int)min((int64_t)CAST_GROUP, tiles_y - band * CAST_GROUP);
        const int64_t gcol = rem / ((int64_t)rows_in_band * CAST_GROUP);
        const int64_t r2 = rem - gcol * rows_in_band * CAST_GROUP;
        const int cols_in_g = (int)min((int64_t)CAST_GROUP, tiles_x - gcol * CAST_GROUP);
        ty = (int)(band * CAST_GROUP + r2 / cols_in_g);
        tx = (int)(gcol * CAST_GROUP + r2 % cols_in_g);
    }
    const int64_t r0 = (int64_t)ty * CAST_TILE;
    const int64_t c0 = (int64_t)tx * CAST_TILE;
    const int64_t col = c0 + 8 * a;

    // dynamic scaling: the amax kernel's per-workgroup maxima (at most WS_WORDS = 4 x 64 lanes x 4 words), requested
    // ahead of the tile so that they arrive first.  Every wave fetches all of them: no LDS, no barrier.
    static_assert(WS_WORDS <= 4 * 64 * 4, "four 16-byte loads per lane cover the workspace");
    uint4 ws_words[4];
    if (amax_ws) {
#pragma unroll
        for (int q = 0; q < 4; q++)
            ws_words[q] = q * 256 < amax_nblocks ? ((const uint4*)amax_ws)[q * 64 + (t & 63)] : make_uint4(0u, 0u, 0u, 0u);
    }

    Row8<DT> in[2][4];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int j = 0; j < 4; j++) load_row8<DT>(in[h][j], x, r0 + 64 * h + 4 * b + j, col, rows, cols, ld);

    // The scale: given -- or, for dynamic scaling, derived here from the per-workgroup maxima the amax kernel left in
    // amax_ws (every wave of every workgroup reduces the <= 1024 words itself; saves the one-block launch that would do
    // it once).  The words were requested before the tile and nothing here waits for anybody else, so the reduction
    // runs while the tile's loads are still in flight.  (A first version shared the work among the four waves through
    // LDS: its two barriers, in the middle of the block, cost more than the redundant loads do.)  Words past
    // amax_nblocks are leftovers of an earlier, larger call and are masked.  Same arithmetic as amax_finalize_kernel,
    // in the tensor's dtype.
    float scale;
    if (amax_ws) {
        uint32_t wm = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int first = q * 256 + (t & 63) * 4;
            const uint32_t w[4] = {ws_words[q].x, ws_words[q].y, ws_words[q].z, ws_words[q].w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint32_t v = first + c < amax_nblocks ? w[c] : 0u;
                wm = wm > v ? wm : v;
            }
        }
        wm = wave_max_u32(wm);
        scale = amax_to_scale_dev(abs_bits_to_float(wm, DT), DT, FMT, DT == F8MI_FP16);
        if (blockIdx.x == 0 && t == 0) *scale_out = scale;
    } else {
        scale = *scale_dev;
    }
    constexpr float fmax = FMT == F8MI_E4M3FN ? 448.0f : 57344.0f;

    uint32_t m = 0;
    if (amax_out) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int j = 0; j < 4; j++) m = absmax_row<DT>(in[h][j], m);
        m = absmax_done<DT>(m);
    }

    // Zero-padded k-blocked outputs (F8MI_LAYOUT_KBLOCK64_PAD128): the tile grid ends exactly where the padding does, so
    // a tile writes all of its 128 columns (`out`) or rows (`out_t`); what lies past the tensor's edge is forced to
    // zero bytes (elements read as +0 would become NaN codes under a NaN scale).
    const bool pad = out_kb == F8MI_LAYOUT_KBLOCK64_PAD128 || out_t_kb == F8MI_LAYOUT_KBLOCK64_PAD128;
    uint32_t keep_lo = 0xffffffffu, keep_hi = 0xffffffffu;  // bytes of the lane's eight columns that lie inside the row
    if (pad && col + 8 > cols) {
        const int valid = col < cols ? (int)(cols - col) : 0;
        keep_lo = valid >= 4 ? 0xffffffffu : (valid ? (1u << (8 * valid)) - 1u : 0u);
        keep_hi = valid > 4 ? (1u << (8 * (valid - 4))) - 1u : 0u;
    }
#pragma unroll
    for (int h = 0; h < 2; h++) {
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float f[8];
#pragma unroll
            for (int i = 0; i < 8; i += 2)
                scale_clamp2<PROD>(elem<DT>(in[h][j], i), elem<DT>(in[h][j], i + 1), scale, fmax, f[i], f[i + 1]);
            lo[j] = cvt4_fp8<FMT>(f[0], f[1], f[2], f[3]);
            hi[j] = cvt4_fp8<FMT>(f[4], f[5], f[6], f[7]);
            const int64_t row = r0 + 64 * h + 4 * b + j;
            if (pad) {
                lo[j] = row < rows ? lo[j] & keep_lo : 0u;
                hi[j] = row < rows ? hi[j] & keep_hi : 0u;
            }
            if (out && row < rows && (col < cols || out_kb == F8MI_LAYOUT_KBLOCK64_PAD128)) {
                // k-blocked: [cols/64][rows][64] (cols % 64 == 0 or padded to it: the eight columns are always whole)
                uint8_t* p = out_kb ? out + ((col >> 6) * rows + row) * 64 + (col & 63) : out + row * cols + col;
                if (out_kb || col + 8 <= cols) {
                    store8(p, lo[j], hi[j]);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i++)
                        if (col + i < cols) p[i] = (uint8_t)((i < 4 ? lo[j] >> (8 * i) : hi[j] >> (8 * (i - 4))) & 0xffu);
                }
            }
        }
        if (out_t) {
            uint32_t tc[8];
            transpose4x4_bytes(lo[0], lo[1], lo[2], lo[3], tc[0], tc[1], tc[2], tc[3]);
            transpose4x4_bytes(hi[0], hi[1], hi[2], hi[3], tc[4], tc[5], tc[6], tc[7]);
            const int d = 16 * h + b;              // dword index (rows 4d .. 4d+3) within a tile column
            const int dsw = d ^ ((a & 7) << 2);    // swizzle by column group
#pragma unroll
            for (int cc = 0; cc < 8; cc++) tileT[(8 * a + cc) * (CAST_TILE / 4) + dsw] = tc[cc];
        }
    }

    if (out_t) {
        __syncthreads();
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const int id = p * CAST_THREADS + t;
            const int c = id >> 3, q = id & 7;  // tile column c (a row of out_t), 16-byte piece q
            const int qsw = q ^ ((c >> 3) & 7);
            const uint4 v = *(const uint4*)&tileT[c * (CAST_TILE / 4) + 4 * qsw];
            const int64_t gc = c0 + c;
            const int64_t gr = r0 + 16 * q;
            if (gc < cols && (gr < rows || out_t_kb == F8MI_LAYOUT_KBLOCK64_PAD128)) {
                // k-blocked: [rows/64][cols][64] (rows % 64 == 0 or padded to it: the sixteen rows are always whole)
                uint8_t* dst = out_t_kb ? out_t + ((gr >> 6) * cols + gc) * 64 + (gr & 63) : out_t + gc * rows + gr;
                if (out_t_kb || gr + 16 <= rows) {
                    store16(dst, v);
                } else {
                    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int i = 0; i < 16; i++)
                        if (gr + i < rows) dst[i] = (uint8_t)((w[i >> 2] >> (8 * (i & 3))) & 0xffu);
                }
            }
        }
    }

    if (amax_out && amax_spread) {
        // Every wave folds its maximum (the bit pattern in the input's dtype) into one of SPREAD_WORDS words with an
        // atomic that returns nothing: no LDS, no barrier, no round trip to wait for, and a word sees about one atomic
        // per (tiles * 4 / SPREAD_WORDS) waves, spread over the whole run of the kernel.  cast_spread_finalize_kernel
        // turns the words into *amax_out.  (Measured per tensor of the benchmark, 128 MB .. 1.8 GB, against the cast
        // without amax: folding into *amax_out itself, one compare-and-atomic per workgroup at its end as below, +6 ..
        // +20 us -- the workgroup holds its LDS and wave slots for the round trip of that last read; this + 0 .. 2 us,
        // plus 4 us for the finalize launch.)
        m = wave_max_u32(m);
        if ((t & 63) == 0 && m)
            (void)__hip_atomic_fetch_max(&amax_spread[(blockIdx.x * (CAST_THREADS / 64) + (t >> 6)) & (SPREAD_WORDS - 1)], m,
                                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if (amax_out) {
        m = wave_max_u32(m);
        const int wave = t >> 6, lane = t & 63;
        if (lane == 0) red[wave] = m;
        __syncthreads();
        if (wave == 0) {
            uint32_t v = lane < CAST_THREADS / 64 ? red[lane] : 0u;
            m = wave_max_u32(v);
        }
        publish_amax_cast(m, amax_out, DT);
    }
}

// Dynamic scaling of a small tensor in ONE launch: amax, scale and cast by a single workgroup that holds the whole
// tensor in registers (at most four items of eight elements per lane, loaded back to back).  Same arithmetic,
// element for element, as amax kernel + cast kernel; it exists because three or four launches cost more than
// the work when the tensor is a few rows of activations.
constexpr int SMALL_THREADS = 1024;
constexpr int SMALL_ITEMS_PER_THREAD = 4;
constexpr int64_t SMALL_MAX_ITEMS = (int64_t)SMALL_THREADS * SMALL_ITEMS_PER_THREAD;  // 32 K elements: 64 KB of bf16

template <int DT, int FMT>
__global__ __launch_bounds__(SMALL_THREADS) void cast_dynamic_small_kernel(const void* __restrict__ x, int64_t rows, int64_t cols,
                                                                           int64_t ld, float* __restrict__ scale_out,
                                                                           uint8_t* __restrict__ out, uint8_t* __restrict__ out_t,
                                                                           int out_kb, int out_t_kb) {
    __shared__ uint32_t red[SMALL_THREADS / 64];
    __shared__ uint32_t amax_bits;
    const int t = threadIdx.x;
    const int64_t groups = (cols + 7) / 8, items = rows * groups;  // an item: eight consecutive elements of a row
    Row8<DT> r[SMALL_ITEMS_PER_THREAD];
    uint32_t m = 0;
#pragma unroll
    for (int u = 0; u < SMALL_ITEMS_PER_THREAD; u++) {
        const int64_t it = t + (int64_t)u * SMALL_THREADS;
        // past the last item: row == rows, which load_row8 reads as zeros
        load_row8<DT>(r[u], x, it < items ? it / groups : rows, (it % groups) * 8, rows, cols, ld);
    }
#pragma unroll
    for (int u = 0; u < SMALL_ITEMS_PER_THREAD; u++) m = absmax_row<DT>(r[u], m);
    m = wave_max_u32(absmax_done<DT>(m));
    if ((t & 63) == 0) red[t >> 6] = m;
    __syncthreads();
    if (t < 64) {
        uint32_t v = t < SMALL_THREADS / 64 ? red[t] : 0u;
        v = wave_max_u32(v);
        if (t == 0) amax_bits = v;
    }
    __syncthreads();
    // the scale in the tensor's own dtype, as tensor_to_scale computes it (fp16 tensors: clamped to 65504)
    const float scale = amax_to_scale_dev(abs_bits_to_float(amax_bits, DT), DT, FMT, DT == F8MI_FP16);
    if (t == 0) *scale_out = scale;
    constexpr float fmax = FMT == F8MI_E4M3FN ? 448.0f : 57344.0f;
#pragma unroll
    for (int u = 0; u < SMALL_ITEMS_PER_THREAD; u++) {
        const int64_t it = t + (int64_t)u * SMALL_THREADS;
        if (it >= items) continue;
        const int64_t row = it / groups, col = (it % groups) * 8;
        float f[8];
#pragma unroll
        for (int i = 0; i < 8; i += 2) scale_clamp2<DT>(elem<DT>(r[u], i), elem<DT>(r[u], i + 1), scale, fmax, f[i], f[i + 1]);
        const uint32_t lo = cvt4_fp8<FMT>(f[0], f[1], f[2], f[3]), hi = cvt4_fp8<FMT>(f[4], f[5], f[6], f[7]);
        if (out) {
            uint8_t* p = out_kb ? out + ((col >> 6) * rows + row) * 64 + (col & 63) : out + row * cols + col;
            if (col + 8 <= cols) {
                store8_any(p, lo, hi);
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (col + i < cols) p[i] = (uint8_t)((i < 4 ? lo >> (8 * i) : hi >> (8 * (i - 4))) & 0xffu);
            }
        }
        if (out_t) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int64_t c = col + i;
                if (c < cols) {
                    uint8_t* p = out_t_kb ? out_t + ((row >> 6) * cols + c) * 64 + (row & 63) : out_t + c * rows + row;
                    *p = (uint8_t)((i < 4 ? lo >> (8 * i) : hi >> (8 * (i - 4))) & 0xffu);
                }
            }
        }
    }
}

template <int DT>
static int launch_cast_small(int fmt, hipStream_t stream, const void* x, int64_t rows, int64_t cols, int64_t ld,
                             float* scale_dev, uint8_t* out, uint8_t* out_t, int out_kb, int out_t_kb) {
    const dim3 g(1), b(SMALL_THREADS);
    if (fmt == F8MI_E4M3FN) hipLaunchKernelGGL((cast_dynamic_small_kernel<DT, F8MI_E4M3FN>), g, b, 0, stream, x, rows, cols, ld, scale_dev, out, out_t, out_kb, out_t_kb);
    else hipLaunchKernelGGL((cast_dynamic_small_kernel<DT, F8MI_E5M2>), g, b, 0, stream, x, rows, cols, ld, scale_dev, out, out_t, out_kb, out_t_kb);
    return check_hip(hipGetLastError(), "cast (dynamic, one workgroup) kernel launch");
}

// where a dynamic-scaling cast takes its scale from (see cast_layout_impl)
struct AmaxSource {
    const uint32_t* ws;
    int nblocks;
    float* scale_out;
    uint32_t* spread;  // delayed scaling: the zeroed words the fused amax is folded into (null: straight into *amax_dev)
};

__global__ void cast_zero_amax_kernel(float* amax_out) {
    if (threadIdx.x == 0) *amax_out = 0.0f;
}

// Second half of the fused amax with a workspace: the maximum of the SPREAD_WORDS words becomes *amax_out (widened to
// fp32) and every word goes back to zero, which is the state the next call expects.  One workgroup.
__global__ __launch_bounds__(SPREAD_WORDS) void cast_spread_finalize_kernel(uint32_t* __restrict__ spread, float* __restrict__ amax_out, int in_dt) {
    __shared__ uint32_t red[SPREAD_WORDS / 64];
    uint32_t m = spread[threadIdx.x];
    if (m) spread[threadIdx.x] = 0u;
    m = wave_max_u32(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x < 64) {
        m = wave_max_u32(threadIdx.x < SPREAD_WORDS / 64 ? red[threadIdx.x] : 0u);
        if (threadIdx.x == 0) *amax_out = abs_bits_to_float(m, in_dt);
    }
}

template <int DT, int PROD, int FMT>
static int launch_cast2(dim3 g, hipStream_t stream, const void* x, int64_t rows, int64_t cols, int64_t ld,
                        const float* scale_dev, uint8_t* out, uint8_t* out_t, float* amax_dev, int64_t tiles_x, int64_t tiles_y, int out_kb, int out_t_kb,
                        const AmaxSource& src) {
    hipLaunchKernelGGL((cast_kernel<DT, PROD, FMT>), g, dim3(CAST_THREADS), 0, stream, x, rows, cols, ld, scale_dev, out, out_t, amax_dev, tiles_x, tiles_y, out_kb, out_t_kb, src.ws, src.nblocks, src.scale_out, src.spread);
    return check_hip(hipGetLastError(), "cast kernel launch");
}

template <int DT, int PROD>
static int launch_cast1(int fmt, dim3 g, hipStream_t stream, const void* x, int64_t rows, int64_t cols,
                        int64_t ld, const float* scale_dev, uint8_t* out, uint8_t* out_t, float* amax_dev,
                        int64_t tiles_x, int64_t tiles_y, int out_kb, int out_t_kb, const AmaxSource& src) {
    if (fmt == F8MI_E4M3FN) return launch_cast2<DT, PROD, F8MI_E4M3FN>(g, stream, x, rows, cols, ld, scale_dev, out, out_t, amax_dev, tiles_x, tiles_y, out_kb, out_t_kb, src);
    return launch_cast2<DT, PROD, F8MI_E5M2>(g, stream, x, rows, cols, ld, scale_dev, out, out_t, amax_dev, tiles_x, tiles_y, out_kb, out_t_kb, src);
}

// Validates and launches the cast.  `src.ws` null: the scale is read from scale_dev (f8mi_cast_layout).  Not null
// (dynamic scaling, product in the input's dtype): the kernel derives the scale from the src.nblocks per-workgroup
// maxima in src.ws and workgroup 0 stores it to src.scale_out.
static int cast_layout_impl(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, const float* scale_dev,
                            int product_dtype, int fp8_fmt, uint8_t* out, int out_layout, uint8_t* out_t, int out_t_layout,
                            float* amax_dev, hipStream_t stream, const AmaxSource& src) {
    if (out_layout < F8MI_LAYOUT_ROWMAJOR || out_layout > F8MI_LAYOUT_KBLOCK64_PAD128 || out_t_layout < F8MI_LAYOUT_ROWMAJOR || out_t_layout > F8MI_LAYOUT_KBLOCK64_PAD128) { set_error("f8mi_cast: unknown layout code"); return F8MI_ERR_INVALID_ARG; }
    if (out && out_layout == F8MI_LAYOUT_KBLOCK64 && cols % 64 != 0) { set_error("f8mi_cast: k-blocked `out` needs cols %% 64 == 0 (cols=%lld); F8MI_LAYOUT_KBLOCK64_PAD128 takes any", (long long)cols); return F8MI_ERR_UNSUPPORTED; }
    if (out_t && out_t_layout == F8MI_LAYOUT_KBLOCK64 && rows % 64 != 0) { set_error("f8mi_cast: k-blocked `out_t` needs rows %% 64 == 0 (rows=%lld); F8MI_LAYOUT_KBLOCK64_PAD128 takes any", (long long)rows); return F8MI_ERR_UNSUPPORTED; }
    // the kernel takes the layout codes as they are (0: row-major, otherwise k-blocked; PAD128: whole tiles are written)
    const int out_kb = out ? out_layout : F8MI_LAYOUT_ROWMAJOR, out_t_kb = out_t ? out_t_layout : F8MI_LAYOUT_ROWMAJOR;
    // ld == 0: every row reads the same `cols` elements (the kernels address row * ld + col)
    if (rows < 0 || cols < 0 || (ld < cols && ld != 0)) { set_error("f8mi_cast: bad shape rows=%lld cols=%lld ld=%lld", (long long)rows, (long long)cols, (long long)ld); return F8MI_ERR_INVALID_ARG; }
    if (in_dtype < 0 || in_dtype > 2 || fp8_fmt < 0 || fp8_fmt > 1) { set_error("f8mi_cast: unknown dtype/format code"); return F8MI_ERR_INVALID_ARG; }
    if (product_dtype != in_dtype && product_dtype != F8MI_FP32) { set_error("f8mi_cast: product_dtype must be the input dtype or fp32"); return F8MI_ERR_INVALID_ARG; }
    if (!scale_dev && !src.ws) { set_error("f8mi_cast: null scale"); return F8MI_ERR_INVALID_ARG; }
    if (!out && !out_t && !amax_dev) { set_error("f8mi_cast: no output requested"); return F8MI_ERR_INVALID_ARG; }
    if (rows == 0 || cols == 0) {
        if (amax_dev) {
            hipLaunchKernelGGL(cast_zero_amax_kernel, dim3(1), dim3(64), 0, stream, amax_dev);
            return check_hip(hipGetLastError(), "cast_zero_amax_kernel");
        }
        return F8MI_OK;
    }
    if (!x) { set_error("f8mi_cast: null tensor"); return F8MI_ERR_INVALID_ARG; }
    const int64_t ty = (rows + CAST_TILE - 1) / CAST_TILE, tx = (cols + CAST_TILE - 1) / CAST_TILE;
    if (tx * ty > 0x7fffffffLL) { set_error("f8mi_cast: more than 2^31 tiles"); return F8MI_ERR_UNSUPPORTED; }
    dim3 g((unsigned)(tx * ty));
    const int64_t tiles_x = tx, tiles_y = ty;
    const size_t esz = in_dtype == F8MI_FP32 ? 4 : 2;
    const double n = (double)rows * (double)cols;
    // every launch of this call: the cast and what a fused amax adds before or after it
    ProfScope prof(F8MI_K_CAST, (ld == 0 ? (double)cols : n) * esz + n * ((out ? 1 : 0) + (out_t ? 1 : 0)), stream);
    if (amax_dev && !src.spread) {
        hipLaunchKernelGGL(cast_zero_amax_kernel, dim3(1), dim3(64), 0, stream, amax_dev);
        if (int rc = check_hip(hipGetLastError(), "cast_zero_amax_kernel")) return rc;
    }
    int rc;
    if (in_dtype == F8MI_BF16) {
        if (product_dtype == F8MI_BF16) rc = launch_cast1<F8MI_BF16, F8MI_BF16>(fp8_fmt, g, stream, x, rows, cols, ld, scale_dev, out, out_t, amax_dev, tiles_x, tiles_y, out_kb, out_t_kb, src);
        else rc = launch_cast1<F8MI_BF16, F8MI_FP32>(fp8_fmt, g, stream, x, rows, cols, ld, scale_dev, out, out_t, amax_dev, tiles_x, tiles_y, out_kb, out_t_kb, src);
    } else if (in_dtype == F8MI_FP16) {
        if (product_dtype == F8MI_FP16) rc = launch_cast1<F8MI_FP16, F8MI_FP16>(fp8_fmt, g, stream, x, rows, cols, ld, scale_dev, out, out_t, amax_dev, tiles_x, tiles_y, out_kb, out_t_kb, src);
        else rc = launch_cast1<F8MI_FP16, F8MI_FP32>(fp8_fmt, g, stream, x, rows, cols, ld, scale_dev, out, out_t, amax_dev, tiles_x, tiles_y, out_kb, out_t_kb, src);
    } else {
        rc = launch_cast1<F8MI_FP32, F8MI_FP32>(fp8_fmt, g, stream, x, rows, cols, ld, scale_dev, out, out_t, amax_dev, tiles_x, tiles_y, out_kb, out_t_kb, src);
    }
    if (rc || !(amax_dev && src.spread)) return rc;
    hipLaunchKernelGGL(cast_spread_finalize_kernel, dim3(1), dim3(SPREAD_WORDS), 0, stream, src.spread, amax_dev, in_dtype);
    return check_hip(hipGetLastError(), "cast_spread_finalize_kernel");
}

}  // namespace f8mi

using namespace f8mi;

extern "C" int f8mi_cast_layout(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype,
                                const float* scale_dev, int product_dtype, int fp8_fmt, uint8_t* out, int out_layout,
                                uint8_t* out_t, int out_t_layout, float* amax_dev, void* stream) {
    return cast_layout_impl(x, rows, cols, ld, in_dtype, scale_dev, product_dtype, fp8_fmt, out, out_layout, out_t, out_t_layout, amax_dev,
                            (hipStream_t)stream, AmaxSource{nullptr, 0, nullptr, nullptr});
}

extern "C" int f8mi_cast(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, const float* scale_dev,
                         int product_dtype, int fp8_fmt, uint8_t* out, uint8_t* out_t, float* amax_dev,
                         void* workspace, void* stream) {
    (void)workspace;
    return f8mi_cast_layout(x, rows, cols, ld, in_dtype, scale_dev, product_dtype, fp8_fmt, out, F8MI_LAYOUT_ROWMAJOR, out_t,
                            F8MI_LAYOUT_ROWMAJOR, amax_dev, stream);
}

extern "C" size_t f8mi_delayed_workspace_bytes(void) { return SPREAD_WORDS * sizeof(uint32_t); }

extern "C" int f8mi_cast_delayed(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, const float* scale_dev, int fp8_fmt,
                                 uint8_t* out, int out_layout, uint8_t* out_t, int out_t_layout, float* amax_dev, void* workspace,
                                 void* stream) {
    if (!amax_dev) { set_error("f8mi_cast_delayed: null amax"); return F8MI_ERR_INVALID_ARG; }
    if (!workspace || (uintptr_t)workspace % 4 != 0) { set_error("f8mi_cast_delayed: null or misaligned workspace"); return F8MI_ERR_INVALID_ARG; }
    return cast_layout_impl(x, rows, cols, ld, in_dtype, scale_dev, F8MI_FP32, fp8_fmt, out, out_layout, out_t, out_t_layout, amax_dev,
                            (hipStream_t)stream, AmaxSource{nullptr, 0, nullptr, (uint32_t*)workspace});
}

extern "C" int f8mi_cast_dynamic(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, int fp8_fmt, float* scale_dev,
                                 uint8_t* out, int out_layout, uint8_t* out_t, int out_t_layout, void* workspace, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (!scale_dev) { set_error("f8mi_cast_dynamic: null scale"); return F8MI_ERR_INVALID_ARG; }
    if (rows < 0 || cols < 0 || (ld < cols && ld != 0) || in_dtype < 0 || in_dtype > 2 || fp8_fmt < 0 || fp8_fmt > 1) { set_error("f8mi_cast_dynamic: bad shape or dtype/format code"); return F8MI_ERR_INVALID_ARG; }
    const size_t esz = in_dtype == F8MI_FP32 ? 4 : 2;
    const int64_t n = rows * cols;
    const bool padded = (out && out_layout == F8MI_LAYOUT_KBLOCK64_PAD128) || (out_t && out_t_layout == F8MI_LAYOUT_KBLOCK64_PAD128);  // the tile kernel writes the padding
    if (n > 0 && rows * ((cols + 7) / 8) <= SMALL_MAX_ITEMS && (out || out_t) && !padded) {
        if ((out_layout != F8MI_LAYOUT_ROWMAJOR && out_layout != F8MI_LAYOUT_KBLOCK64) || (out_t_layout != F8MI_LAYOUT_ROWMAJOR && out_t_layout != F8MI_LAYOUT_KBLOCK64)) { set_error("f8mi_cast_dynamic: unknown layout code"); return F8MI_ERR_INVALID_ARG; }
        if (out && out_layout == F8MI_LAYOUT_KBLOCK64 && cols % 64 != 0) { set_error("f8mi_cast_dynamic: k-blocked `out` needs cols %% 64 == 0 (cols=%lld)", (long long)cols); return F8MI_ERR_UNSUPPORTED; }
        if (out_t && out_t_layout == F8MI_LAYOUT_KBLOCK64 && rows % 64 != 0) { set_error("f8mi_cast_dynamic: k-blocked `out_t` needs rows %% 64 == 0 (rows=%lld)", (long long)rows); return F8MI_ERR_UNSUPPORTED; }
        if (!x) { set_error("f8mi_cast_dynamic: null tensor"); return F8MI_ERR_INVALID_ARG; }
        const int out_kb = out_layout == F8MI_LAYOUT_KBLOCK64, out_t_kb = out_t_layout == F8MI_LAYOUT_KBLOCK64;
        ProfScope prof(F8MI_K_CAST, (double)n * (esz + (out ? 1 : 0) + (out_t ? 1 : 0)), stream);
        if (in_dtype == F8MI_BF16) return launch_cast_small<F8MI_BF16>(fp8_fmt, stream, x, rows, cols, ld, scale_dev, out, out_t, out_kb, out_t_kb);
        if (in_dtype == F8MI_FP16) return launch_cast_small<F8MI_FP16>(fp8_fmt, stream, x, rows, cols, ld, scale_dev, out, out_t, out_kb, out_t_kb);
        return launch_cast_small<F8MI_FP32>(fp8_fmt, stream, x, rows, cols, ld, scale_dev, out, out_t, out_kb, out_t_kb);
    }
    if (n == 0 || (!out && !out_t))  // only the scale is wanted
        return f8mi_amax_scale(x, rows, cols, ld, in_dtype, fp8_fmt, in_dtype, in_dtype == F8MI_FP16, nullptr, scale_dev, workspace, stream_);
    if (!x || !workspace) { set_error("f8mi_cast_dynamic: null tensor or workspace"); return F8MI_ERR_INVALID_ARG; }
    if ((uintptr_t)workspace % 16 != 0) {  // the cast reads the workspace in 16-byte pieces: an odd one takes the two calls as they are
        int rc = f8mi_amax_scale(x, rows, cols, ld, in_dtype, fp8_fmt, in_dtype, in_dtype == F8MI_FP16, nullptr, scale_dev, workspace, stream_);
        if (rc) return rc;
        return f8mi_cast_layout(x, rows, cols, ld, in_dtype, scale_dev, in_dtype, fp8_fmt, out, out_layout, out_t, out_t_layout, nullptr, stream_);
    }
    // amax pass: per-workgroup maxima into the workspace; the cast's workgroups reduce them and derive the scale
    // themselves (no one-block finalize launch in between), workgroup 0 stores it to *scale_dev
    int nblocks = 0;
    {
        ProfScope prof(F8MI_K_AMAX, (double)(ld == 0 ? cols : n) * esz, stream);
        if (int rc = launch_amax_partials(x, rows, cols, ld, in_dtype, (uint32_t*)workspace, stream, &nblocks)) return rc;
    }
    return cast_layout_impl(x, rows, cols, ld, in_dtype, nullptr, in_dtype, fp8_fmt, out, out_layout, out_t, out_t_layout, nullptr, stream,
                            AmaxSource{(const uint32_t*)workspace, nblocks, scale_dev, nullptr});
}

namespace f8mi {

// ---- dynamic scaling for callers that cannot allocate ---------------------------------------------------------
// The per-workgroup partial maxima of the amax pass (one word per workgroup, at most WS_WORDS of them whatever the
// tensor's size) go to a device array that is part of the library's code object instead of a workspace the caller
// brings.  Every GPU holds its own copy of the array at its own address from the moment the library is loaded on
// it until the process ends; `scratch` below is only the host-side handle of it, the address is looked up once per
// device and kept.  Nothing in it has to start at zero: a call writes the words it reads back.
static __device__ __align__(256) uint32_t scratch[WS_WORDS];
static_assert(sizeof(scratch) == F8MI_STATIC_SCRATCH_BYTES, "f8mi.h states the size of the static scratch");

constexpr int STATIC_MAX_DEVICES = 64;
static std::atomic<uint32_t*> g_scratch_ptr[STATIC_MAX_DEVICES];

// Device address of `scratch` on the current device (nullptr + error message on failure).
static uint32_t* static_scratch_ptr() {
    int dev = -1;
    if (check_hip(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) { set_error("f8mi_cast_dynamic_static: device index %d, at most %d devices", dev, STATIC_MAX_DEVICES); return nullptr; }
    uint32_t* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p) return p;
    void* addr = nullptr;
    if (check_hip(hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
    if (!addr) { set_error("f8mi_cast_dynamic_static: the static scratch has no address on device %d", dev); return nullptr; }
    g_scratch_ptr[dev].store((uint32_t*)addr, std::memory_order_release);  // two threads racing here store the same value
    return (uint32_t*)addr;
}

}  // namespace f8mi

extern "C" int f8mi_cast_dynamic_static(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, int fp8_fmt, float* scale_dev,
                                        uint8_t* out, int out_layout, uint8_t* out_t, int out_t_layout, void* stream) {
    if (rows < 0 || cols < 0) { set_error("f8mi_cast_dynamic_static: bad shape rows=%lld cols=%lld", (long long)rows, (long long)cols); return F8MI_ERR_INVALID_ARG; }
    if (rows > 0 && cols > F8MI_STATIC_MAX_ELEMS / rows) {
        set_error("f8mi_cast_dynamic_static: %lld x %lld elements, at most %lld per call (use f8mi_cast_dynamic with a workspace)",
                  (long long)rows, (long long)cols, (long long)F8MI_STATIC_MAX_ELEMS);
        return F8MI_ERR_INVALID_ARG;
    }
    uint32_t* ws = f8mi::static_scratch_ptr();
    if (!ws) return F8MI_ERR_HIP;
    return f8mi_cast_dynamic(x, rows, cols, ld, in_dtype, fp8_fmt, scale_dev, out, out_layout, out_t, out_t_layout, ws, stream);
}
