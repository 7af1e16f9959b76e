// K1: max|x| and the fp8 scale in one pass (HBM-bound: reads sizeof(T)*n bytes).
//
// |x| is reduced on the raw bit patterns: for IEEE formats the unsigned order
// of sign-cleared patterns is the order of the magnitudes, and every NaN
// pattern is larger than inf, so a NaN anywhere wins the max exactly like
// torch.max propagates it.  Each block stores its result in its own word of the
// workspace; a second, one-block launch on the same stream reduces those words and
// writes amax + scale.  (One word plus a "last block" ticket, both updated with
// atomics, cost about 80 ns per block, serialised at the end of the kernel: 40 us of
// a 90 us kernel with 512 blocks.)
#include "f8mi_common.h"

namespace f8mi {

constexpr int AMAX_THREADS = 256;
constexpr int AMAX_UNROLL = 8;  // 16-byte loads in flight per thread

// Loads are non-temporal (F8MI_AMAX_PLAIN_LOADS_MAX_BYTES in f8mi_knobs.h has what ordinary loads were measured to cost).
template <bool NT>
__device__ __forceinline__ uint4 amax_load16(const uint4* p) {
    if constexpr (NT) return load_nt16(p);
    else return *p;
}

// Folds the sign-cleared patterns of one 16-byte vector into the running maximum `m`.  16-bit types keep two
// 16-bit maxima side by side in `m` (absmax16x2) until absmax_done merges them.
template <int DT>
__device__ __forceinline__ uint32_t absmax_vec(uint4 v, uint32_t m) {
    if constexpr (DT == F8MI_FP32) {
        uint32_t a = v.x & 0x7fffffffu, b = v.y & 0x7fffffffu, c = v.z & 0x7fffffffu, d = v.w & 0x7fffffffu;
        a = a > b ? a : b;
        c = c > d ? c : d;
        a = a > c ? a : c;
        return m > a ? m : a;
    } else {
        return absmax16x2(v.w, absmax16x2(v.z, absmax16x2(v.y, absmax16x2(v.x, m))));
    }
}
template <int DT>
__device__ __forceinline__ uint32_t absmax_done(uint32_t m) {
    if constexpr (DT == F8MI_FP32) return m;
    else return fold16(m);
}

template <int DT>
__device__ __forceinline__ uint32_t absmax_elem(const void* x, int64_t i) {
    if constexpr (DT == F8MI_FP32) return ((const uint32_t*)x)[i] & 0x7fffffffu;
    else return (uint32_t)(((const uint16_t*)x)[i] & 0x7fffu);
}

__device__ __forceinline__ uint32_t block_max_u32(uint32_t m, uint32_t* lds) {
    m = wave_max_u32(m);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) lds[wave] = m;
    __syncthreads();
    if (wave == 0) {
        uint32_t v = lane < (int)(blockDim.x >> 6) ? lds[lane] : 0u;
        m = wave_max_u32(v);
    }
    return m;  // valid in wave 0
}

// Reduces the per-block maxima and publishes amax / scale.  One block.
__global__ __launch_bounds__(AMAX_THREADS) void amax_finalize_kernel(const uint32_t* __restrict__ ws, int nblocks,
                                                                      float* amax_out, float* scale_out, int in_dt,
                                                                      int math_dt, int fmt, int orig_is_fp16) {
    __shared__ uint32_t red[AMAX_THREADS / 64];
    uint32_t m = 0;
    for (int i = threadIdx.x; i < nblocks; i += AMAX_THREADS) {
        const uint32_t v = ws[i];
        m = m > v ? m : v;
    }
    m = block_max_u32(m, red);
    if (threadIdx.x == 0) {
        const float amax = abs_bits_to_float(m, in_dt);
        if (amax_out) *amax_out = amax;
        if (scale_out) *scale_out = amax_to_scale_dev(amax, math_dt, fmt, orig_is_fp16);
    }
}

// x is dense (ld == cols) and 16-byte aligned.  A block walks over tiles of AMAX_THREADS * AMAX_UNROLL
// 16-byte vectors (32 KB of contiguous memory); inside a tile consecutive lanes read consecutive
// vectors, so every wave-level load is 1 KB of one DRAM page.  (Striding each lane's loads by the whole
// grid instead costs more than half of the bandwidth.)
template <int DT, bool NT>
__global__ __launch_bounds__(AMAX_THREADS) void amax_dense_kernel(const void* __restrict__ x, int64_t n,
                                                                   uint32_t* __restrict__ ws) {
    __shared__ uint32_t red[AMAX_THREADS / 64];
    constexpr int EPV = DT == F8MI_FP32 ? 4 : 8;
    constexpr int64_t TILE = (int64_t)AMAX_THREADS * AMAX_UNROLL;
    const int64_t nvec = n / EPV;
    const uint4* xv = (const uint4*)x;
    uint32_t m = 0;
    const int64_t ntiles = (nvec + TILE - 1) / TILE;
    for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const int64_t base = t * TILE + threadIdx.x;
        uint4 v[AMAX_UNROLL];
        if (base - threadIdx.x + TILE <= nvec) {
#pragma unroll
            for (int u = 0; u < AMAX_UNROLL; u++) v[u] = amax_load16<NT>(&xv[base + u * AMAX_THREADS]);
        } else {
#pragma unroll
            for (int u = 0; u < AMAX_UNROLL; u++) {
                const int64_t i = base + u * AMAX_THREADS;
                v[u] = i < nvec ? amax_load16<NT>(&xv[i]) : make_uint4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int u = 0; u < AMAX_UNROLL; u++) m = absmax_vec<DT>(v[u], m);
    }
    m = absmax_done<DT>(m);
    if (blockIdx.x == 0) {  // scalar tail (< EPV elements)
        int64_t t = nvec * EPV + threadIdx.x;
        if (t < n) {
            uint32_t a = absmax_elem<DT>(x, t);
            m = m > a ? m : a;
        }
    }
    m = block_max_u32(m, red);
    if (threadIdx.x == 0) ws[blockIdx.x] = m;
}

// Any row stride / alignment: one element per thread step.
template <int DT>
__global__ __launch_bounds__(AMAX_THREADS) void amax_strided_kernel(const void* __restrict__ x, int64_t rows,
                                                                     int64_t cols, int64_t ld, uint32_t* __restrict__ ws) {
    __shared__ uint32_t red[AMAX_THREADS / 64];
    uint32_t m = 0;
    const int64_t n = rows * cols;
    const int64_t stride = (int64_t)gridDim.x * AMAX_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * AMAX_THREADS + threadIdx.x; i < n; i += stride) {
        int64_t r = i / cols, c = i - r * cols;
        uint32_t a = absmax_elem<DT>(x, r * ld + c);
        m = m > a ? m : a;
    }
    m = block_max_u32(m, red);
    if (threadIdx.x == 0) ws[blockIdx.x] = m;
}

// ---- several tensors in one pass ------------------------------------------------------------
// The tensors are cut into the same 32 KB tiles as above and the tiles numbered through all tensors
// (entry t owns tiles [first_tile[t], first_tile[t+1]), numel / tile elements + 1 of them).  Every read is
// guarded by the entry's own numel, whatever the tile numbers say.  A block takes a contiguous
// range of tile numbers, so it changes tensor rarely; on every change, and at its end, it folds its
// maximum into that tensor's workspace word with one atomic (a few per block, spread over n addresses).
__global__ void amax_multi_zero_kernel(uint32_t* ws, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) ws[i] = 0u;
}

template <int DT>
__global__ __launch_bounds__(AMAX_THREADS) void amax_multi_kernel(const f8mi_tensor_ref* __restrict__ refs, int n,
                                                                   int64_t total_tiles, uint32_t* __restrict__ ws) {
    __shared__ uint32_t red[AMAX_THREADS / 64];
    constexpr int EPV = DT == F8MI_FP32 ? 4 : 8;
    constexpr int64_t TILE = (int64_t)AMAX_THREADS * AMAX_UNROLL;
    const int64_t t0 = total_tiles * blockIdx.x / gridDim.x, t1 = total_tiles * (blockIdx.x + 1) / gridDim.x;
    if (t0 >= t1) return;
    // the tensor that owns tile t0: last entry with first_tile <= t0
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (refs[mid].first_tile <= t0) lo = mid; else hi = mid - 1;
    }
    int cur = lo;
    uint32_t m = 0, mv = 0;  // maximum of single elements; of whole vectors (two 16-bit maxima side by side, see absmax_vec)
    for (int64_t t = t0; t < t1; t++) {
        while (cur + 1 < n && refs[cur + 1].first_tile <= t) {  // block-uniform: flush and move on
            mv = absmax_done<DT>(mv);
            m = block_max_u32(m > mv ? m : mv, red);
            if (threadIdx.x == 0 && m) atomicMax(&ws[cur], m);
            __syncthreads();
            m = 0;
            mv = 0;
            cur++;
        }
        const f8mi_tensor_ref r = refs[cur];
        const int64_t nvec = r.numel / EPV;
        const uint4* xv = (const uint4*)r.data;
        const int64_t base = (t - r.first_tile) * TILE + threadIdx.x;
        uint4 v[AMAX_UNROLL];
        if (base - threadIdx.x + TILE <= nvec) {
#pragma unroll
            for (int u = 0; u < AMAX_UNROLL; u++) v[u] = load_nt16(&xv[base + u * AMAX_THREADS]);
        } else {
#pragma unroll
            for (int u = 0; u < AMAX_UNROLL; u++) {
                const int64_t i = base + u * AMAX_THREADS;
                v[u] = i < nvec ? load_nt16(&xv[i]) : make_uint4(0, 0, 0, 0);
            }
            // numel / (elements per tile) + 1 tiles per tensor: the last one is always partial (possibly without
            // any whole vector) and also takes the < EPV trailing elements
            const int64_t e = nvec * EPV + threadIdx.x;
            if (e < r.numel && base - threadIdx.x + TILE > nvec && base - threadIdx.x <= nvec) {
                const uint32_t a = absmax_elem<DT>(r.data, e);
                m = m > a ? m : a;
            }
        }
#pragma unroll
        for (int u = 0; u < AMAX_UNROLL; u++) mv = absmax_vec<DT>(v[u], mv);
    }
    mv = absmax_done<DT>(mv);
    m = block_max_u32(m > mv ? m : mv, red);
    if (threadIdx.x == 0 && m) atomicMax(&ws[cur], m);
}

__global__ void amax_multi_finalize_kernel(const uint32_t* __restrict__ ws, int n, float* amax_out, float* scale_out,
                                           int in_dt, int math_dt, int fmt, int orig_is_fp16) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float amax = abs_bits_to_float(ws[i], in_dt);
    if (amax_out) amax_out[i] = amax;
    if (scale_out) scale_out[i] = amax_to_scale_dev(amax, math_dt, fmt, orig_is_fp16);
}

// Empty tensor: torch.max raises; we define amax = 0 so the scale is fmax/eps.
__global__ void amax_empty_kernel(float* amax_out, float* scale_out, int math_dt, int fmt, int orig_is_fp16) {
    if (threadIdx.x == 0) {
        if (amax_out) *amax_out = 0.0f;
        if (scale_out) *scale_out = amax_to_scale_dev(0.0f, math_dt, fmt, orig_is_fp16);
    }
}

static int g_cu_count = 0;

int cu_count() {
    if (g_cu_count == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            g_cu_count = n;
        else
            g_cu_count = 256;
    }
    return g_cu_count;
}

}  // namespace f8mi

using namespace f8mi;

namespace f8mi {

// First half of f8mi_amax_scale: per-workgroup maxima of the |x| bit patterns into ws[0 .. *nblocks).  rows * cols > 0,
// arguments already validated.  The second half is amax_finalize_kernel -- or the consumer reduces the words itself
// (the dynamic-scaling cast does: one launch less).
int launch_amax_partials(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, uint32_t* ws, hipStream_t stream,
                         int* nblocks) {
    if (ld == 0 && rows > 1) rows = 1;  // every row is the same `cols` elements: the maximum of one of them
    const int64_t n = rows * cols;
    const size_t esz = in_dtype == F8MI_FP32 ? 4 : 2;
    const bool dense = (ld == cols || rows == 1) && ((uintptr_t)x % 16 == 0);
    int64_t blocks;
    if (dense) {
        const int64_t epv = 16 / esz;
        const int64_t nvec = n / epv;
        blocks = (nvec + (int64_t)AMAX_THREADS * AMAX_UNROLL - 1) / ((int64_t)AMAX_THREADS * AMAX_UNROLL);
        int64_t cap = (int64_t)cu_count() * 2;  // few, long-lived blocks, two per CU
        if (cap > WS_WORDS) cap = WS_WORDS;
        if (blocks > cap) blocks = cap;
        if (blocks < 1) blocks = 1;
        dim3 g((unsigned)blocks), b(AMAX_THREADS);
        const bool nt = (int64_t)(n * esz) > (int64_t)F8MI_AMAX_PLAIN_LOADS_MAX_BYTES;
        if (in_dtype == F8MI_BF16) {
            if (nt) hipLaunchKernelGGL((amax_dense_kernel<F8MI_BF16, true>), g, b, 0, stream, x, n, ws);
            else hipLaunchKernelGGL((amax_dense_kernel<F8MI_BF16, false>), g, b, 0, stream, x, n, ws);
        } else if (in_dtype == F8MI_FP16) {
            if (nt) hipLaunchKernelGGL((amax_dense_kernel<F8MI_FP16, true>), g, b, 0, stream, x, n, ws);
            else hipLaunchKernelGGL((amax_dense_kernel<F8MI_FP16, false>), g, b, 0, stream, x, n, ws);
        } else {
            if (nt) hipLaunchKernelGGL((amax_dense_kernel<F8MI_FP32, true>), g, b, 0, stream, x, n, ws);
            else hipLaunchKernelGGL((amax_dense_kernel<F8MI_FP32, false>), g, b, 0, stream, x, n, ws);
        }
    } else {
        blocks = (n + AMAX_THREADS - 1) / AMAX_THREADS;
        int64_t cap = (int64_t)cu_count() * 8;
        if (cap > WS_WORDS) cap = WS_WORDS;
        if (blocks > cap) blocks = cap;
        dim3 g((unsigned)blocks), b(AMAX_THREADS);
        if (in_dtype == F8MI_BF16) hipLaunchKernelGGL(amax_strided_kernel<F8MI_BF16>, g, b, 0, stream, x, rows, cols, ld, ws);
        else if (in_dtype == F8MI_FP16) hipLaunchKernelGGL(amax_strided_kernel<F8MI_FP16>, g, b, 0, stream, x, rows, cols, ld, ws);
        else hipLaunchKernelGGL(amax_strided_kernel<F8MI_FP32>, g, b, 0, stream, x, rows, cols, ld, ws);
    }
    *nblocks = (int)blocks;
    return check_hip(hipGetLastError(), "amax kernel launch");
}

}  // namespace f8mi

extern "C" int f8mi_amax_scale(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, int fp8_fmt,
                               int math_dtype, int orig_is_fp16, float* amax_dev, float* scale_dev, void* workspace,
                               void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (rows < 0 || cols < 0 || (ld < cols && ld != 0)) { set_error("f8mi_amax_scale: bad shape rows=%lld cols=%lld ld=%lld", (long long)rows, (long long)cols, (long long)ld); return F8MI_ERR_INVALID_ARG; }
    if (in_dtype < 0 || in_dtype > 2 || math_dtype < 0 || math_dtype > 2 || fp8_fmt < 0 || fp8_fmt > 1) { set_error("f8mi_amax_scale: unknown dtype/format code"); return F8MI_ERR_INVALID_ARG; }
    if (!amax_dev && !scale_dev) { set_error("f8mi_amax_scale: no output requested"); return F8MI_ERR_INVALID_ARG; }
    if (rows * cols == 0) {
        hipLaunchKernelGGL(amax_empty_kernel, dim3(1), dim3(64), 0, stream, amax_dev, scale_dev, math_dtype, fp8_fmt, orig_is_fp16);
        return check_hip(hipGetLastError(), "amax_empty_kernel");
    }
    if (!x || !workspace) { set_error("f8mi_amax_scale: null tensor or workspace"); return F8MI_ERR_INVALID_ARG; }
    uint32_t* ws = (uint32_t*)workspace;
    int blocks = 0;
    ProfScope prof(F8MI_K_AMAX, (double)(ld == 0 ? cols : rows * cols) * (in_dtype == F8MI_FP32 ? 4 : 2), stream);
    if (int rc = launch_amax_partials(x, rows, cols, ld, in_dtype, ws, stream, &blocks)) return rc;
    hipLaunchKernelGGL(amax_finalize_kernel, dim3(1), dim3(AMAX_THREADS), 0, stream, ws, blocks, amax_dev, scale_dev, in_dtype,
                       math_dtype, fp8_fmt, orig_is_fp16);
    return check_hip(hipGetLastError(), "amax finalize kernel launch");
}

extern "C" int f8mi_amax_scale_multi(const f8mi_tensor_ref* refs_dev, int n, int64_t total_tiles, int in_dtype, int fp8_fmt,
                                     int math_dtype, int orig_is_fp16, float* amax_dev, float* scale_dev, void* workspace,
                                     void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (n < 0 || n > WS_WORDS) { set_error("f8mi_amax_scale_multi: n=%d tensors, at most %d per call", n, WS_WORDS); return F8MI_ERR_INVALID_ARG; }
    if (in_dtype < 0 || in_dtype > 2 || math_dtype < 0 || math_dtype > 2 || fp8_fmt < 0 || fp8_fmt > 1) { set_error("f8mi_amax_scale_multi: unknown dtype/format code"); return F8MI_ERR_INVALID_ARG; }
    if (!amax_dev && !scale_dev) { set_error("f8mi_amax_scale_multi: no output requested"); return F8MI_ERR_INVALID_ARG; }
    if (n == 0) return F8MI_OK;
    if (!refs_dev || !workspace || total_tiles < n) { set_error("f8mi_amax_scale_multi: null table or workspace, or fewer tiles than tensors"); return F8MI_ERR_INVALID_ARG; }
    uint32_t* ws = (uint32_t*)workspace;
    hipLaunchKernelGGL(amax_multi_zero_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, ws, n);
    int64_t blocks = (int64_t)cu_count() * 2;
    if (blocks > total_tiles) blocks = total_tiles;
    {
        // profiling counter: tiles * 32 KB, an upper bound of the bytes read (less than one tile per tensor too many)
        ProfScope prof(F8MI_K_AMAX, (double)total_tiles * AMAX_THREADS * AMAX_UNROLL * 16, stream);
        dim3 g((unsigned)blocks), b(AMAX_THREADS);
        if (in_dtype == F8MI_BF16) hipLaunchKernelGGL(amax_multi_kernel<F8MI_BF16>, g, b, 0, stream, refs_dev, n, total_tiles, ws);
        else if (in_dtype == F8MI_FP16) hipLaunchKernelGGL(amax_multi_kernel<F8MI_FP16>, g, b, 0, stream, refs_dev, n, total_tiles, ws);
        else hipLaunchKernelGGL(amax_multi_kernel<F8MI_FP32>, g, b, 0, stream, refs_dev, n, total_tiles, ws);
    }
    int rc = check_hip(hipGetLastError(), "amax multi kernel launch");
    if (rc) return rc;
    hipLaunchKernelGGL(amax_multi_finalize_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, ws, n, amax_dev, scale_dev, in_dtype,
                       math_dtype, fp8_fmt, orig_is_fp16);
    return check_hip(hipGetLastError(), "amax multi finalize kernel launch");
}

extern "C" int64_t f8mi_amax_tile_elems(int in_dtype) {
    return (int64_t)AMAX_THREADS * AMAX_UNROLL * (in_dtype == F8MI_FP32 ? 4 : 8);
}
