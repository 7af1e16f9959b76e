// K4: delayed-scaling bookkeeping for every (layer, tensor) pair in one launch,
// and the first-iteration initialisation of one tensor's buffers.  Latency-bound
// (3L * (H + 2) floats); one lane per entry.
#include "f8mi_common.h"

namespace f8mi {

__device__ __forceinline__ void sync_entry(const f8mi_sync_entry& e, int hist_len, int orig_is_fp16, int writeback) {
    const float amax = *e.amax;
    // S = roll(history, 1); S[0] = amax  ->  max(S) = max(amax, history[0 .. H-2])
    float mx = amax;
    bool nan = amax != amax;
    for (int j = 0; j + 1 < hist_len; j++) {
        const float h = e.history[j];
        nan |= (h != h);
        mx = h > mx ? h : mx;
    }
    if (nan) mx = __uint_as_float(0x7fc00000u);
    if (writeback) {
        for (int j = hist_len - 1; j > 0; j--) e.history[j] = e.history[j - 1];
        e.history[0] = amax;
    }
    *e.scale = amax_to_scale_dev(mx, F8MI_FP32, (int)e.fp8_fmt, orig_is_fp16);
}

__global__ void sync_kernel(const f8mi_sync_entry* __restrict__ entries, int n, int hist_len, int orig_is_fp16,
                            int writeback) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    sync_entry(entries[i], hist_len, orig_is_fp16, writeback);
}

// The same with the entries passed by value as a kernel argument (no table in device memory to build, copy or
// keep): SYNC_CHUNK entries per launch.
constexpr int SYNC_CHUNK = 32;
struct SyncChunk {
    f8mi_sync_entry e[SYNC_CHUNK];
};

__global__ void sync_args_kernel(SyncChunk chunk, int n, int hist_len, int orig_is_fp16, int writeback) {
    const int i = threadIdx.x;
    if (blockIdx.x != 0 || i >= n) return;
    sync_entry(chunk.e[i], hist_len, orig_is_fp16, writeback);
}

__global__ void delayed_init_kernel(const float* amax_dev, float* history, float* scale, int hist_len, int fmt,
                                    int orig_is_fp16) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    const float amax = *amax_dev;
    history[0] = amax;
    float mx = amax;
    bool nan = amax != amax;
    for (int j = 1; j < hist_len; j++) {
        const float h = history[j];
        nan |= (h != h);
        mx = h > mx ? h : mx;
    }
    if (nan) mx = __uint_as_float(0x7fc00000u);
    *scale = amax_to_scale_dev(mx, F8MI_FP32, fmt, orig_is_fp16);
}

}  // namespace f8mi

using namespace f8mi;

extern "C" int f8mi_sync(const f8mi_sync_entry* entries_dev, int n, int hist_len, int orig_is_fp16,
                         int writeback_history, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (n < 0 || hist_len < 1) { set_error("f8mi_sync: bad n=%d or hist_len=%d", n, hist_len); return F8MI_ERR_INVALID_ARG; }
    if (n == 0) return F8MI_OK;
    if (!entries_dev) { set_error("f8mi_sync: null entry table"); return F8MI_ERR_INVALID_ARG; }
    ProfScope prof(F8MI_K_SYNC, (double)n * (hist_len + 2) * 4.0, stream);
    const int threads = 64;
    hipLaunchKernelGGL(sync_kernel, dim3((n + threads - 1) / threads), dim3(threads), 0, stream, entries_dev, n,
                       hist_len, orig_is_fp16, writeback_history);
    return check_hip(hipGetLastError(), "sync_kernel launch");
}

extern "C" int f8mi_sync_host(const f8mi_sync_entry* entries_host, int n, int hist_len, int orig_is_fp16,
                              int writeback_history, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (n < 0 || hist_len < 1) { set_error("f8mi_sync_host: bad n=%d or hist_len=%d", n, hist_len); return F8MI_ERR_INVALID_ARG; }
    if (n == 0) return F8MI_OK;
    if (!entries_host) { set_error("f8mi_sync_host: null entry array"); return F8MI_ERR_INVALID_ARG; }
    for (int i = 0; i < n; i++)
        if (!entries_host[i].amax || !entries_host[i].history || !entries_host[i].scale || entries_host[i].fp8_fmt < 0 || entries_host[i].fp8_fmt > 1) {
            set_error("f8mi_sync_host: entry %d has a null pointer or an unknown fp8 format", i);
            return F8MI_ERR_INVALID_ARG;
        }
    ProfScope prof(F8MI_K_SYNC, (double)n * (hist_len + 2) * 4.0, stream);
    for (int first = 0; first < n; first += SYNC_CHUNK) {
        SyncChunk chunk = {};
        const int m = n - first < SYNC_CHUNK ? n - first : SYNC_CHUNK;
        for (int i = 0; i < m; i++) chunk.e[i] = entries_host[first + i];
        hipLaunchKernelGGL(sync_args_kernel, dim3(1), dim3(64), 0, stream, chunk, m, hist_len, orig_is_fp16, writeback_history);
        if (int rc = check_hip(hipGetLastError(), "sync_args_kernel launch")) return rc;
    }
    return F8MI_OK;
}

extern "C" int f8mi_delayed_init(const float* amax_dev, float* history_dev, float* scale_dev, int hist_len,
                                 int fp8_fmt, int orig_is_fp16, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (!amax_dev || !history_dev || !scale_dev || hist_len < 1 || fp8_fmt < 0 || fp8_fmt > 1) { set_error("f8mi_delayed_init: bad argument"); return F8MI_ERR_INVALID_ARG; }
    hipLaunchKernelGGL(delayed_init_kernel, dim3(1), dim3(64), 0, stream, amax_dev, history_dev, scale_dev, hist_len,
                       fp8_fmt, orig_is_fp16);
    return check_hip(hipGetLastError(), "delayed_init_kernel launch");
}
