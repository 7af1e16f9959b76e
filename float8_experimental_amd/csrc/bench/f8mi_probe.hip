// Benchmark aid, built into its own shared object (libf8mi_probe.so): what the fp8 matrix cores of this GPU
// sustain with no memory traffic at all.  It is not part of libf8mi.so: it copies from host memory and waits for
// the stream, which the library's entry points never do.
// A register-only loop of v_mfma_f32_16x16x128_f8f6f4 (the GEMM's instruction) over 64 accumulator
// tiles per wave, one wave per SIMD on every CU.  On all-zero operands the loop runs at the clock limit;
// on random fp8 bytes it runs into the power limit, which is the ceiling a real GEMM works under.
//
//   int f8mi_probe_mfma(int random_data, int iters, void* scratch_dev, size_t scratch_bytes, double* tflops, void* stream)
//     random_data 0: all-zero operands, 1: random finite e4m3 bytes, 2: the first 256 KiB of scratch_dev as the
//     caller left them (fp8 bytes of a real tensor); plus 16 * order, which operand of consecutive instructions
//     changes: order 0 the first (as in the GEMM: the second stays for eight), 1 the second, 2 both, 3 neither;
//     scratch_dev: >= 1 MiB of device memory of the caller's;  *tflops receives the rate.  Returns 0, or -1 (bad argument) / -3 (a HIP call failed).
#include <vector>

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

namespace f8mi {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

template <int ORDER>
__global__ __launch_bounds__(256) void mfma_probe_kernel(const int* __restrict__ in, float* __restrict__ out, int iters) {
    v8i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) {
            a[i][j] = in[(threadIdx.x * 8 + j + i * 2048) & 65535];
            b[i][j] = in[(threadIdx.x * 8 + j + i * 2048 + 17) & 65535];
        }
    v4f acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int j = 0; j < 8; j++)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    b[(ORDER == 1 || ORDER == 3 ? i : j) & 3], a[(ORDER == 1 ? j : ORDER == 2 ? i + j : i) & 3], acc[i][j], 0, 0, 0, 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) s += acc[i][j][e];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace f8mi

using namespace f8mi;

static int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return 0;
    fprintf(stderr, "f8mi_probe_mfma: %s: %s\n", what, hipGetErrorString(e));
    return -3;
}

extern "C" int f8mi_probe_mfma(int random_data, int iters, void* scratch_dev, size_t scratch_bytes, double* tflops, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    int dev = 0, n_cu = 0;
    if (check_hip(hipGetDevice(&dev), "hipGetDevice") || check_hip(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev), "hipDeviceGetAttribute")) return -3;
    const size_t need = 65536 * sizeof(int) + (size_t)n_cu * 256 * sizeof(float);
    const int order = random_data >> 4;
    random_data &= 15;
    if (order < 0 || order > 3 || random_data > 2) { fprintf(stderr, "f8mi_probe_mfma: unknown mode\n"); return -1; }
    auto kern = order == 0 ? mfma_probe_kernel<0> : order == 1 ? mfma_probe_kernel<1> : order == 2 ? mfma_probe_kernel<2> : mfma_probe_kernel<3>;
    if (!scratch_dev || scratch_bytes < need || !tflops || iters < 1) { fprintf(stderr, "f8mi_probe_mfma: needs %zu bytes of device scratch, a result pointer and iters >= 1\n", need); return -1; }
    int* in = (int*)scratch_dev;
    float* out = (float*)((char*)scratch_dev + 65536 * sizeof(int));
    std::vector<int> h(65536, 0);
    if (random_data == 1) {
        uint32_t state = 12345u;
        for (auto& w : h) {
            uint32_t v = 0;
            for (int byte = 0; byte < 4; byte++) {
                state = state * 1664525u + 1013904223u;
                // sign random, exponent field 4..8 of 15 (finite, mid-range), mantissa random
                const uint32_t e4m3 = ((state >> 24) & 0x80u) | ((4u + ((state >> 16) % 5u)) << 3) | ((state >> 8) & 7u);
                v |= e4m3 << (8 * byte);
            }
            w = (int)v;
        }
    }
    int rc = 0;
    if (random_data != 2) rc = check_hip(hipMemcpyAsync(in, h.data(), 65536 * sizeof(int), hipMemcpyHostToDevice, stream), "hipMemcpyAsync");
    if (rc) return rc;
    rc = check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    if (rc) return rc;
    hipEvent_t e0, e1;
    if ((rc = check_hip(hipEventCreate(&e0), "hipEventCreate"))) return rc;
    if ((rc = check_hip(hipEventCreate(&e1), "hipEventCreate"))) { (void)hipEventDestroy(e0); return rc; }
    hipLaunchKernelGGL(kern, dim3(n_cu), dim3(256), 0, stream, in, out, iters / 8 + 1);  // warm-up
    (void)hipEventRecord(e0, stream);
    hipLaunchKernelGGL(kern, dim3(n_cu), dim3(256), 0, stream, in, out, iters);
    (void)hipEventRecord(e1, stream);
    rc = check_hip(hipEventSynchronize(e1), "hipEventSynchronize");
    float ms = 0.f;
    if (!rc) rc = check_hip(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc) return rc;
    const double flop = 64.0 * 2 * 16 * 16 * 128 * (double)iters * 4 * n_cu;
    *tflops = flop / (ms * 1e-3) / 1e12;
    return 0;
}
