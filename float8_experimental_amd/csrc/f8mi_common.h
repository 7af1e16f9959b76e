// Shared host/device helpers of libf8mi (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/f8mi.h"
#include "f8mi_knobs.h"

namespace f8mi {

// ----------------------------------------------------------------- host side

void set_error(const char* fmt, ...);
int check_hip(hipError_t e, const char* what);
int cu_count();  // compute units of the current device (f8mi_amax.hip)

// Profiling brackets (no-ops unless f8mi_prof_enable(1) was called).
struct ProfScope {
    int kernel;
    double work;
    hipStream_t stream;
    void* rec;
    ProfScope(int kernel, double work, hipStream_t stream);
    ~ProfScope();
};

// workspace (uint32 words): one partial max of |x| bit patterns per block of the amax kernel
constexpr int WS_WORDS = 1024;

// Per-workgroup maxima of the |x| bit patterns into ws[0 .. *nblocks) (f8mi_amax.hip): the first half of
// f8mi_amax_scale.  rows * cols > 0, arguments already validated; no profiling bracket of its own.
int launch_amax_partials(const void* x, int64_t rows, int64_t cols, int64_t ld, int in_dtype, uint32_t* ws, hipStream_t stream,
                         int* nblocks);

// ---------------------------------------------------------------- device side

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t float_to_bits(float f) { return __float_as_uint(f); }

__device__ __forceinline__ float bf16_bits_to_float(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 bits, round to nearest even; NaN -> quiet NaN.
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? 0x7fc0u : r;
}

__device__ __forceinline__ float round_to_bf16(float f) { return bf16_bits_to_float(float_to_bf16_bits(f)); }

// Two fp32 -> two bf16 (round to nearest even, NaN stays NaN) packed in one dword: one
// v_cvt_pk_bf16_f32 instead of ~5 integer operations per value.
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f2){a, b}, bf2));
}

__device__ __forceinline__ float fp16_bits_to_float(uint32_t h) {
    return __half2float(__ushort_as_half((unsigned short)h));
}

// fp32 -> fp16 -> fp32.  The empty asm pins `f` as a rounded fp32 value first: without it
// the compiler folds a preceding multiply into one mixed-precision fma (single rounding,
// and +0 addend, which turns -0 into +0), while the reference rounds twice.
__device__ __forceinline__ float round_to_fp16(float f) {
    asm volatile("" : "+v"(f));
    return __half2float(__float2half_rn(f));
}

template <int DT>
__device__ __forceinline__ float round_to(float f) {
    if constexpr (DT == F8MI_BF16) return round_to_bf16(f);
    else if constexpr (DT == F8MI_FP16) return round_to_fp16(f);
    else return f;
}

__device__ __forceinline__ float round_to_rt(float f, int dt) {
    if (dt == F8MI_BF16) return round_to_bf16(f);
    if (dt == F8MI_FP16) return round_to_fp16(f);
    return f;
}

__device__ __forceinline__ float fp8_max(int fmt) { return fmt == F8MI_E4M3FN ? 448.0f : 57344.0f; }

// |x| bit pattern (as it sits in the dtype) -> the value widened to fp32.
__device__ __forceinline__ float abs_bits_to_float(uint32_t bits, int dt) {
    if (dt == F8MI_BF16) return bf16_bits_to_float(bits);
    if (dt == F8MI_FP16) return fp16_bits_to_float(bits);
    return __uint_as_float(bits);
}

// amax -> scale: clamp(amax, min=1e-12).reciprocal() * fmax, each step rounded to
// `math_dt`, 1e-12 itself rounded to it first; optional clamp to fp16's max.
__device__ __forceinline__ float amax_to_scale_dev(float amax, int math_dt, int fmt, int orig_is_fp16) {
    float eps = round_to_rt(1e-12f, math_dt);
    float c = (amax != amax) ? amax : (amax < eps ? eps : amax);
    float r = round_to_rt(__fdiv_rn(1.0f, c), math_dt);
    float s = round_to_rt(__fmul_rn(r, fp8_max(fmt)), math_dt);
    if (orig_is_fp16 && s > 65504.0f) s = 65504.0f;
    return s;
}

// Two fp32 -> two OCP fp8 bytes (low 16 bits of the result), round to nearest
// even via the gfx950 conversion instructions.  Inputs must already be clamped
// to the finite range or be NaN.  NaN gives 0x7F (sign kept): the e4m3fn
// instruction does that by itself, the e5m2 one returns the quiet-NaN code 0x7E,
// so the low mantissa bit is set by hand to match torch's 0x7F.
template <int FMT>
__device__ __forceinline__ uint32_t cvt2_fp8(float a, float b) {
    uint32_t r;
    if constexpr (FMT == F8MI_E4M3FN) {
        r = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    } else {
        r = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
        r |= (a != a ? 0x0001u : 0u) | (b != b ? 0x0100u : 0u);
    }
    return r & 0xffffu;
}

// Four fp32 -> four fp8 bytes in one dword: the second conversion writes the upper half of the
// register the first one produced (no shift / or).
template <int FMT>
__device__ __forceinline__ uint32_t cvt4_fp8(float a, float b, float c, float d) {
    if constexpr (FMT == F8MI_E4M3FN) {
        int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
        return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
    } else {
        int r = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
        uint32_t w = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(c, d, r, true);
        // the e5m2 instruction answers NaN with the quiet code 0x7E; torch's is 0x7F
        const bool any_nan = (a != a) | (b != b) | (c != c) | (d != d);
        if (any_nan) w |= (a != a ? 0x1u : 0u) | (b != b ? 0x100u : 0u) | (c != c ? 0x10000u : 0u) | (d != d ? 0x1000000u : 0u);
        return w;
    }
}

// Workgroup barrier that waits for this wave's LDS traffic only (__syncthreads also waits for every global load
// the wave has in flight).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 16-byte streaming load (data is used once: keep it out of the way of reused lines)
__device__ __forceinline__ uint4 load_nt16(const void* p) {
    u32x4 v = __builtin_nontemporal_load((const u32x4*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// 16- and 8-byte accesses at addresses aligned to the element size only (rows of a tensor whose row pitch is not a
// multiple of 16 bytes).  Still one global_load / global_store instruction: gfx950 serves vector memory accesses at any
// byte alignment, and the compiler emits the wide instruction for these under-aligned types.
typedef u32x4 u32x4_any __attribute__((aligned(1)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x2 u32x2_any __attribute__((aligned(1)));
__device__ __forceinline__ uint4 load_nt16_any(const void* p) {
    u32x4 v = __builtin_nontemporal_load((const u32x4_any*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store16_any(void* p, uint4 v) { *(u32x4_any*)p = (u32x4){v.x, v.y, v.z, v.w}; }
__device__ __forceinline__ void store8_any(void* p, uint32_t lo, uint32_t hi) { *(u32x2_any*)p = (u32x2){lo, hi}; }

// Running maximum of sign-cleared 16-bit patterns, two per dword: `m` holds two independent 16-bit maxima
// (v_and + v_pk_max_u16 per dword instead of five scalar operations); fold16 merges the halves at the end.
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t absmax16x2(uint32_t w, uint32_t m) {
    const u16x2 a = __builtin_bit_cast(u16x2, w & 0x7fff7fffu), b = __builtin_bit_cast(u16x2, m);
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}
__device__ __forceinline__ uint32_t fold16(uint32_t m) {
    const uint32_t lo = m & 0xffffu, hi = m >> 16;
    return lo > hi ? lo : hi;
}

// wave-wide max of a uint32 (wave64)
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        uint32_t o = (uint32_t)__shfl_xor((int)v, off, 64);
        v = v > o ? v : o;
    }
    return v;
}

}  // namespace f8mi
