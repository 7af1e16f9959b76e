/*
 * f8_oracle.c -- scalar CPU restatement of the Float8Linear hot path of
 * pytorch-labs/float8_experimental.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the parity tests,
 * the smoke test and the CPU-baseline leg of the benchmark compare the HIP
 * kernels against.  Nothing in the shipped package may call into it.
 *
 * Every routine below restates, one scalar at a time and with every
 * intermediate rounding made explicit, what the reference obtains by composing
 * torch operators.  The reference locations are given per function
 * (paths relative to the reference checkout).
 *
 * Pins (tests/test_oracle_*.py): the committed golden vectors written by the
 * reference itself (tests/golden/*.npz), torch's own fp8 conversion over all
 * 65536 bf16 patterns and a strided fp32 sweep, closed forms (powers of two,
 * all 256 fp8 codes as fixed points, ties-to-even midpoints), brute force on
 * tiny GEMMs.
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off -shared -fPIC
 * (contraction must stay off: the roundings below are the specification).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define F8O_BF16 0
#define F8O_FP16 1
#define F8O_FP32 2

#define F8O_E4M3FN 0
#define F8O_E5M2 1

/* ------------------------------------------------------------------ bits */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float f8o_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even; NaN -> canonical quiet NaN (sign kept). */
uint16_t f8o_f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(((u >> 16) & 0x8000u) | 0x7fc0u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float f8o_fp16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0x1f) return u2f(sign | 0x7f800000u | (m << 13));
    if (e == 0) {
        if (m == 0) return u2f(sign);
        /* subnormal: value = m * 2^-24 */
        float v = (float)m * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* fp32 -> fp16, round to nearest even, overflow -> inf, NaN -> quiet NaN. */
uint16_t f8o_f32_to_fp16(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 incl. inf */
    int e = (int)(a >> 23) - 127;
    uint32_t mant = (a & 0x7fffffu) | (a >= 0x00800000u ? 0x800000u : 0u);
    if (a < 0x00800000u) return sign; /* fp32 subnormal: far below fp16 range */
    int shift = 13;
    if (e < -14) shift += (-14 - e);
    if (shift > 25) return sign;
    uint32_t q = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    uint32_t code;
    if (e >= -14) code = ((uint32_t)(e + 15) << 10) + (q - 0x400u);
    else code = q;
    if (code >= 0x7c00u) code = 0x7c00u;
    return (uint16_t)(sign | code);
}

/* --------------------------------------------------------------- fp8 codec */

/*
 * fp32 -> OCP fp8, round to nearest even, subnormals kept, no saturation.
 * Restates what `tensor.to(torch.float8_e4m3fn / float8_e5m2)` yields
 * (reference: float8_utils.py:137 calls it after the clamp):
 *   e4m3fn (bias 7, max 448, no inf): anything that rounds above 448, +-inf
 *          and NaN become the NaN code 0x7F (sign kept);
 *   e5m2   (bias 15, max 57344): anything that rounds above 57344 and +-inf
 *          become inf 0x7C, NaN becomes 0x7F (sign kept).
 */
uint8_t f8o_f32_to_fp8(float f, int fmt) {
    const int mbits = fmt == F8O_E4M3FN ? 3 : 2;
    const int bias = fmt == F8O_E4M3FN ? 7 : 15;
    uint32_t u = f2u(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
    if (a == 0x7f800000u) return (uint8_t)(sign | (fmt == F8O_E4M3FN ? 0x7fu : 0x7cu));
    if (a < 0x00800000u) return sign; /* zero and fp32 subnormals */
    int e = (int)(a >> 23) - 127;
    uint32_t mant = (a & 0x7fffffu) | 0x800000u;
    int emin = 1 - bias;
    int shift = 23 - mbits;
    if (e < emin) shift += emin - e;
    if (shift > 25) return sign;
    uint32_t q = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    uint32_t code;
    if (e >= emin) {
        if (e + bias > 31) code = 0xffu;
        else code = ((uint32_t)(e + bias) << mbits) + (q - (1u << mbits));
    } else {
        code = q;
    }
    if (fmt == F8O_E4M3FN) { if (code > 0x7fu) code = 0x7fu; }
    else { if (code > 0x7cu) code = 0x7cu; }
    return (uint8_t)(sign | code);
}

/* OCP fp8 -> fp32 (exact). */
float f8o_fp8_to_f32(uint8_t c, int fmt) {
    const int mbits = fmt == F8O_E4M3FN ? 3 : 2;
    const int bias = fmt == F8O_E4M3FN ? 7 : 15;
    int sign = c >> 7;
    int e = (c & 0x7f) >> mbits;
    int m = c & ((1 << mbits) - 1);
    float v;
    if (fmt == F8O_E4M3FN) {
        if ((c & 0x7f) == 0x7f) return u2f(sign ? 0xffc00000u : 0x7fc00000u);
    } else {
        if (e == 31) {
            if (m == 0) return sign ? -INFINITY : INFINITY;
            return u2f(sign ? 0xffc00000u : 0x7fc00000u);
        }
    }
    if (e == 0) v = ldexpf((float)m, 1 - bias - mbits);
    else v = ldexpf((float)(m + (1 << mbits)), e - bias - mbits);
    return sign ? -v : v;
}

void f8o_f32_to_fp8_n(const float* x, size_t n, int fmt, uint8_t* out) {
    for (size_t i = 0; i < n; i++) out[i] = f8o_f32_to_fp8(x[i], fmt);
}

void f8o_fp8_to_f32_n(const uint8_t* c, size_t n, int fmt, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = f8o_fp8_to_f32(c[i], fmt);
}

float f8o_fp8_max(int fmt) { return fmt == F8O_E4M3FN ? 448.0f : 57344.0f; }

/* ------------------------------------------------------------------- amax */

static inline float load_elem(const void* x, size_t i, int dtype) {
    if (dtype == F8O_BF16) return f8o_bf16_to_f32(((const uint16_t*)x)[i]);
    if (dtype == F8O_FP16) return f8o_fp16_to_f32(((const uint16_t*)x)[i]);
    return ((const float*)x)[i];
}

/*
 * max(abs(x)), NaN-propagating, returned widened to fp32 (the value is exactly
 * representable in x's dtype).  Reference: float8_utils.py:102-112
 * (`torch.max(torch.abs(x))`; the all-reduce there needs >1 process).
 */
float f8o_amax(const void* x, size_t n, int dtype) {
    float best = 0.0f;
    int nan = 0;
    for (size_t i = 0; i < n; i++) {
        float v = fabsf(load_elem(x, i, dtype));
        if (v != v) nan = 1;
        else if (v > best) best = v;
    }
    return nan ? NAN : best;
}

/* ------------------------------------------------------------------ scale */

static float round_to(float v, int dtype) {
    if (dtype == F8O_BF16) return f8o_bf16_to_f32(f8o_f32_to_bf16(v));
    if (dtype == F8O_FP16) return f8o_fp16_to_f32(f8o_f32_to_fp16(v));
    return v;
}

/*
 * amax -> scale.  Reference: float8_utils.py:35-57.  `fmax / clamp(amax, EPS)`
 * with a Python float on the left is evaluated by torch as
 * `clamp(amax, min=EPS).reciprocal() * fmax`, and every step is rounded to the
 * dtype of `amax` (`math_dtype`): the tensor's own dtype for dynamic scaling
 * (float8_utils.py:115-120), fp32 for the delayed-scaling buffers
 * (float8_utils.py:60-99).  EPS = 1e-12 is itself rounded to that dtype (it is
 * 0 in fp16).  When the high-precision dtype is fp16 the scale is clamped to
 * 65504 (float8_utils.py:54-55).  The result is stored as fp32.
 */
float f8o_amax_to_scale(float amax, int math_dtype, int fp8_fmt, int orig_is_fp16) {
    float eps = round_to((float)1e-12, math_dtype);
    float c = (amax != amax) ? amax : (amax < eps ? eps : amax);
    float r = round_to(1.0f / c, math_dtype);
    float s = round_to(r * f8o_fp8_max(fp8_fmt), math_dtype);
    if (orig_is_fp16 && !(s != s) && s > 65504.0f) s = 65504.0f;
    return s;
}

/* ------------------------------------------------------------------- cast */

/*
 * Saturated cast of one element.  Reference: float8_tensor.py:158-159
 * (`tensor * scale`, then to_fp8_saturated) and float8_utils.py:123-139
 * (`clamp(-fmax, fmax)` then `.to(fp8)`).
 * `product_dtype` is the dtype torch's type promotion gives `tensor * scale`:
 *   - the tensor's dtype when `scale` is a 0-dim fp32 tensor (dynamic scaling),
 *     i.e. the fp32 product is rounded to bf16/fp16 before clamp and conversion;
 *   - fp32 when `scale` has shape [1] (delayed-scaling buffers) or x is fp32.
 */
uint8_t f8o_cast_one(float x, float scale, int product_dtype, int fp8_fmt) {
    float fmax = f8o_fp8_max(fp8_fmt);
    float y = round_to(x * scale, product_dtype);
    if (!(y != y)) {
        if (y > fmax) y = fmax;
        if (y < -fmax) y = -fmax;
    }
    return f8o_f32_to_fp8(y, fp8_fmt);
}

/* rows x cols elements at `x` (row stride ld, in elements) -> out (dense row-major)
 * and/or out_t (dense [cols][rows]); either output may be NULL. */
void f8o_cast(const void* x, size_t rows, size_t cols, size_t ld, int in_dtype, float scale,
              int product_dtype, int fp8_fmt, uint8_t* out, uint8_t* out_t) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++) {
            uint8_t b = f8o_cast_one(load_elem(x, r * ld + c, in_dtype), scale, product_dtype, fp8_fmt);
            if (out) out[r * cols + c] = b;
            if (out_t) out_t[c * rows + r] = b;
        }
}

/* ------------------------------------------------------------------- gemm */

/*
 * Emulated scaled matmul.  Reference: float8_aten_api.py:16-28
 *   mm(m1.float() / s1, m2.float() / s2).to(out_dtype)
 * A is [m][k] (row stride lda), B is given as its transpose Bt[n][k] (row stride
 * ldb) -- both operands contiguous along the reduction, which is how all three
 * GEMMs of the linear layer reach the kernel.  The elementwise dequantisation
 * (a true division, rounded to fp32) is kept; the reduction runs in double so
 * the oracle carries no summation-order noise of its own, then rounds once to
 * fp32 and once to the output dtype.  out is float[m][n] (values already rounded
 * to out_dtype).
 */
void f8o_gemm_emulated(const uint8_t* A, int a_fmt, size_t lda, float sa, const uint8_t* Bt, int b_fmt,
                       size_t ldb, float sb, size_t m, size_t n, size_t k, int out_dtype, float* out) {
    float lut_a[256], lut_b[256];
    for (int i = 0; i < 256; i++) {
        lut_a[i] = f8o_fp8_to_f32((uint8_t)i, a_fmt) / sa;
        lut_b[i] = f8o_fp8_to_f32((uint8_t)i, b_fmt) / sb;
    }
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            double acc = 0.0;
            const uint8_t* ar = A + i * lda;
            const uint8_t* br = Bt + j * ldb;
            for (size_t p = 0; p < k; p++) acc += (double)lut_a[ar[p]] * (double)lut_b[br[p]];
            out[i * n + j] = round_to((float)acc, out_dtype);
        }
}

/* ------------------------------------------------------------------- sync */

/*
 * One (layer, tensor-kind) entry of sync_float8_amax_and_scale_history.
 * Reference: float8_linear_utils.py:37-56 and :287-319, float8_utils.py:80-99.
 *   S = roll(history, 1); S[0] = amax; scale = amax_to_scale(max(S)) in fp32.
 * The reference rolls a stacked COPY of the histories (torch.vstack) and copies
 * only the scales back, so `history` itself is left untouched; `writeback` = 0
 * reproduces that, `writeback` = 1 stores S into `history`.
 * Returns the new scale.
 */
float f8o_sync_entry(float amax, float* history, int hist_len, int fp8_fmt, int orig_is_fp16, int writeback) {
    float mx = amax;
    int nan = amax != amax;
    for (int i = 0; i + 1 < hist_len; i++) {
        float h = history[i];
        if (h != h) nan = 1;
        else if (h > mx) mx = h;
    }
    if (nan) mx = NAN;
    if (writeback) {
        for (int i = hist_len - 1; i > 0; i--) history[i] = history[i - 1];
        history[0] = amax;
    }
    return f8o_amax_to_scale(mx, F8O_FP32, fp8_fmt, orig_is_fp16);
}

/*
 * First-iteration initialisation of one tensor's delayed-scaling buffers.
 * Reference: float8_scaling_utils.py:99-125:
 *   cur_amax <- amax; history[0] <- amax; scale <- amax_to_scale(max(history)).
 * Returns the new scale; history[0] is written.
 */
float f8o_delayed_init(float amax, float* history, int hist_len, int fp8_fmt, int orig_is_fp16) {
    history[0] = amax;
    float mx = -INFINITY;
    int nan = 0;
    for (int i = 0; i < hist_len; i++) {
        float h = history[i];
        if (h != h) nan = 1;
        else if (h > mx) mx = h;
    }
    if (nan) mx = NAN;
    return f8o_amax_to_scale(mx, F8O_FP32, fp8_fmt, orig_is_fp16);
}
