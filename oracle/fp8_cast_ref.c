/*
 * CPU oracle, bit-level part.  TEST INFRASTRUCTURE ONLY: linked by tests/, the smoke check and the
 * cpu_baseline leg of bench.py; never by the product library.
 *
 * Restates, with integer bit manipulation and double arithmetic only (no fp8 library type), the
 * scalar pieces of the float8 cast that the reference reaches through torchao==0.15.0
 * (reference call site: src/olmo_core/float8/__init__.py:133-150; dtype names
 * src/olmo_core/config.py:365-392):
 *   amax over |x|  ->  scale = (float)(FP8_MAX * (1.0 / max((double)amax, 1e-12)))
 *   [-> clear the mantissa of scale: round down to a power of two]
 *   y = (float)x * scale ; clamp to [-FP8_MAX, FP8_MAX] ; round-to-nearest-even to OCP e4m3fn/e5m2.
 * It is an implementation independent of torch's converters, so that tests can pin torch-CPU's
 * `.to(torch.float8_*)` (used by oracle/float8_oracle.py) against it exhaustively and vice versa.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define ORC_E4M3 0
#define ORC_E5M2 1

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

double orc_fp8_max(int dtype) { return dtype == ORC_E4M3 ? 448.0 : 57344.0; }

/* Unsaturated IEEE-style round-to-nearest-even conversion float32 -> fp8 byte.
 * e4m3fn: 4 exponent bits, bias 7, no infinity, 0x7F/0xFF = NaN, max finite 0x7E = 448.
 * e5m2 : 5 exponent bits, bias 15, 0x7C = inf, 0x7D..0x7F = NaN, max finite 0x7B = 57344. */
uint8_t orc_f32_to_fp8(float f, int dtype)
{
    const int mbits = dtype == ORC_E4M3 ? 3 : 2;
    const int bias = dtype == ORC_E4M3 ? 7 : 15;
    const uint32_t u = f2u(f);
    const uint8_t sign = (uint8_t)((u >> 31) << 7);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7F;                 /* NaN keeps its sign bit */
    if (a == 0x7F800000u) return sign | (dtype == ORC_E4M3 ? 0x7F : 0x7C);
    const int e = (int)(a >> 23) - 127;
    uint32_t code;
    if (e >= 1 - bias) {
        /* normal in the target: RNE on the (23 - mbits) dropped mantissa bits */
        const int shift = 23 - mbits;
        uint32_t r = a + ((1u << (shift - 1)) - 1u) + ((a >> shift) & 1u);
        r >>= shift;                                          /* [8-bit exp | mbits mantissa] */
        int fe = (int)(r >> mbits) - 127 + bias;
        code = ((uint32_t)fe << mbits) | (r & ((1u << mbits) - 1u));
        if (dtype == ORC_E4M3) { if (code > 0x7E) code = 0x7F; }
        else { if (code > 0x7B) code = 0x7C; }
    } else {
        /* subnormal in the target: value / 2^(1-bias-mbits) rounded to an integer (ties to even;
         * rint() under the default rounding mode).  A result of 2^mbits is the smallest normal. */
        double v = ldexp((double)u2f(a), bias - 1 + mbits);
        code = (uint32_t)rint(v);
    }
    return sign | (uint8_t)code;
}

/* value of an fp8 byte, for the emulated matmul */
float orc_fp8_to_f32(uint8_t b, int dtype)
{
    const int mbits = dtype == ORC_E4M3 ? 3 : 2;
    const int bias = dtype == ORC_E4M3 ? 7 : 15;
    const int ebits = 7 - mbits;
    const int e = (b >> mbits) & ((1 << ebits) - 1);
    const int m = b & ((1 << mbits) - 1);
    double v;
    if (dtype == ORC_E4M3 && (b & 0x7F) == 0x7F) v = NAN;
    else if (dtype == ORC_E5M2 && e == 31) v = m ? NAN : INFINITY;
    else if (e == 0) v = ldexp((double)m, 1 - bias - mbits);
    else v = ldexp(1.0 + (double)m / (1 << mbits), e - bias);
    return (float)((b & 0x80) ? -v : v);
}

/* amax of |x| over n bf16 values, NaN-propagating, returned as float */
float orc_amax_bf16(const uint16_t* x, size_t n)
{
    float m = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        float v = fabsf(bf16_to_f32(x[i]));
        if (isnan(v)) return NAN;
        if (v > m) m = v;
    }
    return m;
}

float orc_amax_f32(const float* x, size_t n)
{
    float m = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        float v = fabsf(x[i]);
        if (isnan(v)) return NAN;
        if (v > m) m = v;
    }
    return m;
}

/* scale from amax: float64 reciprocal times FP8_MAX, rounded once to float32 */
float orc_scale_from_amax(float amax, int dtype, int pow2)
{
    double a = (double)amax;
    if (!(isnan(a))) a = a < 1e-12 ? 1e-12 : a;     /* clamp(min=EPS) keeps NaN */
    float s = (float)((1.0 / a) * orc_fp8_max(dtype));
    if (pow2 && !isnan(s)) s = u2f(f2u(s) & 0x7F800000u);   /* 2^floor(log2 s) for normal s; 0 stays 0 */
    return s;
}

/* saturating cast of one float already multiplied by the scale */
uint8_t orc_saturate_cast(float y, int dtype)
{
    const float m = (float)orc_fp8_max(dtype);
    if (y > m) y = m;            /* comparisons are false for NaN: NaN passes through */
    if (y < -m) y = -m;
    return orc_f32_to_fp8(y, dtype);
}

void orc_cast_bf16(const uint16_t* x, size_t n, float scale, int dtype, uint8_t* out)
{
    for (size_t i = 0; i < n; ++i) {
        volatile float y = bf16_to_f32(x[i]) * scale;   /* one fp32 multiply, not contracted */
        out[i] = orc_saturate_cast(y, dtype);
    }
}

void orc_cast_f32(const float* x, size_t n, float scale, int dtype, uint8_t* out)
{
    for (size_t i = 0; i < n; ++i) {
        volatile float y = x[i] * scale;
        out[i] = orc_saturate_cast(y, dtype);
    }
}

/* emulated matmul for tiny shapes: out[m,n] = sum_k (a[m,k]/sa[m or 0]) * (b[n,k]/sb[n or 0]),
 * accumulated in double (a tolerance reference, not a bit reference). a: [M,K], b: [N,K]. */
void orc_emulated_mm(const uint8_t* a, int a_dtype, const float* sa, int sa_is_vec,
                     const uint8_t* b, int b_dtype, const float* sb, int sb_is_vec,
                     int64_t M, int64_t N, int64_t K, double* out)
{
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            const float s_a = sa[sa_is_vec ? m : 0], s_b = sb[sb_is_vec ? n : 0];
            for (int64_t k = 0; k < K; ++k) {
                float av = orc_fp8_to_f32(a[m * K + k], a_dtype) / s_a;
                float bv = orc_fp8_to_f32(b[n * K + k], b_dtype) / s_b;
                acc += (double)av * (double)bv;
            }
            out[m * N + n] = acc;
        }
}
