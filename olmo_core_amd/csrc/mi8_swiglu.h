// SwiGLU arithmetic on eight packed bf16 values at a time, shared by the flat pointwise kernels
// (mi8_pointwise.hip) and the group-aware ones that also take the amax of their outputs (mi8_cast.hip).
// Rounding points follow torch's eager bf16 evaluation: every elementwise op computes in fp32 and rounds its
// result to bf16 before the next op reads it.
#pragma once
#include "mi8_common.h"

namespace mi8 {

__device__ __forceinline__ float bf16_round(float f)
{
    __bf16 h = (__bf16)f;
    return (float)h;
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    __bf16 a = (__bf16)lo, b = (__bf16)hi;
    return (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
}

// 1 / (1 + e^-x) on the hardware exp2 and reciprocal (about one ulp each): the result feeds a bf16 rounding, and
// the library routines cost several times the instructions, which bounds these kernels before memory does.
// e^-x overflowing to +inf gives 0, underflowing to 0 gives 1, NaN stays NaN.
__device__ __forceinline__ float sigmoid_f32(float x)
{
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896341f));
}

__device__ __forceinline__ void unpack8(uint4 v, float (&f)[8])
{
    f[0] = bits_to_f32(v.x << 16);
    f[1] = bits_to_f32(v.x & 0xFFFF0000u);
    f[2] = bits_to_f32(v.y << 16);
    f[3] = bits_to_f32(v.y & 0xFFFF0000u);
    f[4] = bits_to_f32(v.z << 16);
    f[5] = bits_to_f32(v.z & 0xFFFF0000u);
    f[6] = bits_to_f32(v.w << 16);
    f[7] = bits_to_f32(v.w & 0xFFFF0000u);
}

__device__ __forceinline__ uint4 pack8(const float (&f)[8])
{
    return make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
}

// h = silu(x1) * x3
__device__ __forceinline__ uint4 swiglu_fwd8(uint4 x1, uint4 x3)
{
    float a[8], b[8], o[8];
    unpack8(x1, a);
    unpack8(x3, b);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float s = bf16_round(a[k] * sigmoid_f32(a[k]));  // silu output as a bf16 tensor
        o[k] = s * b[k];
    }
    return pack8(o);
}

// the same for four packed values (the fused epilogue of the two input projections holds four columns per lane)
__device__ __forceinline__ uint2 swiglu_fwd4(uint2 x1, uint2 x3)
{
    const float a[4] = {bits_to_f32(x1.x << 16), bits_to_f32(x1.x & 0xFFFF0000u), bits_to_f32(x1.y << 16),
                        bits_to_f32(x1.y & 0xFFFF0000u)};
    const float b[4] = {bits_to_f32(x3.x << 16), bits_to_f32(x3.x & 0xFFFF0000u), bits_to_f32(x3.y << 16),
                        bits_to_f32(x3.y & 0xFFFF0000u)};
    float o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float s = bf16_round(a[k] * sigmoid_f32(a[k]));
        o[k] = s * b[k];
    }
    return make_uint2(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]));
}

// gradients of h = silu(x1) * x3 with respect to x1 and x3
__device__ __forceinline__ void swiglu_bwd8(uint4 x1, uint4 x3, uint4 gh, uint4& g1, uint4& g3)
{
    float a[8], b[8], g[8], o1[8], o3[8];
    unpack8(x1, a);
    unpack8(x3, b);
    unpack8(gh, g);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float sig = sigmoid_f32(a[k]);
        const float s = bf16_round(a[k] * sig);    // saved silu output
        o3[k] = g[k] * s;                          // d/dx3
        const float gs = bf16_round(g[k] * b[k]);  // gradient reaching silu's output
        o1[k] = gs * (sig * (1.0f + a[k] * (1.0f - sig)));
    }
    g1 = pack8(o1);
    g3 = pack8(o3);
}

// ---- upper bounds on the SwiGLU gradients, for finding their amax without computing every element ----------
//
// With L(x) = the 15 exponent-and-mantissa bits of a bf16 value read as an integer, L(x) / 128 - 127 <= log2 |x|
// <= L(x) / 128 - 127 + 0.0861 (a piecewise-linear log2; it also holds, as an upper bound, for zeros and
// denormals).  So for S = L(g) + L(a):  |g| |a| <= 2^((S + 23) / 128 - 254), and by the rounding points of
// swiglu_bwd8
//     |g3| = |bf16(g * bf16(a * sigmoid(a)))| <= |g| |a| (1 + 2^-8)
//     |g1| = |bf16(bf16(g * b) * silu'(a))|   <= |g| |b| * 1.1 * (1 + 2^-8)^2        (|silu'| < 1.1)
// which gives  log2 |g3| <= (S3 + 24) / 128 - 254  and  log2 |g1| <= (S1 + 44) / 128 - 254.  A value t that is a
// normal bf16 number has log2 t >= L(t) / 128 - 127, hence elements with S at most L(t) + 127 * 128 - margin are at
// most t in magnitude.  L is monotone in |x|, so the same holds with the maxima of L over a row segment in place
// of the elements' own: a segment (64 consecutive columns of a row) carries one 16-bit code per tensor, the largest
// L in it, and the sum of the codes of gh and of (x1, x3) bounds every element of the segment.  A non-finite value
// has L >= 0x7F80, and so has every sum it enters: segments with a sum that large are always computed (finite
// inputs reach it only when |g| |x| > 2).
constexpr int kSegCols = 64;
constexpr uint32_t kSwigluMargin3 = 24, kSwigluMargin1 = 44, kBf16ExpBias128 = 127 * 128;

typedef unsigned short swiglu_us2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_umax16(uint32_t a, uint32_t b)
{
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(swiglu_us2, a), __builtin_bit_cast(swiglu_us2, b)));
}

// max L over eight packed bf16 values, in both 16-bit halves of the result
__device__ __forceinline__ uint32_t max_code8(uint32_t x, uint32_t y, uint32_t z, uint32_t w)
{
    const uint32_t m = pk_umax16(pk_umax16(x & 0x7FFF7FFFu, y & 0x7FFF7FFFu), pk_umax16(z & 0x7FFF7FFFu, w & 0x7FFF7FFFu));
    return pk_umax16(m, (m >> 16) | (m << 16));
}

// Must the elements of a segment whose codes sum to s be computed to know whether they exceed the maxima found so
// far (t1, t3: float32 bit patterns of bf16 values)?
__device__ __forceinline__ bool swiglu_segment_needed(uint32_t s, uint32_t t1, uint32_t t3)
{
    if (s >= 0x7F80u) return true;  // possibly a non-finite input
    const uint32_t l1 = t1 >> 16, l3 = t3 >> 16;
    // per gradient: a maximum that is inf / NaN cannot be changed by finite inputs; one below 2^-119 is no usable
    // threshold yet
    const bool need1 = l1 < 0x7F80u && (l1 < 0x0400u || s + kSwigluMargin1 > l1 + kBf16ExpBias128);
    const bool need3 = l3 < 0x7F80u && (l3 < 0x0400u || s + kSwigluMargin3 > l3 + kBf16ExpBias128);
    return need1 || need3;
}

}  // namespace mi8
