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

}  // namespace mi8
