// Diagnostics: back-to-back fp8 MFMAs with nothing else running, on all-zero or on random operand registers.
// The rate on random operands is what the chip sustains under its power limit (the clock drops under matrix load),
// the rate on zeros what the matrix pipes do at full clock: the two numbers bracket what a GEMM can reach.
#include "mi8_common.h"

namespace mi8 {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t mix(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

// one wave: a 128 x 128 x 128 product per iteration from resident fragments (64 MFMAs of 16x16x128 or 32 of 32x32x64)
template <int MODE>
__global__ __launch_bounds__(256, 1) void mfma_loop_kernel(int iters, int random, float* __restrict__ sink)
{
    v8i a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t ra = mix(threadIdx.x * 131 + i * 17 + e + blockIdx.x * 7919);
            const uint32_t rb = mix(threadIdx.x * 257 + i * 29 + e * 3 + 1 + blockIdx.x * 104729);
            // random fp8 bytes of moderate magnitude, never NaN: the top exponent bit of every byte is cleared
            a[i][e] = random ? (int)(ra & 0xBFBFBFBFu) : 0;
            b[i][e] = random ? (int)(rb & 0xBFBFBFBFu) : 0;
        }
    float s = 0;
    if constexpr (MODE == 0) {
        v16f acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int x = 0; x < 16; ++x)
                    acc[x] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[(x & 3) + 4 * h], a[(x >> 2) + 4 * h], acc[x], 0, 0,
                                                                             0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += acc[i][e];
    } else {
        v4f acc[64];
#pragma unroll
        for (int i = 0; i < 64; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int x = 0; x < 64; ++x)
                acc[x] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[x & 7], a[x >> 3], acc[x], 0, 0, 0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 64; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) s += acc[i][e];
    }
    sink[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace
}  // namespace mi8

using namespace mi8;

extern "C" int mi8_probe_mfma_loop(int mfma_shape, int random_operands, int iterations, int workgroups, float* sink,
                                   void* stream)
{
    MI8_REQUIRE(sink, MI8_ERR_ARG, "mi8_probe_mfma_loop: sink is null");
    MI8_REQUIRE((mfma_shape == 0 || mfma_shape == 1) && iterations > 0 && iterations <= (1 << 22) && workgroups > 0 &&
                    workgroups <= 4096,
                MI8_ERR_ARG, "mi8_probe_mfma_loop: shape 0 (32x32x64) or 1 (16x16x128), 1..2^22 iterations, 1..4096 workgroups");
    hipStream_t st = (hipStream_t)stream;
    if (mfma_shape == 0)
        hipLaunchKernelGGL((mfma_loop_kernel<0>), dim3(workgroups), dim3(256), 0, st, iterations, random_operands, sink);
    else
        hipLaunchKernelGGL((mfma_loop_kernel<1>), dim3(workgroups), dim3(256), 0, st, iterations, random_operands, sink);
    return launch_status("mi8_probe_mfma_loop");
}
