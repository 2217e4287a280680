// SwiGLU pointwise kernels of the feed-forward block, with the amax reduction of their outputs fused in so
// that the tensorwise cast that follows needs no separate pass over the (largest) activation tensor.
// Rounding points follow torch's eager bf16 evaluation: every elementwise op computes in fp32 and rounds
// its result to bf16 before the next op reads it.
#include "mi8_swiglu.h"

namespace mi8 {
namespace {

constexpr int kThreads = 256;

// max over |bf16| of the 8 packed values, as a float32 bit pattern
__device__ __forceinline__ uint32_t absmax_packed(uint4 v)
{
    uint32_t m = 0;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        m = umax32(m, (w[i] & 0x7FFFu) << 16);
        m = umax32(m, w[i] & 0x7FFF0000u);
    }
    return m;
}

__device__ __forceinline__ void publish_block_max(uint32_t m, uint32_t* slots)
{
    __shared__ uint32_t smem[4];
    m = wave_umax(m);
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) slots[blockIdx.x] = umax32(umax32(smem[0], smem[1]), umax32(smem[2], smem[3]));
}

__global__ __launch_bounds__(kThreads) void swiglu_fwd_kernel(const uint4* __restrict__ x1,
                                                              const uint4* __restrict__ x3, uint4* __restrict__ h,
                                                              int64_t nvec, uint32_t* __restrict__ slots)
{
    uint32_t m = 0;
    // every workgroup streams its own contiguous range, two vectors per lane in flight
    const BlockRange r = block_range(nvec);
    int64_t i = r.lo + threadIdx.x;
    for (; i + kThreads < r.hi; i += 2 * kThreads) {
        const uint4 a0 = x1[i], b0 = x3[i], a1 = x1[i + kThreads], b1 = x3[i + kThreads];
        const uint4 o0 = swiglu_fwd8(a0, b0), o1 = swiglu_fwd8(a1, b1);
        h[i] = o0;
        h[i + kThreads] = o1;
        m = umax32(m, umax32(absmax_packed(o0), absmax_packed(o1)));
    }
    for (; i < r.hi; i += kThreads) {
        const uint4 out = swiglu_fwd8(x1[i], x3[i]);
        h[i] = out;
        m = umax32(m, absmax_packed(out));
    }
    if (slots) publish_block_max(m, slots);
}

__global__ __launch_bounds__(kThreads) void swiglu_bwd_kernel(const uint4* __restrict__ x1,
                                                              const uint4* __restrict__ x3,
                                                              const uint4* __restrict__ gh, uint4* __restrict__ g1,
                                                              uint4* __restrict__ g3, int64_t nvec,
                                                              uint32_t* __restrict__ slots1,
                                                              uint32_t* __restrict__ slots3)
{
    uint32_t m1 = 0, m3 = 0;
    // every workgroup streams its own contiguous range, two vectors of each input per lane in flight
    const BlockRange r = block_range(nvec);
    int64_t i = r.lo + threadIdx.x;
    for (; i + kThreads < r.hi; i += 2 * kThreads) {
        const uint4 a0 = x1[i], b0 = x3[i], c0 = gh[i];
        const uint4 a1 = x1[i + kThreads], b1 = x3[i + kThreads], c1 = gh[i + kThreads];
        uint4 p1, p3, q1, q3;
        swiglu_bwd8(a0, b0, c0, p1, p3);
        swiglu_bwd8(a1, b1, c1, q1, q3);
        if (g1) {  // (without outputs: only the amax of what would be written)
            g1[i] = p1;
            g3[i] = p3;
            g1[i + kThreads] = q1;
            g3[i + kThreads] = q3;
        }
        m1 = umax32(m1, umax32(absmax_packed(p1), absmax_packed(q1)));
        m3 = umax32(m3, umax32(absmax_packed(p3), absmax_packed(q3)));
    }
    for (; i < r.hi; i += kThreads) {
        uint4 p1, p3;
        swiglu_bwd8(x1[i], x3[i], gh[i], p1, p3);
        if (g1) {
            g1[i] = p1;
            g3[i] = p3;
        }
        m1 = umax32(m1, absmax_packed(p1));
        m3 = umax32(m3, absmax_packed(p3));
    }
    if (slots1) publish_block_max(m1, slots1);
    if (slots3) {
        __syncthreads();
        publish_block_max(m3, slots3);
    }
}

}  // namespace
}  // namespace mi8

using namespace mi8;

extern "C" int mi8_swiglu_fwd(const void* x1, const void* x3, void* h, int64_t n, uint32_t* slots_h, void* stream)
{
    MI8_REQUIRE(x1 && x3 && h, MI8_ERR_ARG, "mi8_swiglu_fwd: null pointer");
    MI8_REQUIRE(n > 0 && n % 8 == 0, MI8_ERR_UNSUPPORTED, "mi8_swiglu_fwd: n (%lld) must be a positive multiple of 8",
                (long long)n);
    MI8_REQUIRE(aligned16(x1) && aligned16(x3) && aligned16(h), MI8_ERR_UNSUPPORTED,
                "mi8_swiglu_fwd: pointers must be 16-byte aligned");
    const int blocks = mi8_amax_slots_for(n);
    hipLaunchKernelGGL(swiglu_fwd_kernel, dim3(blocks), dim3(kThreads), 0, (hipStream_t)stream, (const uint4*)x1,
                       (const uint4*)x3, (uint4*)h, n / 8, slots_h);
    return launch_status("mi8_swiglu_fwd");
}

extern "C" int mi8_swiglu_bwd(const void* x1, const void* x3, const void* gh, void* g1, void* g3, int64_t n,
                              uint32_t* slots_g1, uint32_t* slots_g3, void* stream)
{
    MI8_REQUIRE(x1 && x3 && gh, MI8_ERR_ARG, "mi8_swiglu_bwd: null pointer");
    MI8_REQUIRE((g1 != nullptr) == (g3 != nullptr), MI8_ERR_ARG, "mi8_swiglu_bwd: give both outputs or neither");
    MI8_REQUIRE(g1 || (slots_g1 && slots_g3), MI8_ERR_ARG, "mi8_swiglu_bwd: nothing to compute");
    MI8_REQUIRE(n > 0 && n % 8 == 0, MI8_ERR_UNSUPPORTED, "mi8_swiglu_bwd: n (%lld) must be a positive multiple of 8",
                (long long)n);
    MI8_REQUIRE(aligned16(x1) && aligned16(x3) && aligned16(gh) && aligned16(g1) && aligned16(g3),
                MI8_ERR_UNSUPPORTED, "mi8_swiglu_bwd: pointers must be 16-byte aligned");
    const int blocks = mi8_amax_slots_for(n);
    hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(blocks), dim3(kThreads), 0, (hipStream_t)stream, (const uint4*)x1,
                       (const uint4*)x3, (const uint4*)gh, (uint4*)g1, (uint4*)g3, n / 8, slots_g1, slots_g3);
    return launch_status("mi8_swiglu_bwd");
}
