// Locating a row tile's group in a device-resident list of group sizes (the ragged row groups of a dropless-MoE
// expert layer); shared by the grouped GEMM problems and the grouped cast / SwiGLU kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi8 {
namespace gemm {
namespace {

// ---- locating a group in the device-resident size list ---------------------------------------------------
// Groups are consecutive row ranges; sizes are clamped so that their running sum never passes T.  A group of
// m rows owns ceil(m / U) "units" (row tiles).  The 64 lanes of a wave each take one group of a 64-group chunk
// and prefix-sum rows and units with shuffles, so a lookup costs one load latency instead of E dependent
// ones.  Must be called by all lanes of the wave together; the result is wave-uniform.
struct GroupSpan {
    int e;                 // group index (E if the key is past the end)
    int64_t rows_before;   // rows of the groups before it
    int64_t m;             // its clamped size
    int64_t units_before;  // units of the groups before it (all units if the key is past the end)
};

__device__ __forceinline__ int64_t uniform64(int64_t v)
{
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ int64_t wave_inclusive_sum(int64_t v, int lane)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int64_t o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}

// BY_UNIT: key is a unit index, find the group that owns it; otherwise key is the group index itself.
template <int U, bool BY_UNIT>
__device__ __forceinline__ GroupSpan locate_group(const int64_t* sizes, int E, int64_t T, int64_t key)
{
    const int lane = (int)threadIdx.x & 63;
    int64_t rows_c = 0, units_c = 0;
    for (int base = 0; base < E; base += 64) {
        const int e = base + lane;
        int64_t m = (e < E) ? sizes[e] : 0;
        m = m < 0 ? 0 : (m > T ? T : m);
        int64_t end = rows_c + wave_inclusive_sum(m, lane);
        int64_t start = end - m;
        end = end < T ? end : T;
        start = start < T ? start : T;
        const int64_t me = end - start;
        const int64_t un = (me + U - 1) / U;
        const int64_t uend = units_c + wave_inclusive_sum(un, lane);
        const bool hit = (e < E) && (BY_UNIT ? key < uend : key == e);
        const uint64_t mask = __ballot(hit);
        if (mask) {
            const int src = __ffsll((unsigned long long)mask) - 1;
            GroupSpan r;
            r.e = base + src;
            r.rows_before = uniform64(__shfl(start, src, 64));
            r.m = uniform64(__shfl(me, src, 64));
            r.units_before = uniform64(__shfl(uend - un, src, 64));
            return r;
        }
        rows_c = uniform64(__shfl(end, 63, 64));
        units_c = uniform64(__shfl(uend, 63, 64));
    }
    return GroupSpan{E, rows_c, 0, units_c};
}

}  // namespace
}  // namespace gemm
}  // namespace mi8
