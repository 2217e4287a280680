// amax of the two SwiGLU gradients (g1, g3 of h = silu(x1) * x3) without computing every element.
//
// The tensorwise cast of g1 and g3 needs their global amax before a single byte can be written, and computing the
// gradients costs a pass over gh, x1 and x3 (6 bytes and about 28 vector instructions per element).  Instead:
//   1. the kernels that produce the tensors leave one 16-bit code per row segment (64 consecutive columns of a
//      row): the largest magnitude in it, as the integer L of mi8_swiglu.h - one code array for gh (written by the
//      epilogue of the GEMM that computes it) and one for the larger of x1 and x3 (written by the fused forward
//      launch); mi8_rowseg_max_codes computes the same arrays from tensors in memory,
//   2. the sum of a segment's two codes bounds log2 of both gradients on all of its elements; the segments whose
//      sums come close to the largest sum are computed exactly, and their maxima are thresholds,
//   3. every other segment whose sum exceeds the thresholds is computed exactly as well.
// A segment that is never computed has all its elements below a value that some computed element reached, so the
// result is the exact amax, whatever order the segments are visited in.  On activations without heavy tails steps
// 2 and 3 touch well under a percent of the segments.
//
// Codes are uint16 [ceil(cols / 64)][rows]: the codes of one column block are contiguous over the rows.
#include "mi8_swiglu.h"

namespace mi8 {
namespace {

constexpr int kThreads = 256;
// step 2 takes the segments within this distance of the largest sum (2^(-64 / 128) = 0.71 of the largest bound)
constexpr uint32_t kSeedSlack = 64;

__device__ __forceinline__ uint32_t absmax_packed8(uint4 v)
{
    return (max_code8(v.x, v.y, v.z, v.w) & 0xFFFFu) << 16;
}

// ---- codes of one or two tensors in memory: eight lanes per segment ------------------------------------------
__global__ __launch_bounds__(kThreads) void rowseg_codes_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
                                                                int64_t rows, int64_t cols, int64_t nseg,
                                                                uint16_t* __restrict__ codes)
{
    const int sub = threadIdx.x & 7;
    const int64_t seg = (int64_t)blockIdx.x * (kThreads / 8) + (threadIdx.x >> 3);  // = cb * rows + r
    uint32_t m = 0;
    if (seg < nseg) {
        const int64_t cb = seg / rows, r = seg % rows;
        const int64_t c = cb * kSegCols + sub * 8;
        if (c < cols) {
            const uint4 va = *reinterpret_cast<const uint4*>(a + r * cols + c);
            m = max_code8(va.x, va.y, va.z, va.w);
            if (b) {
                const uint4 vb = *reinterpret_cast<const uint4*>(b + r * cols + c);
                m = pk_umax16(m, max_code8(vb.x, vb.y, vb.z, vb.w));
            }
        }
    }
    m &= 0xFFFFu;
    m = umax32(m, (uint32_t)__shfl_xor((int)m, 1, 64));
    m = umax32(m, (uint32_t)__shfl_xor((int)m, 2, 64));
    m = umax32(m, (uint32_t)__shfl_xor((int)m, 4, 64));
    if (sub == 0 && seg < nseg) codes[seg] = (uint16_t)m;
}

// ---- the largest sum ------------------------------------------------------------------------------------------------
// Every lane of the scans below takes eight consecutive segments (one 16-byte load per code array), every wave 512.
// state: [0] amax bits of g1, [1] of g3, [2] n = workgroups per launch, [4 .. 4 + n) one partial maximum of the sums per
// workgroup of the first scan, then n partial maxima of g1 and n of g3 from the seeds (no atomics there, nothing to
// clear beforehand: the first scan's first workgroup zeroes [0] and [1]).
constexpr int kSegsPerLane = 8, kSegsPerWave = 64 * kSegsPerLane, kSegsPerBlock = (kThreads / 64) * kSegsPerWave;
constexpr int kStateHeader = 4;

// the eight sums of a lane (zero beyond the end of the arrays)
__device__ __forceinline__ void load_sums(const uint16_t* __restrict__ gc, const uint16_t* __restrict__ xc, int64_t first,
                                          int64_t nseg, uint32_t (&s)[kSegsPerLane])
{
    if (first + kSegsPerLane <= nseg) {
        const uint4 g = *reinterpret_cast<const uint4*>(gc + first), x = *reinterpret_cast<const uint4*>(xc + first);
        const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, xw[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            s[2 * k] = (gw[k] & 0xFFFFu) + (xw[k] & 0xFFFFu);
            s[2 * k + 1] = (gw[k] >> 16) + (xw[k] >> 16);
        }
    } else {
#pragma unroll
        for (int k = 0; k < kSegsPerLane; ++k) s[k] = first + k < nseg ? (uint32_t)gc[first + k] + (uint32_t)xc[first + k] : 0u;
    }
}

__global__ __launch_bounds__(kThreads) void swiglu_max_sum_kernel(const uint16_t* __restrict__ gc, const uint16_t* __restrict__ xc,
                                                                  int64_t nseg, uint32_t* __restrict__ state)
{
    __shared__ uint32_t smem[kThreads / 64];
    uint32_t s[kSegsPerLane];
    load_sums(gc, xc, ((int64_t)blockIdx.x * kThreads + threadIdx.x) * kSegsPerLane, nseg, s);
    uint32_t m = 0;
#pragma unroll
    for (int k = 0; k < kSegsPerLane; ++k) m = umax32(m, s[k]);
    m = wave_umax(m);
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        state[kStateHeader + blockIdx.x] = umax32(umax32(smem[0], smem[1]), umax32(smem[2], smem[3]));
        if (blockIdx.x == 0) {
            state[0] = 0;
            state[1] = 0;
            state[2] = gridDim.x;
        }
    }
}

// ---- exact maxima of the segments that need them ----------------------------------------------------------------
// SEED: segments whose sums are within kSeedSlack of the largest (or may hold a non-finite input); every workgroup
// leaves its two maxima as partials (a thousand atomics on one word would take longer than the scan).  Otherwise:
// the thresholds are the maxima of those partials, and the remaining segments whose sums exceed them are computed;
// what they find is merged with the thresholds by atomics (few: only a wave that can raise a value asks).
// A wave lists the flagged ones among its 512 segments in LDS, and its eight groups of eight lanes compute them,
// eight segments at a time.
template <bool SEED>
__global__ __launch_bounds__(kThreads) void swiglu_sparse_amax_kernel(const uint16_t* __restrict__ x1,
                                                                      const uint16_t* __restrict__ x3,
                                                                      const uint16_t* __restrict__ gh, int64_t rows,
                                                                      int64_t cols, int64_t nseg,
                                                                      const uint16_t* __restrict__ gc,
                                                                      const uint16_t* __restrict__ xc,
                                                                      uint32_t* __restrict__ state)
{
    __shared__ uint16_t picked[kThreads / 64][kSegsPerWave];
    __shared__ int32_t n_picked[kThreads / 64];
    __shared__ uint32_t smem[3][kThreads / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane & 7, grp = lane >> 3;
    const int n = (int)state[2];  // = gridDim.x of all three launches
    uint32_t* const seed1 = state + kStateHeader + n;
    uint32_t* const seed3 = seed1 + n;
    // the largest sum (and, after the seeds, the thresholds): maxima over the previous launch's partials
    uint32_t top = 0, t1 = 0, t3 = 0;
    for (int i = threadIdx.x; i < n; i += kThreads) {
        top = umax32(top, state[kStateHeader + i]);
        if (!SEED) {
            t1 = umax32(t1, seed1[i]);
            t3 = umax32(t3, seed3[i]);
        }
    }
    top = wave_umax(top);
    t1 = wave_umax(t1);
    t3 = wave_umax(t3);
    if (lane == 0) {
        smem[0][wave] = top;
        smem[1][wave] = t1;
        smem[2][wave] = t3;
        n_picked[wave] = 0;
    }
    __syncthreads();
    top = umax32(umax32(smem[0][0], smem[0][1]), umax32(smem[0][2], smem[0][3]));
    t1 = umax32(umax32(smem[1][0], smem[1][1]), umax32(smem[1][2], smem[1][3]));
    t3 = umax32(umax32(smem[2][0], smem[2][1]), umax32(smem[2][2], smem[2][3]));
    __syncthreads();
    if (!SEED && blockIdx.x == 0 && threadIdx.x == 0) {  // the result starts from the seeds' maxima
        atomicMax(&state[0], t1);
        atomicMax(&state[1], t3);
    }

    const int64_t wave_first = ((int64_t)blockIdx.x * (kThreads / 64) + wave) * kSegsPerWave;
    uint32_t s[kSegsPerLane];
    load_sums(gc, xc, wave_first + lane * kSegsPerLane, nseg, s);
#pragma unroll
    for (int k = 0; k < kSegsPerLane; ++k) {
        const bool in_range = wave_first + lane * kSegsPerLane + k < nseg;
        const bool seed = s[k] >= 0x7F80u || s[k] + kSeedSlack >= top;
        const bool need = in_range && (SEED ? seed : (!seed && swiglu_segment_needed(s[k], t1, t3)));
        if (need) picked[wave][atomicAdd(&n_picked[wave], 1)] = (uint16_t)(lane * kSegsPerLane + k);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int count = n_picked[wave];
    uint32_t m1 = 0, m3 = 0;
    for (int k = grp; k < count; k += 8) {
        const int64_t seg = wave_first + picked[wave][k];
        const int64_t cb = seg / rows, r = seg % rows;
        const int64_t c = cb * kSegCols + sub * 8;
        if (c < cols) {
            const int64_t off = r * cols + c;
            uint4 p1, p3;
            swiglu_bwd8(*reinterpret_cast<const uint4*>(x1 + off), *reinterpret_cast<const uint4*>(x3 + off),
                        *reinterpret_cast<const uint4*>(gh + off), p1, p3);
            m1 = umax32(m1, absmax_packed8(p1));
            m3 = umax32(m3, absmax_packed8(p3));
        }
    }
    m1 = wave_umax(m1);
    m3 = wave_umax(m3);
    if (SEED) {
        if (lane == 0) {
            smem[1][wave] = m1;
            smem[2][wave] = m3;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            seed1[blockIdx.x] = umax32(umax32(smem[1][0], smem[1][1]), umax32(smem[1][2], smem[1][3]));
            seed3[blockIdx.x] = umax32(umax32(smem[2][0], smem[2][1]), umax32(smem[2][2], smem[2][3]));
        }
    } else if (lane == 0) {
        if (m1 > t1 && m1 > __hip_atomic_load(&state[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(&state[0], m1);
        if (m3 > t3 && m3 > __hip_atomic_load(&state[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(&state[1], m3);
    }
}

}  // namespace
}  // namespace mi8

using namespace mi8;

extern "C" int64_t mi8_rowseg_code_count(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0) return 0;
    return rows * ceil_div(cols, kSegCols);
}

extern "C" int64_t mi8_swiglu_amax_state_words(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0) return 0;
    return kStateHeader + 3 * ceil_div(rows * ceil_div(cols, kSegCols), kSegsPerBlock);
}

extern "C" int mi8_rowseg_max_codes(const void* a, const void* b, int64_t rows, int64_t cols, uint16_t* codes, void* stream)
{
    MI8_REQUIRE(a && codes, MI8_ERR_ARG, "mi8_rowseg_max_codes: null pointer");
    MI8_REQUIRE(rows > 0 && cols > 0 && cols % 8 == 0, MI8_ERR_UNSUPPORTED,
                "mi8_rowseg_max_codes: needs rows > 0 and cols (%lld) a positive multiple of 8", (long long)cols);
    MI8_REQUIRE(aligned16(a) && aligned16(b), MI8_ERR_UNSUPPORTED, "mi8_rowseg_max_codes: tensors must be 16-byte aligned");
    const int64_t nseg = rows * ceil_div(cols, kSegCols);
    MI8_REQUIRE(nseg < ((int64_t)1 << 31), MI8_ERR_UNSUPPORTED, "mi8_rowseg_max_codes: tensor too large");
    hipLaunchKernelGGL(rowseg_codes_kernel, dim3((unsigned)ceil_div(nseg, kThreads / 8)), dim3(kThreads), 0, (hipStream_t)stream,
                       (const uint16_t*)a, (const uint16_t*)b, rows, cols, nseg, codes);
    return launch_status("mi8_rowseg_max_codes");
}

extern "C" int mi8_swiglu_bwd_amax_from_codes(const void* x1, const void* x3, const void* gh, int64_t rows, int64_t cols,
                                              const uint16_t* gh_codes, const uint16_t* x_codes, uint32_t* state, void* stream)
{
    MI8_REQUIRE(x1 && x3 && gh && gh_codes && x_codes && state, MI8_ERR_ARG, "mi8_swiglu_bwd_amax_from_codes: null pointer");
    MI8_REQUIRE(rows > 0 && cols > 0 && cols % 8 == 0, MI8_ERR_UNSUPPORTED,
                "mi8_swiglu_bwd_amax_from_codes: needs rows > 0 and cols (%lld) a positive multiple of 8", (long long)cols);
    MI8_REQUIRE(aligned16(x1) && aligned16(x3) && aligned16(gh), MI8_ERR_UNSUPPORTED,
                "mi8_swiglu_bwd_amax_from_codes: tensors must be 16-byte aligned");
    const int64_t nseg = rows * ceil_div(cols, kSegCols);
    MI8_REQUIRE(nseg < ((int64_t)1 << 31), MI8_ERR_UNSUPPORTED, "mi8_swiglu_bwd_amax_from_codes: tensor too large");
    MI8_REQUIRE(aligned16(gh_codes) && aligned16(x_codes), MI8_ERR_UNSUPPORTED,
                "mi8_swiglu_bwd_amax_from_codes: code arrays must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)ceil_div(nseg, kSegsPerBlock);
    hipLaunchKernelGGL(swiglu_max_sum_kernel, dim3(grid), dim3(kThreads), 0, st, gh_codes, x_codes, nseg, state);
    hipLaunchKernelGGL((swiglu_sparse_amax_kernel<true>), dim3(grid), dim3(kThreads), 0, st, (const uint16_t*)x1,
                       (const uint16_t*)x3, (const uint16_t*)gh, rows, cols, nseg, gh_codes, x_codes, state);
    hipLaunchKernelGGL((swiglu_sparse_amax_kernel<false>), dim3(grid), dim3(kThreads), 0, st, (const uint16_t*)x1,
                       (const uint16_t*)x3, (const uint16_t*)gh, rows, cols, nseg, gh_codes, x_codes, state);
    return launch_status("mi8_swiglu_bwd_amax_from_codes");
}
