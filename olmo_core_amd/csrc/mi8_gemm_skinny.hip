// Scaled float8 GEMM for a few rows of A:  C[M,N] = (A[M,K] . B[N,K]^T) * (1/sa) * (1/sb),  M <= 64.
//
// This is the shape of a generation loop (a handful of tokens against a weight matrix): the arithmetic is
// nothing, the time is reading B once, so the kernel is built to keep HBM busy rather than the matrix cores.
// A tiled kernel does badly here: the few tiles it finds occupy a few compute units, and each walks all of K
// with one memory latency per 128-byte step.
//
// One workgroup owns 16 (M <= 16) or 32 rows of B (columns of C) and all of A; its eight waves each take a
// contiguous eighth of K, so N/16 or N/32 workgroups x 8 waves stream disjoint pieces of B straight from global
// memory into MFMA operand registers (no LDS staging: nothing is reused inside a wave).  v_mfma_f32_16x16x128
// takes 16 rows x 128 bytes per operand, lane l feeding bytes 32*(l/16)..+31 of row l%16 - the B rows go in
// as the first operand, blocks of 16 rows of A as the second, and the 16 x 16 result is C transposed:
// element j of lane l is C[m = l%16][n = 4*(l/16) + j].  Loads of several 128-byte steps are issued before
// the first MFMA of a batch so that every wave has a few KB in flight.  The eight partial results meet in
// LDS and waves 0..MT-1 scale, round and store one block of 16 rows of C each.
//
// A (at most 64 x K bytes) is re-read by every workgroup and stays in L2; with more than 16 rows of A that
// traffic would exceed the read of B, so a workgroup then takes 32 rows of B per pass over A.  Rows of A past M and rows of B past N
// are clamped to the last valid row and their results dropped; K bytes past K (K % 16 == 0) are fed as zeros.
#include "mi8_gemm.h"

namespace mi8 {
namespace gemm {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kSkinnyWaves = 8;  // K slices per workgroup
constexpr int kStep = 128;       // K bytes per MFMA

// 16 bytes of an operand row, or zeros past the end of K
__device__ __forceinline__ v4i load16(const uint8_t* p, bool ok)
{
    return ok ? *reinterpret_cast<const v4i*>(p) : v4i{0, 0, 0, 0};
}

// MT: blocks of 16 rows of A; NB: blocks of 16 rows of B per workgroup (each wave's A fragments serve NB MFMAs,
// which divides the L2 traffic of re-reading A by NB); U: 128-byte steps loaded ahead of their MFMAs; TW / TX:
// MFMA type codes of the B rows (first operand) and the A rows (second operand), 0 = e4m3, 1 = e5m2.
template <int MT, int NB, int U, int TW, int TX>
__global__ __launch_bounds__(kSkinnyWaves * 64) void gemm_fp8_skinny_kernel(GemmArgs g)
{
    __shared__ v4f red[kSkinnyWaves][MT][64];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kg = lane >> 4;
    const int n0 = (int)blockIdx.x * (16 * NB);

    const uint8_t* wp[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int n = n0 + nb * 16 + r16 < g.N ? n0 + nb * 16 + r16 : g.N - 1;
        wp[nb] = g.B + (int64_t)n * g.ldb + kg * 32;
    }
    const uint8_t* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r16 < g.M ? mt * 16 + r16 : g.M - 1;
        xp[mt] = g.A + (int64_t)m * g.lda + kg * 32;
    }

    const int steps = (g.K + kStep - 1) / kStep;
    const int per_wave = (steps + kSkinnyWaves - 1) / kSkinnyWaves;
    const int s_begin = wave * per_wave;
    const int s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;

    v4f acc[NB][MT];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nb][mt] = v4f{0, 0, 0, 0};

    for (int s = s_begin; s < s_end; s += U) {
        v4i w[U][NB][2], x[U][MT][2];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t off = (int64_t)(s + u) * kStep;
            const int k = (s + u) * kStep + kg * 32;  // this lane's first K byte of the step
            const bool in = s + u < s_end;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const bool ok = in && k + 16 * h < g.K;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) w[u][nb][h] = load16(wp[nb] + off + 16 * h, ok);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) x[u][mt][h] = load16(xp[mt] + off + 16 * h, ok);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const v8i fx = __builtin_shufflevector(x[u][mt][0], x[u][mt][1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    const v8i fw = __builtin_shufflevector(w[u][nb][0], w[u][nb][1], 0, 1, 2, 3, 4, 5, 6, 7);
                    acc[nb][mt] =
                        __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fw, fx, acc[nb][mt], TW, TX, 0, 0, 0, 0);
                }
            }
        }
    }

    // same scale arithmetic as the tiled kernels: IEEE division for single scales, v_rcp_f32 for scale vectors
    const int m = (wave < MT ? wave : 0) * 16 + r16;  // wave mt finishes block mt of the rows of A
    const bool m_ok = wave < MT && m < g.M;
    const float isa = !m_ok ? 0.0f : g.sa_vec ? __builtin_amdgcn_rcpf(g.sa[m]) : 1.0f / g.sa[0];
    const float isb_scalar = g.sb_vec ? 0.0f : 1.0f / g.sb[0];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        if (nb > 0) __syncthreads();  // the previous block's sums have been read
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) red[wave][mt][lane] = acc[nb][mt];
        __syncthreads();
        if (!m_ok) continue;
        v4f sum = red[0][wave][lane];
#pragma unroll
        for (int w2 = 1; w2 < kSkinnyWaves; ++w2) sum += red[w2][wave][lane];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + nb * 16 + kg * 4 + j;
            if (n >= g.N) continue;
            const float isb = g.sb_vec ? __builtin_amdgcn_rcpf(g.sb[n]) : isb_scalar;
            const float v = sum[j] * isa * isb;
            if (g.c_f32)
                reinterpret_cast<float*>(g.C)[(int64_t)m * g.ldc + n] = v;
            else
                reinterpret_cast<uint16_t*>(g.C)[(int64_t)m * g.ldc + n] = f32_to_bf16_bits(v);
        }
    }
}

template <int MT, int NB, int U>
int launch_skinny_typed(const GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st)
{
    const dim3 grid((g.N + 16 * NB - 1) / (16 * NB)), block(kSkinnyWaves * 64);
    const bool we5 = b_dtype == MI8_E5M2, xe5 = a_dtype == MI8_E5M2;
    if (!we5 && !xe5) hipLaunchKernelGGL((gemm_fp8_skinny_kernel<MT, NB, U, 0, 0>), grid, block, 0, st, g);
    if (!we5 && xe5) hipLaunchKernelGGL((gemm_fp8_skinny_kernel<MT, NB, U, 0, 1>), grid, block, 0, st, g);
    if (we5 && !xe5) hipLaunchKernelGGL((gemm_fp8_skinny_kernel<MT, NB, U, 1, 0>), grid, block, 0, st, g);
    if (we5 && xe5) hipLaunchKernelGGL((gemm_fp8_skinny_kernel<MT, NB, U, 1, 1>), grid, block, 0, st, g);
    return launch_status("mi8_gemm_fp8");
}

}  // namespace

int launch_skinny(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st)
{
    if (g.M > kSkinnyMaxM) {
        set_error("mi8_gemm_fp8: the few-rows variant takes M <= %d (M=%d)", kSkinnyMaxM, g.M);
        return MI8_ERR_UNSUPPORTED;
    }
    if (g.M <= 16) return launch_skinny_typed<1, 1, 4>(g, a_dtype, b_dtype, st);
    if (g.M <= 32) return launch_skinny_typed<2, 2, 2>(g, a_dtype, b_dtype, st);
    return launch_skinny_typed<4, 2, 2>(g, a_dtype, b_dtype, st);
}

}  // namespace gemm
}  // namespace mi8
