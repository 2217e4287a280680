// The general fp8 GEMM tile routine (any M, N; K % 16 == 0), shared by the dense and grouped kernels.
#pragma once
#include "mi8_gemm.h"

namespace mi8 {
namespace gemm {

// One BM x BN output tile of C = A . B^T with register-staged global->LDS copies (general shapes: any M, N;
// K % 16 == 0, possibly 0).  Shared by the dense kernel and the grouped kernels, which call it on a per-group
// view of the operands.  `lds` must hold 2 * (BM + BN) * 128 bytes.
template <int BM, int BN, int WM, int WN, int CBSZ, int BLGP>
__device__ __forceinline__ void gemm_tile_body(const GemmArgs& g, const int m0, const int n0, uint8_t* lds)
{
    constexpr int NT = WM * WN * 64;
    constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
    constexpr int TM = WTM / 32, TN = WTN / 32;  // 32x32 MFMA tiles per wave
    constexpr int ROWS_PER_PASS = NT / 8;        // 8 lanes x 16 bytes cover one 128-byte row
    constexpr int PA = BM / ROWS_PER_PASS, PB = BN / ROWS_PER_PASS;
    constexpr int STAGE = (BM + BN) * BK;
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile/threads mismatch");

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, half = lane >> 5;

    // ---- global -> register staging: this lane's rows and 16-byte chunk --------------------------
    const int ld_row = tid >> 3, ld_chunk = tid & 7;
    uint32_t a_off[PA], b_off[PB];
#pragma unroll
    for (int p = 0; p < PA; ++p) {
        int r = m0 + p * ROWS_PER_PASS + ld_row;
        r = r < g.M ? r : g.M - 1;  // rows past the edge re-read the last row; never stored
        a_off[p] = (uint32_t)((int64_t)r * g.lda + ld_chunk * 16);
    }
#pragma unroll
    for (int p = 0; p < PB; ++p) {
        int r = n0 + p * ROWS_PER_PASS + ld_row;
        r = r < g.N ? r : g.N - 1;
        b_off[p] = (uint32_t)((int64_t)r * g.ldb + ld_chunk * 16);
    }
    // LDS store position of this lane's chunk inside a stage (same for every pass up to the row offset)
    uint32_t st_off[(PA > PB ? PA : PB)];
#pragma unroll
    for (int p = 0; p < (PA > PB ? PA : PB); ++p) {
        const int r = p * ROWS_PER_PASS + ld_row;
        st_off[p] = (uint32_t)(r * BK + ((ld_chunk ^ swz(r)) << 4));
    }

    uint4 ra[PA], rb[PB];
    auto load_tile = [&](int kt) {
        const int k = kt * BK + ld_chunk * 16;
        const bool ok = k < g.K;
        const uint8_t* ap = g.A + (int64_t)kt * BK;
        const uint8_t* bp = g.B + (int64_t)kt * BK;
#pragma unroll
        for (int p = 0; p < PA; ++p)
            ra[p] = ok ? *reinterpret_cast<const uint4*>(ap + a_off[p]) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int p = 0; p < PB; ++p)
            rb[p] = ok ? *reinterpret_cast<const uint4*>(bp + b_off[p]) : make_uint4(0, 0, 0, 0);
    };
    auto store_tile = [&](int stage) {
        uint8_t* sa_ = lds + stage * STAGE;
        uint8_t* sb_ = sa_ + BM * BK;
#pragma unroll
        for (int p = 0; p < PA; ++p) *reinterpret_cast<uint4*>(sa_ + st_off[p]) = ra[p];
#pragma unroll
        for (int p = 0; p < PB; ++p) *reinterpret_cast<uint4*>(sb_ + st_off[p]) = rb[p];
    };

    // ---- fragment read offsets (row part; the chunk part depends on the k sub-step) --------------
    // lane l feeds row (l % 32) of a 32-row tile with K bytes [32*half, 32*half+32) of the 64-byte sub-step
    uint32_t fa_row[TM], fb_row[TN];
    int fa_swz[TM], fb_swz[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int r = wm * WTM + i * 32 + l32;
        fa_row[i] = (uint32_t)(r * BK);
        fa_swz[i] = swz(r);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int r = wn * WTN + j * 32 + l32;
        fb_row[j] = (uint32_t)(BM * BK + r * BK);
        fb_swz[j] = swz(r);
    }

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const int nk = (g.K + BK - 1) / BK;
    if (nk > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) load_tile(kt + 1);
        const uint8_t* st = lds + cur * STAGE;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int c0 = 4 * kk + 2 * half;
            v8i fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const v4i lo = *reinterpret_cast<const v4i*>(st + fa_row[i] + (((c0) ^ fa_swz[i]) << 4));
                const v4i hi = *reinterpret_cast<const v4i*>(st + fa_row[i] + (((c0 + 1) ^ fa_swz[i]) << 4));
                fa[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const v4i lo = *reinterpret_cast<const v4i*>(st + fb_row[j] + (((c0) ^ fb_swz[j]) << 4));
                const v4i hi = *reinterpret_cast<const v4i*>(st + fb_row[j] + (((c0 + 1) ^ fb_swz[j]) << 4));
                fb[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], CBSZ, BLGP,
                                                                                 0, 0, 0, 0);
        }
        if (kt + 1 < nk) store_tile(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue: scale, round to bf16, store ------------------------------------------------------
    // accumulator element e of lane l is C[row = 8*(e/4) + 4*(l/32) + e%4][col = l%32] of its 32x32 tile.
    // Scalar scales are inverted with an IEEE division; per-row / per-column scale vectors with v_rcp_f32
    // (exact for the power-of-two scales of the axiswise recipes, within 1 ulp otherwise).
    float isb[TN];
    bool col_ok[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn * WTN + j * 32 + l32;
        col_ok[j] = col < g.N;
        isb[j] = g.sb_vec ? (col_ok[j] ? __builtin_amdgcn_rcpf(g.sb[col]) : 0.0f) : g.sb ? 1.0f / g.sb[0] : 1.0f;
    }
    const float isa_scalar = g.sa_vec ? 0.0f : g.sa ? 1.0f / g.sa[0] : 1.0f;  // (null: the raw sums are wanted)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int row = m0 + wm * WTM + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
            if (row >= g.M) continue;
            const float isa = g.sa_vec ? __builtin_amdgcn_rcpf(g.sa[row]) : isa_scalar;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (!col_ok[j]) continue;
                const int col = n0 + wn * WTN + j * 32 + l32;
                const float v = acc[i][j][e] * isa * isb[j];
                if (g.c_f32) {
                    float* c = reinterpret_cast<float*>(g.C) + (int64_t)row * g.ldc + col;
                    *c = g.accumulate ? *c + v : v;
                } else {
                    uint16_t* c = reinterpret_cast<uint16_t*>(g.C) + (int64_t)row * g.ldc + col;
                    uint16_t r = f32_to_bf16_bits(v);
                    if (g.accumulate)  // both terms are bf16 values, summed in float32 and rounded once
                        r = f32_to_bf16_bits(bits_to_f32((uint32_t)*c << 16) + bits_to_f32((uint32_t)r << 16));
                    *c = r;
                }
            }
        }
    }
}


}  // namespace gemm
}  // namespace mi8
