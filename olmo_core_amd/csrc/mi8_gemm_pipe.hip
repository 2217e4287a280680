// Software-pipelined, persistent variant of the scaled fp8 GEMM for K % 128 == 0.
//
// One workgroup of 4 waves per CU (one wave per SIMD, the full 512-register budget), 256 x 256 x 128 tiles,
// two LDS stages.  Each wave owns a 128 x 128 sub-tile = 4 x 4 MFMA tiles of 32x32x64 and runs this schedule
// per 128-byte K step (two 64-byte sub-steps s0, s1):
//
//     MFMA(s0 fragments, first half) | issue LDS reads of s1 fragments, LDS writes of the next stage (from
//     registers loaded one step ago), global loads of the stage after next | MFMA(s0, second half)
//     barrier
//     issue LDS reads of the next stage's s0 fragments | MFMA(s1 fragments)
//
// so that every LDS/global latency and the barrier wait sit behind 16 queued matrix instructions.
// The workgroup is persistent: it walks its XCD's share of the output tiles, which removes the per-tile launch
// gap and keeps the 32 workgroups of one XCD on neighbouring tiles (shared A/B panels in that XCD's L2).
// Operand roles are swapped in the MFMA (B fragments first) so that a lane ends up with four consecutive
// output columns per accumulator quad; the bf16 tile is then staged through LDS and written with 16-byte
// stores covering whole 256-byte row segments.
#include "mi8_gemm.h"

namespace mi8 {
namespace gemm {
namespace {

constexpr int BM = 256, BN = 256;
constexpr int WTM = 128, WTN = 128;
constexpr int TM = 4, TN = 4;
constexpr int NT = 256;
constexpr int P = 8;                      // 16-byte chunks per lane per operand per stage
constexpr int STAGE = (BM + BN) * BK;     // 64 KB
constexpr int LDS_BYTES = 2 * STAGE;      // 128 KB

struct Frags {
    v8i a[TM];
    v8i b[TN];
};

template <int CBSZ_A, int BLGP_B>
__global__ __launch_bounds__(NT, 1) void gemm_fp8_pipe_kernel(GemmArgs g)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;
    const int ld_row = tid >> 3, ld_chunk = tid & 7;

    // LDS store offset of this lane's chunk for rows ld_row + 32 p: swz(ld_row + 32 p) = swz(ld_row) ^ 4 (p & 1),
    // so two lane-dependent bases (even / odd p) plus the compile-time row offset p * 32 * 128 cover all eight
    uint32_t st_base[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) st_base[t] = (uint32_t)(ld_row * BK + ((ld_chunk ^ swz(ld_row) ^ (4 * t)) << 4));

    // fragment read offsets, same decomposition: rows r0 + 32 i; chunk (4 s + 2 half + q) ^ swz(r0 + 32 i)
    // = (4 (s ^ (i & 1)) + 2 half + q) ^ swz(r0)  ->  xa[s ^ (i & 1)][q] + i * 32 * 128
    uint32_t xa[2][2], xb[2][2];
    {
        const int ra0 = wm * WTM + l32, rb0 = wn * WTN + l32;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                xa[t][q] = (uint32_t)(ra0 * BK + (((4 * t + 2 * half + q) ^ swz(ra0)) << 4));
                xb[t][q] = (uint32_t)(BM * BK + rb0 * BK + (((4 * t + 2 * half + q) ^ swz(rb0)) << 4));
            }
    }

    auto read_frags = [&](Frags& f, int stage, int s) __attribute__((always_inline)) {
        const uint8_t* st = lds + stage * STAGE;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const v4i lo = *reinterpret_cast<const v4i*>(st + xa[s ^ (i & 1)][0] + i * 32 * BK);
            const v4i hi = *reinterpret_cast<const v4i*>(st + xa[s ^ (i & 1)][1] + i * 32 * BK);
            f.a[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const v4i lo = *reinterpret_cast<const v4i*>(st + xb[s ^ (j & 1)][0] + j * 32 * BK);
            const v4i hi = *reinterpret_cast<const v4i*>(st + xb[s ^ (j & 1)][1] + j * 32 * BK);
            f.b[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };

    const int total = g.tiles_m * g.tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int xcd = (int)blockIdx.x & 7;
    const int slot = (int)blockIdx.x >> 3;              // this workgroup's index among its XCD's workgroups
    const int slots = ((int)gridDim.x + 7 - xcd) >> 3;  // workgroups resident on this XCD
    const int nk = g.K / BK;
    const int64_t a_step = 32 * g.lda, b_step = 32 * g.ldb;  // uniform distance between a lane's chunks

    for (int local = slot; local < per_xcd; local += slots) {
        const int t = xcd * per_xcd + local;
        if (t >= total) break;
        int tm, tn;
        tile_coords(g, t, tm, tn);
        // the last tile row / column is shifted back so that every tile is full (M, N >= 256): the overlap is
        // recomputed with the same K order and rewritten with identical values
        const int m0 = (tm * BM + BM <= g.M) ? tm * BM : g.M - BM;
        const int n0 = (tn * BN + BN <= g.N) ? tn * BN : g.N - BN;

        const uint32_t a_off0 = (uint32_t)((int64_t)(m0 + ld_row) * g.lda + ld_chunk * 16);
        const uint32_t b_off0 = (uint32_t)((int64_t)(n0 + ld_row) * g.ldb + ld_chunk * 16);

        v4i ra[P], rb[P];  // plain vector registers (struct copies would be lowered to memcpy through scratch)
        auto load_tile = [&](int kt) __attribute__((always_inline)) {
            const uint8_t* ap = g.A + (int64_t)kt * BK;
            const uint8_t* bp = g.B + (int64_t)kt * BK;
#pragma unroll
            for (int p = 0; p < P; ++p) ra[p] = *reinterpret_cast<const v4i*>(ap + p * a_step + a_off0);
#pragma unroll
            for (int p = 0; p < P; ++p) rb[p] = *reinterpret_cast<const v4i*>(bp + p * b_step + b_off0);
        };
        auto store_tile = [&](int stage) __attribute__((always_inline)) {
            uint8_t* sa_ = lds + stage * STAGE;
            uint8_t* sb_ = sa_ + BM * BK;
#pragma unroll
            for (int p = 0; p < P; ++p) *reinterpret_cast<v4i*>(sa_ + st_base[p & 1] + p * 32 * BK) = ra[p];
#pragma unroll
            for (int p = 0; p < P; ++p) *reinterpret_cast<v4i*>(sb_ + st_base[p & 1] + p * 32 * BK) = rb[p];
        };

        v16f acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

        // D' = B . A^T : first MFMA operand is the B fragment (its type code goes to cbsz)
        auto mma_rows = [&](const Frags& f, int i_begin, int i_end) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                if (i < i_begin || i >= i_end) continue;
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.b[j], f.a[i], acc[i][j], BLGP_B,
                                                                                 CBSZ_A, 0, 0, 0, 0);
            }
        };

        Frags f0, f1;
        __syncthreads();  // the previous tile's epilogue is done with LDS
        load_tile(0);
        store_tile(0);
        if (nk > 1) load_tile(1);
        __syncthreads();
        read_frags(f0, 0, 0);

        for (int kt = 0; kt < nk; ++kt) {
            const int cur = kt & 1;
            mma_rows(f0, 0, 2);
            __builtin_amdgcn_sched_barrier(0);
            read_frags(f1, cur, 1);
            if (kt + 1 < nk) store_tile(cur ^ 1);
            if (kt + 2 < nk) load_tile(kt + 2);
            __builtin_amdgcn_sched_barrier(0);
            mma_rows(f0, 2, 4);
            __syncthreads();
            if (kt + 1 < nk) read_frags(f0, cur ^ 1, 0);
            __builtin_amdgcn_sched_barrier(0);
            mma_rows(f1, 0, 4);
            __builtin_amdgcn_sched_barrier(0);
        }

        // ---- epilogue ---------------------------------------------------------------------------------
        // acc[i][j][e] of lane l is C[row = m(i, l%32)][col = n(j) + 8*(e/4) + 4*(l/32) + e%4]
        __syncthreads();  // every wave is done reading the stages; LDS becomes the output staging area
        float isa[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) isa[i] = 1.0f / g.sa[g.sa_vec ? m0 + wm * WTM + i * 32 + l32 : 0];
        const float isb_scalar = g.sb_vec ? 0.0f : 1.0f / g.sb[0];

        if (g.c_f32) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int col = n0 + wn * WTN + j * 32 + 8 * q + 4 * half;
                    float isb[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) isb[e] = g.sb_vec ? 1.0f / g.sb[col + e] : isb_scalar;
#pragma unroll
                    for (int i = 0; i < TM; ++i) {
                        const int row = m0 + wm * WTM + i * 32 + l32;
                        float4 v;
                        v.x = acc[i][j][4 * q + 0] * isa[i] * isb[0];
                        v.y = acc[i][j][4 * q + 1] * isa[i] * isb[1];
                        v.z = acc[i][j][4 * q + 2] * isa[i] * isb[2];
                        v.w = acc[i][j][4 * q + 3] * isa[i] * isb[3];
                        *reinterpret_cast<float4*>(reinterpret_cast<float*>(g.C) + (int64_t)row * g.ldc + col) = v;
                    }
                }
        } else {
            // stage this wave's 128 x 128 bf16 tile in its private 32 KB of LDS: row pitch 256 bytes, the
            // 16-byte chunk index XORed with (row & 15) so that 16 rows hit 16 different bank groups
            uint8_t* stg = lds + wave * (WTM * WTN * 2);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int cw = j * 32 + 8 * q + 4 * half;  // column inside the wave tile (multiple of 4)
                    const int col = n0 + wn * WTN + cw;
                    float isb[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) isb[e] = g.sb_vec ? 1.0f / g.sb[col + e] : isb_scalar;
#pragma unroll
                    for (int i = 0; i < TM; ++i) {
                        const int rw = i * 32 + l32;
                        uint2 v;
                        v.x = (uint32_t)f32_to_bf16_bits(acc[i][j][4 * q + 0] * isa[i] * isb[0]) |
                              ((uint32_t)f32_to_bf16_bits(acc[i][j][4 * q + 1] * isa[i] * isb[1]) << 16);
                        v.y = (uint32_t)f32_to_bf16_bits(acc[i][j][4 * q + 2] * isa[i] * isb[2]) |
                              ((uint32_t)f32_to_bf16_bits(acc[i][j][4 * q + 3] * isa[i] * isb[3]) << 16);
                        const int chunk = (cw >> 3) ^ (rw & 15);
                        *reinterpret_cast<uint2*>(stg + rw * 256 + chunk * 16 + (cw & 4) * 2) = v;
                    }
                }
            // the staging region is private to the wave: the wave's own LDS ordering is enough
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
            __builtin_amdgcn_wave_barrier();
#pragma unroll 4
            for (int it = 0; it < 32; ++it) {
                const int rw = it * 4 + (lane >> 4);
                const int c16 = lane & 15;
                const uint4 v = *reinterpret_cast<const uint4*>(stg + rw * 256 + ((c16 ^ (rw & 15)) << 4));
                const int row = m0 + wm * WTM + rw;
                const int col = n0 + wn * WTN + c16 * 8;
                *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(g.C) + (int64_t)row * g.ldc + col) = v;
            }
        }
    }
}

int num_cus()
{
    static int cached = 0;
    if (cached == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cached = n;
    }
    return cached;
}

template <int CBSZ_A, int BLGP_B>
int launch(GemmArgs& g, hipStream_t st)
{
    auto kern = gemm_fp8_pipe_kernel<CBSZ_A, BLGP_B>;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        if (e != hipSuccess) {
            set_error("mi8_gemm_fp8: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(e));
            return MI8_ERR_LAUNCH;
        }
        configured = true;
    }
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const int total = g.tiles_m * g.tiles_n;
    int blocks = num_cus();
    if (blocks > total) blocks = total;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(NT), LDS_BYTES, st, g);
    return launch_status("mi8_gemm_fp8(pipelined)");
}

}  // namespace

int launch_pipelined(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st)
{
    if (a_dtype == MI8_E4M3) return b_dtype == MI8_E4M3 ? launch<0, 0>(g, st) : launch<0, 1>(g, st);
    return b_dtype == MI8_E4M3 ? launch<1, 0>(g, st) : launch<1, 1>(g, st);
}

}  // namespace gemm
}  // namespace mi8
