// Persistent fp8 GEMM, 8 waves per workgroup, direct global->LDS loads of full 128-byte rows.
// For full 256 x 256 tiles, K % 128 == 0 and bf16 output.
//
// Why 8 waves: the load bandwidth one CU can pull out of L2 grows with the number of waves that issue loads
// (measured on MI355X with 1 KB global_load_lds_dwordx4 instructions: 4 waves ~54 GB/s, 8 waves ~81 GB/s per
// CU), and a 256 x 256 tile needs 64 KB per 128-byte K step.  Two waves per SIMD also fill each other's
// matrix-pipe gaps.
//
// Workgroup: 2 x 4 waves, each wave a 128 x 64 sub-tile = 4 x 2 MFMA tiles of 32x32x64 (128 accumulator
// registers).  LDS: two 64 KB operand stages ([row][128 B], XOR swizzled) + 32 KB output staging = 160 KB.
// The workgroup walks its tiles as one flat sequence of 128-byte K steps; per step and wave:
//
//     phase A   8 x { MFMA on sub-step 0 ; LDS reads of the sub-step 1 fragments }
//     wait for this wave's loads of step s+1, barrier
//     phase B   8 x { MFMA on sub-step 1 ; LDS reads of step s+1's sub-step 0 fragments ;
//                     one direct load of step s+2 into the stage step s just vacated }
//
// Swizzle: chunk position q (16 bytes) of row r holds global chunk q ^ ((r ^ r>>3) & 7).  A load instruction
// fills 8 consecutive rows (lane l -> row l/8, position l%8), so lane l fetches chunk (l%8) ^ swz(row).
#include "mi8_gemm.h"

namespace mi8 {
namespace gemm {
namespace {

constexpr int BM = 256, BN = 256;
constexpr int WTM = 128, WTN = 64;
constexpr int TM = 4, TN = 2;
constexpr int NT = 512;
constexpr int STAGE = (BM + BN) * BK;          // 64 KB
constexpr int OUT_STAGING = 8 * 32 * WTN * 2;  // 8 waves x (32 rows x 64 bf16) = 32 KB
constexpr int LDS_BYTES = 2 * STAGE + OUT_STAGING;
constexpr int NH = 2 * (TM + TN);              // 16-byte fragment halves per K sub-step: 12

typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// fragment halves of one 64-byte K sub-step in consumption order: A0, B0, B1, A1, A2, A3 (two halves each)
struct Frags {
    v4i h[NH];
};
__device__ __forceinline__ constexpr int frag_a(int i) { return i == 0 ? 0 : 4 + 2 * i; }
__device__ __forceinline__ constexpr int frag_b(int j) { return 2 + 2 * j; }

template <int CBSZ_A, int BLGP_B>
__global__ __launch_bounds__(NT, 1) void gemm_fp8_dma8_kernel(GemmArgs g)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int l32 = lane & 31, half = lane >> 5;

    // ---- fragment read offsets: rows r0 + 32 i; chunk (4 s + 2 half + q) ^ swz(r0 + 32 i)
    //      = (4 (s ^ (i & 1)) + 2 half + q) ^ swz(r0)   [r0 a multiple of 64 plus l32]
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
    // slot x of Frags: 0,1 = A0; 2..5 = B0,B1; 6..11 = A1..A3
    auto read_one = [&](Frags& f, const uint8_t* st, int s, int x) __attribute__((always_inline)) {
        const bool is_a = (x < 2) || (x >= 6);
        const int tile = x < 2 ? 0 : (x < 6 ? (x - 2) >> 1 : (x - 4) >> 1);
        const int q = x & 1;
        const uint32_t off = (is_a ? xa[s ^ (tile & 1)][q] : xb[s ^ (tile & 1)][q]) + tile * 32 * BK;
        f.h[x] = *reinterpret_cast<const v4i*>(st + off);
    };

    // ---- direct loads: wave w fills rows [32 w + 8 p, +8) of each operand, p = 0..3;
    // lane -> row 32 w + 8 p + lr (lr = lane / 8), position lane % 8; swz(row) = (lr ^ (4 w + p)) & 7
    const int lr = lane >> 3;
    const uint32_t c0 = (uint32_t)((lane & 7) ^ lr);
    const uint32_t rowoff_a = (uint32_t)((int64_t)(wave * 32 + lr) * g.lda);
    const uint32_t rowoff_b = (uint32_t)((int64_t)(wave * 32 + lr) * g.ldb);
    // x in 0..7: 0..3 -> A rows 8 x, 4..7 -> B rows 8 (x - 4)
    auto dma_one = [&](const uint8_t* a_origin, const uint8_t* b_origin, int stage, int x) __attribute__((always_inline)) {
        const int p = x & 3;
        const uint32_t chunk = (c0 ^ (uint32_t)((4 * wave + p) & 7)) << 4;
        const uint8_t* src = x < 4 ? a_origin + (int64_t)(8 * p) * g.lda + (rowoff_a + chunk)
                                   : b_origin + (int64_t)(8 * p) * g.ldb + (rowoff_b + chunk);
        uint8_t* dst = lds + stage * STAGE + (x < 4 ? 0 : BM * BK) + (wave * 32 + 8 * p) * BK;
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)dst, 16, 0, 0);
    };

    // ---- this workgroup's tiles: XCD-contiguous ranges, persistent over the `slots` workgroups of its XCD
    const int total = g.tiles_m * g.tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int xcd = (int)blockIdx.x & 7;
    const int slot = (int)blockIdx.x >> 3;
    const int slots = ((int)gridDim.x + 7 - xcd) >> 3;
    const int first = xcd * per_xcd;
    int last = first + per_xcd;
    last = last < total ? last : total;
    const int my_tiles = (first + slot < last) ? (last - first - slot + slots - 1) / slots : 0;
    if (my_tiles == 0) return;
    const int nk = g.K / BK;

    auto tile_origin = [&](int idx, int& m0, int& n0) __attribute__((always_inline)) {
        int tm, tn;
        tile_coords(g, first + slot + idx * slots, tm, tn);
        // the last tile row / column is shifted back so that every tile is full (M, N >= 256): the overlap is
        // recomputed with the same K order and rewritten with identical values
        m0 = (tm * BM + BM <= g.M) ? tm * BM : g.M - BM;
        n0 = (tn * BN + BN <= g.N) ? tn * BN : g.N - BN;
    };

    // load cursor: the K step whose stage is fetched next (two steps ahead of the compute cursor)
    int ld_tile = 0, ld_kt = 0, ld_m0, ld_n0;
    tile_origin(0, ld_m0, ld_n0);
    const uint8_t* ld_a = g.A + (int64_t)ld_m0 * g.lda;
    const uint8_t* ld_b = g.B + (int64_t)ld_n0 * g.ldb;
    auto advance_load_cursor = [&]() __attribute__((always_inline)) {
        ++ld_kt;
        ld_a += BK;
        ld_b += BK;
        if (ld_kt == nk) {
            ld_kt = 0;
            // past the last tile the cursor stays on it: the extra loads fetch valid data nobody reads
            if (ld_tile + 1 < my_tiles) ++ld_tile;
            tile_origin(ld_tile, ld_m0, ld_n0);
            ld_a = g.A + (int64_t)ld_m0 * g.lda;
            ld_b = g.B + (int64_t)ld_n0 * g.ldb;
        }
    };

    v16f acc[TM][TN];
    auto clear_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    };
    // D' = B . A^T : first MFMA operand is the B fragment (its type code goes to cbsz)
    auto mma_one = [&](const Frags& f, int x) __attribute__((always_inline)) {
        const int i = x >> 1, j = x & 1;
        const v8i fa = __builtin_shufflevector(f.h[frag_a(i)], f.h[frag_a(i) + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        const v8i fb = __builtin_shufflevector(f.h[frag_b(j)], f.h[frag_b(j) + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb, fa, acc[i][j], BLGP_B, CBSZ_A, 0, 0, 0, 0);
    };

    // ---- prologue: stages of steps 0 and 1, fragments of step 0 ----------------------------------------
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int x = 0; x < 8; ++x) dma_one(ld_a, ld_b, s, x);
        advance_load_cursor();
    }
    clear_acc();
    Frags f0, f1;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct loads have landed
    __syncthreads();
#pragma unroll
    for (int x = 0; x < NH; ++x) read_one(f0, lds, 0, x);

    const float isb_scalar = 1.0f / g.sb[0];
    int step = 0;
    for (int cp_tile = 0; cp_tile < my_tiles; ++cp_tile) {
        int m0, n0;
        tile_origin(cp_tile, m0, n0);
        for (int kt = 0; kt < nk; ++kt, ++step) {
            const int cur = step & 1;
            const uint8_t* st_cur = lds + cur * STAGE;
            const uint8_t* st_nxt = lds + (cur ^ 1) * STAGE;
            // phase A
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                mma_one(f0, x);
                if (x < 6) {
                    read_one(f1, st_cur, 1, 2 * x);
                    read_one(f1, st_cur, 1, 2 * x + 1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            // the compiler does not track direct-to-LDS loads across a barrier: wait for this wave's
            // outstanding ones (the next step's stage) before telling the others they have landed
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            __syncthreads();
            // phase B
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                mma_one(f1, x);
                if (x < 6) {
                    read_one(f0, st_nxt, 0, 2 * x);
                    read_one(f0, st_nxt, 0, 2 * x + 1);
                }
                dma_one(ld_a, ld_b, cur, x);
                __builtin_amdgcn_sched_barrier(0);
            }
            advance_load_cursor();
        }

        // ---- tile finished: epilogue -------------------------------------------------------------------
        // acc[i][j][e] of lane l is C[row = m(i, l%32)][col = n(j) + 8*(e/4) + 4*(l/32) + e%4]
        uint8_t* stg = lds + 2 * STAGE + wave * (32 * WTN * 2);  // wave-private 4 KB: 32 rows x 128 bytes
        float isb[TN][4][4];
        if (g.sb_vec) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 s4 = *reinterpret_cast<const float4*>(g.sb + n0 + wn * WTN + j * 32 + 8 * q + 4 * half);
                    isb[j][q][0] = __builtin_amdgcn_rcpf(s4.x);
                    isb[j][q][1] = __builtin_amdgcn_rcpf(s4.y);
                    isb[j][q][2] = __builtin_amdgcn_rcpf(s4.z);
                    isb[j][q][3] = __builtin_amdgcn_rcpf(s4.w);
                }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int row = m0 + wm * WTM + i * 32 + l32;
            float mult = 1.0f / g.sa[g.sa_vec ? row : 0];
            if (!g.sb_vec) mult *= isb_scalar;
            // 32 rows x 64 bf16 through the wave's staging area: pitch 128 bytes, the 16-byte chunk index XORed
            // with (row >> 1) & 7 so that 16 consecutive rows cover all banks
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int cw = j * 32 + 8 * q + 4 * half;  // column inside the wave tile, multiple of 4
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = acc[i][j][4 * q + e] * mult;
                        if (g.sb_vec) v[e] *= isb[j][q][e];
                    }
                    uint2 o;
                    o.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
                    o.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
                    const int chunk = (cw >> 3) ^ ((l32 >> 1) & 7);
                    *reinterpret_cast<uint2*>(stg + l32 * 128 + chunk * 16 + (cw & 4) * 2) = o;
                }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int rw = it * 8 + (lane >> 3);
                const int c8 = lane & 7;
                const uint4 v = *reinterpret_cast<const uint4*>(stg + rw * 128 + ((c8 ^ ((rw >> 1) & 7)) << 4));
                const int orow = m0 + wm * WTM + i * 32 + rw;
                const int ocol = n0 + wn * WTN + c8 * 8;
                *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(g.C) + (int64_t)orow * g.ldc + ocol) = v;
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // the reads are done before the next pass overwrites
            __builtin_amdgcn_wave_barrier();
        }
        clear_acc();
    }
    // direct loads issued for steps past the end must have landed before the LDS allocation is released
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    __syncthreads();
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
    auto kern = gemm_fp8_dma8_kernel<CBSZ_A, BLGP_B>;
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
    return launch_status("mi8_gemm_fp8(direct-to-LDS, 8 waves)");
}

}  // namespace

int launch_dma8(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st)
{
    if (a_dtype == MI8_E4M3) return b_dtype == MI8_E4M3 ? launch<0, 0>(g, st) : launch<0, 1>(g, st);
    return b_dtype == MI8_E4M3 ? launch<1, 0>(g, st) : launch<1, 1>(g, st);
}

}  // namespace gemm
}  // namespace mi8
