// Persistent fp8 GEMM with direct global->LDS loads (global_load_lds_dwordx4), for full 256 x 256 tiles,
// K % 64 == 0 and bf16 output.
//
// One workgroup of 4 waves per CU (one wave per SIMD, 512 registers each); a wave owns a 128 x 128 sub-tile =
// 4 x 4 MFMA tiles of 32x32x64 (fp32 accumulators in AGPRs).  LDS = the full 160 KB of a CU: a ring of four
// 32 KB operand stages (256 A rows + 256 B rows of 64 K-bytes each, XOR swizzled) plus 32 KB of output staging.
//
// The workgroup walks its tiles as ONE flat sequence of 64-byte K steps (tile after tile).  Step s:
//
//     wait until this wave's loads of step s+1 have landed; barrier
//     16 x { MFMA on the fragments of step s (already in registers) ;
//            first half : 2 LDS reads of the fragments of step s+1 ;
//            second half: 1 direct global->LDS load of step s+4 into the stage step s just vacated }
//     if step s ends a tile: scale, round, stage through LDS, 16-byte stores; clear the accumulators
//
// so a load has about 2.5 steps (40 matrix instructions) to land, and the loads of the next tile's first steps
// are in flight while the current tile is finished and stored.  A matrix instruction occupies the matrix pipe
// for 64 cycles and nothing queues behind it, so the memory instructions are dealt out between the MFMAs in
// source order and pinned there with scheduling barriers.  Data never passes through VGPRs on its way to LDS
// (a register-staged 16-byte LDS write costs about 40 matrix-pipe cycles).
//
// Swizzle: LDS chunk position q (16 bytes) of row r holds global chunk q ^ sw(r), sw(r) = (r ^ r>>1 ^ r>>3) & 3:
// the fragment reads of 8 or 16 consecutive rows then cover all banks.  A load instruction fills 16 consecutive
// rows (64 lanes x 16 B; lane l -> row l/4, position l%4), so lane l fetches global chunk (l%4) ^ sw(row).
#include "mi8_gemm.h"

namespace mi8 {
namespace gemm {
namespace {

constexpr int BM = 256, BN = 256;
constexpr int WTM = 128, WTN = 128;
constexpr int TM = 4, TN = 4;
constexpr int NT = 256;
constexpr int KS = 64;                         // K bytes per step = one MFMA K
constexpr int NSTAGE = 4;
constexpr int STAGE = (BM + BN) * KS;          // 32 KB
constexpr int OUT_STAGING = 4 * 32 * WTN * 2;  // 4 waves x (32 rows x 128 bf16) = 32 KB
constexpr int LDS_BYTES = NSTAGE * STAGE + OUT_STAGING;

typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

__device__ __forceinline__ int sw4(int r) { return (r ^ (r >> 1) ^ (r >> 3)) & 3; }

// sixteen 16-byte fragment halves of one K step, in the order the MFMAs consume them:
// h[0..1] = A tile 0, h[2..9] = B tiles 0..3, h[10..15] = A tiles 1..3
struct Frags {
    v4i h[16];
};
__device__ __forceinline__ constexpr int frag_a(int i) { return i == 0 ? 0 : 8 + 2 * i; }
__device__ __forceinline__ constexpr int frag_b(int j) { return 2 + 2 * j; }

template <int CBSZ_A, int BLGP_B>
__global__ __launch_bounds__(NT, 1) void gemm_fp8_dma_kernel(GemmArgs g)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;

    // ---- fragment read offsets: row r0 + 32 i, chunks 2 half + q; sw4 only looks at the low five row bits, so
    //      it is the same for every i
    uint32_t xa[2], xb[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        xa[q] = (uint32_t)((wm * WTM + l32) * KS + (((2 * half + q) ^ sw4(l32)) << 4));
        xb[q] = (uint32_t)(BM * KS + (wn * WTN + l32) * KS + (((2 * half + q) ^ sw4(l32)) << 4));
    }
    auto read_one = [&](Frags& f, const uint8_t* st, int x) __attribute__((always_inline)) {
        const bool is_a = (x < 2) || (x >= 10);
        const int tile = x < 2 ? 0 : (x < 10 ? (x - 2) >> 1 : (x - 8) >> 1);
        const uint32_t off = (is_a ? xa[x & 1] : xb[x & 1]) + tile * 32 * KS;
        f.h[x] = *reinterpret_cast<const v4i*>(st + off);
    };

    // ---- direct loads: wave w fills rows [64 w + 16 p, +16) of each operand, p = 0..3
    // lane -> row 64 w + 16 p + lq (lq = lane / 4), position lane % 4; sw4(row) depends on lq and on p & 1
    const int lq = lane >> 2;
    uint32_t voff_a[2], voff_b[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint32_t chunk = (uint32_t)(((lane & 3) ^ sw4(16 * t + lq)) << 4);
        voff_a[t] = (uint32_t)((int64_t)(wave * 64 + lq) * g.lda) + chunk;
        voff_b[t] = (uint32_t)((int64_t)(wave * 64 + lq) * g.ldb) + chunk;
    }
    // x in 0..7: 0..3 -> A rows 16 x, 4..7 -> B rows 16 (x - 4); origins point at the tile's first row, K offset included
    auto dma_one = [&](const uint8_t* a_origin, const uint8_t* b_origin, int stage, int x) __attribute__((always_inline)) {
        const int p = x & 3;
        const uint8_t* src = x < 4 ? a_origin + (int64_t)(16 * p) * g.lda + voff_a[p & 1]
                                   : b_origin + (int64_t)(16 * p) * g.ldb + voff_b[p & 1];
        uint8_t* dst = lds + stage * STAGE + (x < 4 ? 0 : BM * KS) + (wave * 64 + 16 * p) * KS;
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
    const int nk = g.K / KS;

    auto tile_origin = [&](int idx, int& m0, int& n0) __attribute__((always_inline)) {
        int tm, tn;
        tile_coords(g, first + slot + idx * slots, tm, tn);
        // the last tile row / column is shifted back so that every tile is full (M, N >= 256): the overlap is
        // recomputed with the same K order and rewritten with identical values
        m0 = (tm * BM + BM <= g.M) ? tm * BM : g.M - BM;
        n0 = (tn * BN + BN <= g.N) ? tn * BN : g.N - BN;
    };

    // load cursor: the K step whose stage is fetched next (runs NSTAGE steps ahead of the compute cursor)
    int ld_tile = 0, ld_kt = 0, ld_m0, ld_n0;
    tile_origin(0, ld_m0, ld_n0);
    const uint8_t* ld_a = g.A + (int64_t)ld_m0 * g.lda;
    const uint8_t* ld_b = g.B + (int64_t)ld_n0 * g.ldb;
    auto advance_load_cursor = [&]() __attribute__((always_inline)) {
        ++ld_kt;
        ld_a += KS;
        ld_b += KS;
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
        const int i = x >> 2, j = x & 3;
        const v8i fa = __builtin_shufflevector(f.h[frag_a(i)], f.h[frag_a(i) + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        const v8i fb = __builtin_shufflevector(f.h[frag_b(j)], f.h[frag_b(j) + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb, fa, acc[i][j], BLGP_B, CBSZ_A, 0, 0, 0, 0);
    };
    // one K step: consume `cur`, prefetch `nxt` from the stage of step s + 1, refill the stage of step s
    auto k_step = [&](const Frags& cur, Frags& nxt, int s) __attribute__((always_inline)) {
        // vmcnt counts the direct loads in issue order: all but the 16 youngest (steps s+2, s+3) have landed,
        // i.e. the stage of step s+1; the compiler does not track these loads across a barrier
        __builtin_amdgcn_s_waitcnt(0x4F70);  // vmcnt(16)
        __syncthreads();
        const uint8_t* st_next = lds + ((s + 1) & (NSTAGE - 1)) * STAGE;
        const int st_free = s & (NSTAGE - 1);
#pragma unroll
        for (int x = 0; x < 16; ++x) {
            mma_one(cur, x);
            if (x < 8) {
                read_one(nxt, st_next, 2 * x);
                read_one(nxt, st_next, 2 * x + 1);
            } else {
                dma_one(ld_a, ld_b, st_free, x - 8);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        advance_load_cursor();
    };

    // ---- prologue: stages of steps 0..3, fragments of step 0 ------------------------------------------
#pragma unroll
    for (int s = 0; s < NSTAGE; ++s) {
#pragma unroll
        for (int x = 0; x < 8; ++x) dma_one(ld_a, ld_b, s, x);
        advance_load_cursor();
    }
    clear_acc();
    Frags f0, f1;
    __builtin_amdgcn_s_waitcnt(0x4F78);  // vmcnt(24): the stage of step 0 has landed for this wave
    __syncthreads();
#pragma unroll
    for (int x = 0; x < 16; ++x) read_one(f0, lds, x);

    const float isb_scalar = 1.0f / g.sb[0];
    int step = 0;
    for (int cp_tile = 0; cp_tile < my_tiles; ++cp_tile) {
        int m0, n0;
        tile_origin(cp_tile, m0, n0);
        // two steps per iteration so that the fragment buffers alternate without copies
        int kt = 0;
        for (; kt + 1 < nk; kt += 2, step += 2) {
            k_step(f0, f1, step);
            k_step(f1, f0, step + 1);
        }
        if (kt < nk) {
            // odd number of steps: one more, then rename the buffers (a register copy once per tile)
            k_step(f0, f1, step);
            ++step;
#pragma unroll
            for (int x = 0; x < 16; ++x) f0.h[x] = f1.h[x];
        }

        // ---- tile finished: epilogue -------------------------------------------------------------------
        // acc[i][j][e] of lane l is C[row = m(i, l%32)][col = n(j) + 8*(e/4) + 4*(l/32) + e%4]
        uint8_t* stg = lds + NSTAGE * STAGE + wave * (32 * WTN * 2);  // wave-private 8 KB: 32 rows x 256 bytes
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
            // 32 rows x 128 bf16 through the wave's staging area: pitch 256 bytes, 16-byte chunk index XORed
            // with (row & 15) so that 16 rows hit 16 different bank groups
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int cw = j * 32 + 8 * q + 4 * half;
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = acc[i][j][4 * q + e] * mult;
                        if (g.sb_vec) v[e] *= isb[j][q][e];
                    }
                    uint2 o;
                    o.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
                    o.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
                    const int chunk = (cw >> 3) ^ (l32 & 15);
                    *reinterpret_cast<uint2*>(stg + l32 * 256 + chunk * 16 + (cw & 4) * 2) = o;
                }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int it = 0; it < 8; ++it) {
                const int rw = it * 4 + (lane >> 4);
                const int c16 = lane & 15;
                const uint4 v = *reinterpret_cast<const uint4*>(stg + rw * 256 + ((c16 ^ (rw & 15)) << 4));
                const int orow = m0 + wm * WTM + i * 32 + rw;
                const int ocol = n0 + wn * WTN + c16 * 8;
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
    auto kern = gemm_fp8_dma_kernel<CBSZ_A, BLGP_B>;
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
    const int wanted = (total + 7) / 8 * 8;  // every XCD gets as many workgroups as it has tiles
    if (blocks > wanted) blocks = wanted;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(NT), LDS_BYTES, st, g);
    return launch_status("mi8_gemm_fp8(direct-to-LDS)");
}

}  // namespace

int launch_dma(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st)
{
    if (a_dtype == MI8_E4M3) return b_dtype == MI8_E4M3 ? launch<0, 0>(g, st) : launch<0, 1>(g, st);
    return b_dtype == MI8_E4M3 ? launch<1, 0>(g, st) : launch<1, 1>(g, st);
}

}  // namespace gemm
}  // namespace mi8
