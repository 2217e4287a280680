// Persistent fp8 GEMM, 8 waves per workgroup, direct global->LDS loads of full 128-byte rows.
// For full 256 x 256 tiles, K % 128 == 0, bf16 output, and scales that are both single values or both vectors.
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
#include "mi8_gemm_tiles.h"

namespace mi8 {
namespace gemm {
namespace {

constexpr int WTM = 128, TM = 4;               // two waves along M, each 4 MFMA tiles of 32 rows
constexpr int STAGE = (BM + BN) * BK;          // 64 KB
constexpr int OUT_STAGING = 8 * 4096;           // 4 KB of output staging per wave
constexpr int LDS_BYTES = 2 * STAGE + OUT_STAGING;

// The wave layout is 2 x WN.  WN = 4: eight waves of 128 x 64 (two per SIMD, 256 registers each).  WN = 2: four
// waves of 128 x 128 (one per SIMD, 512 registers: twice the accumulators, a third less LDS read traffic, but no
// second wave to fill the matrix pipe while one waits).
template <int WN>
struct Layout {
    static constexpr int kWaves = 2 * WN;
    static constexpr int kThreads = kWaves * 64;
    static constexpr int WTN = BN / WN;            // wave tile columns: 64 or 128
    static constexpr int TN = WTN / 32;            // MFMA tiles along N per wave: 2 or 4
    static constexpr int NH = 2 * (TM + TN);       // 16-byte fragment halves per K sub-step: 12 or 16
    static constexpr int kMmas = TM * TN;          // MFMAs per K sub-step: 8 or 16
    static constexpr int kRowsPerWave = BM / kWaves;  // operand rows a wave fetches per step: 32 or 64
    static constexpr int kLoads = kRowsPerWave / 8;   // direct loads per operand, step and wave: 4 or 8
};

typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// fragment halves of one 64-byte K sub-step in consumption order: A0, B0 .. B(TN-1), A1, A2, A3 (two halves each)
template <int NH>
struct Frags {
    v4i h[NH];
};
template <int TN>
__device__ __forceinline__ constexpr int frag_a(int i) { return i == 0 ? 0 : 2 * TN + 2 * i; }
__device__ __forceinline__ constexpr int frag_b(int j) { return 2 + 2 * j; }


template <typename Problem, int WN, int CBSZ_A, int BLGP_B>
__global__ __launch_bounds__(Layout<WN>::kThreads, 1) void gemm_fp8_dma8_kernel(Problem pb)
{
    using L = Layout<WN>;
    constexpr int WTN = L::WTN, TN = L::TN, NH = L::NH;
    using Frags = mi8::gemm::Frags<NH>;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, half = lane >> 5;

    // ---- fragment read offsets.  MFMA tile `tile` of a wave reads rows r0 + 32 tile (r0 = wave origin + l32, the
    // wave origin a multiple of 64), 16-byte chunk (4 s + 2 half + q) ^ swz(row) of K sub-step s.  Adding 32 to
    // the row flips bit 2 of swz, and 4 s, 2 half, q occupy disjoint bits, so
    //     chunk = ((2 half) ^ swz(r0)) ^ (4 (s ^ (tile & 1)) | q).
    // One register per operand holds the lane's byte offset for (s, q, tile) = 0; the stage base is added once
    // per phase (no carries into the chunk bits) and every read XORs a literal into it.  Keeping only two
    // registers instead of eight precomputed addresses matters: the kernel runs at the 256-register limit.
    const uint32_t xa00 = (uint32_t)((wm * WTM + l32) * BK + (((2 * half) ^ swz(wm * WTM + l32)) << 4));
    const uint32_t xb00 = (uint32_t)(BM * BK + (wn * WTN + l32) * BK + (((2 * half) ^ swz(wn * WTN + l32)) << 4));
    // slot x of Frags: 0,1 = A0; then two per B tile; then A1..A3.  pa / pb: xa00 / xb00 plus the stage's byte offset.
    // The four-wave layout has registers to spare (its accumulators live in the other half of the register file)
    // and one wave per SIMD, so every address instruction between two MFMAs is exposed: it keeps the four XOR
    // variants per operand resident as LDS addresses of the stage being read (kResident) and moves them to the
    // other stage with one add each per K step.
    constexpr bool kResident = (WN == 2);
    uint32_t ra[4], rb[4];
    if constexpr (kResident) {
        const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)lds;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            ra[v] = lds0 + (xa00 ^ (uint32_t)(((4 * (v >> 1)) | (v & 1)) << 4));
            rb[v] = lds0 + (xb00 ^ (uint32_t)(((4 * (v >> 1)) | (v & 1)) << 4));
        }
    }
    auto flip_read_stage = [&](int to_stage) __attribute__((always_inline)) {
        const uint32_t delta = to_stage ? (uint32_t)STAGE : (uint32_t)(-STAGE);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            ra[v] += delta;
            rb[v] += delta;
        }
    };
    auto read_one = [&](Frags& f, uint32_t pa, uint32_t pb_, int s, int x) __attribute__((always_inline)) {
        const bool is_a = (x < 2) || (x >= 2 + 2 * TN);
        const int tile = x < 2 ? 0 : (x < 2 + 2 * TN ? (x - 2) >> 1 : (x - 2 * TN) >> 1);
        const int q = x & 1;
        if constexpr (kResident) {
            const int v = 2 * (s ^ (tile & 1)) + q;
            const uint32_t addr = (is_a ? ra[v] : rb[v]) + tile * 32 * BK;
            f.h[x] = *reinterpret_cast<const __attribute__((address_space(3))) v4i*>((uintptr_t)addr);
        } else {
            const uint32_t off = ((is_a ? pa : pb_) ^ (uint32_t)(((4 * (s ^ (tile & 1))) | q) << 4)) + tile * 32 * BK;
            f.h[x] = *reinterpret_cast<const v4i*>(lds + off);
        }
    };

    // ---- direct loads: wave w fills rows [R w + 8 p, +8) of each operand, R = kRowsPerWave, p = 0..kLoads-1;
    // lane -> row R w + 8 p + lr (lr = lane / 8), position lane % 8; swz(row) = (lr ^ (R/8 w + p)) & 7
    constexpr int RPW = L::kRowsPerWave, NLD = L::kLoads;
    const int lr = lane >> 3;
    const uint32_t c0 = (uint32_t)((lane & 7) ^ lr);
    const uint32_t rowoff_a = (uint32_t)((int64_t)(wave * RPW + lr) * pb.lda);
    const uint32_t rowoff_b = (uint32_t)((int64_t)(wave * RPW + lr) * pb.ldb);
    // x in 0..2 NLD-1: the first NLD -> A rows 8 x, the rest -> B rows 8 (x - NLD)
    // resident lane offsets of the 2 NLD loads (kResident): row offset and swizzled chunk in one register each, so a
    // load is one M0 update and the load itself
    uint32_t dvo[kResident ? 2 * NLD : 1];
    if constexpr (kResident) {
#pragma unroll
        for (int x = 0; x < 2 * NLD; ++x) {
            const int p = x % NLD;
            const int64_t ld = x < NLD ? pb.lda : pb.ldb;
            dvo[x] = (uint32_t)((int64_t)(wave * RPW + 8 * p + lr) * ld) + ((c0 ^ (uint32_t)((NLD * wave + p) & 7)) << 4);
        }
    }
    auto dma_one = [&](const uint8_t* a_origin, const uint8_t* b_origin, int stage, int x) __attribute__((always_inline)) {
        const int p = x % NLD;
        const bool is_a = x < NLD;
        if constexpr (kResident) {
            uint32_t o = dvo[x];
            asm volatile("" : "+v"(o));  // keeps the offset 32 bits wide up to the load (uniform base + lane offset form)
            const uint8_t* src = (is_a ? a_origin : b_origin) + o;
            uint8_t* dst = lds + stage * STAGE + (is_a ? 0 : BM * BK) + (wave * RPW + 8 * p) * BK;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)dst, 16, 0, 0);
            return;
        }
        // uniform 64-bit base + 32-bit lane offset.  The empty asm makes the lane's chunk index opaque at every
        // use: the offset is then rebuilt with two cheap vector instructions next to the load (and folded into
        // its scalar-base addressing) instead of living in eight hoisted 64-bit lane addresses.
        uint32_t c = c0;
        asm volatile("" : "+v"(c));
        const uint32_t voff = (is_a ? rowoff_a : rowoff_b) + ((c ^ (uint32_t)((NLD * wave + p) & 7)) << 4);
        const uint8_t* src = (is_a ? a_origin + (int64_t)(8 * p) * pb.lda : b_origin + (int64_t)(8 * p) * pb.ldb) + voff;
        uint8_t* dst = lds + stage * STAGE + (is_a ? 0 : BM * BK) + (wave * RPW + 8 * p) * BK;
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)dst, 16, 0, 0);
    };

    // ---- this workgroup's tiles: XCD-contiguous ranges, persistent over the `slots` workgroups of its XCD
    // Workgroups are dealt round-robin to the 8 XCDs (blockIdx % 8).  Tiles of equal cost: every XCD takes a
    // contiguous range of the tile order (its L2 then sees neighbouring tiles) and the `slots` workgroups of the
    // XCD stride through it.  Tiles of unequal cost: plain striding over all workgroups, so that the heavy
    // groups are spread over all XCDs.
    const typename Problem::Cache cache = pb.prepare();
    const int total = pb.total_tiles(cache);
    int first_tile, tile_stride, my_tiles;
    if constexpr (Problem::kXcdRanges) {
        const int per_xcd = (total + 7) / 8;
        const int xcd = (int)blockIdx.x & 7;
        const int slot = (int)blockIdx.x >> 3;
        const int slots = ((int)gridDim.x + 7 - xcd) >> 3;
        const int first = xcd * per_xcd;
        int last = first + per_xcd;
        last = last < total ? last : total;
        first_tile = first + slot;
        tile_stride = slots;
        my_tiles = (first_tile < last) ? (last - first_tile + slots - 1) / slots : 0;
    } else {
        first_tile = (int)blockIdx.x;
        tile_stride = (int)gridDim.x;
        my_tiles = (first_tile < total) ? (total - first_tile + tile_stride - 1) / tile_stride : 0;
    }
    if (my_tiles == 0) return;
    auto my_tile = [&](int idx) __attribute__((always_inline)) { return pb.tile(first_tile + idx * tile_stride, cache); };

    // load cursor: the K step whose stage is fetched next (two steps ahead of the compute cursor); it skips
    // tiles without K steps and, past the last tile, keeps fetching valid data nobody reads
    int ld_tile = -1, ld_kt = 0, ld_nk = 0;
    const uint8_t* ld_a = nullptr;
    const uint8_t* ld_b = nullptr;
    auto next_load_tile = [&]() __attribute__((always_inline)) {
        while (ld_tile + 1 < my_tiles) {
            ++ld_tile;
            const TileDesc d = my_tile(ld_tile);
            if (d.nk > 0) {
                ld_a = d.a;
                ld_b = d.b;
                ld_nk = d.nk;
                ld_kt = 0;
                return;
            }
        }
        // no further tile with work: rewind to the start of the current one (or stay null if there never was one)
        if (ld_a) {
            ld_a -= (int64_t)ld_kt * BK;
            ld_b -= (int64_t)ld_kt * BK;
            ld_kt = 0;
        }
    };
    auto advance_load_cursor = [&]() __attribute__((always_inline)) {
        ++ld_kt;
        ld_a += BK;
        ld_b += BK;
        if (ld_kt >= ld_nk) next_load_tile();
    };
    next_load_tile();

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
    // `fresh`: the tile's first touch of this accumulator; the MFMA then takes the constant 0 as its addend, so
    // the 128 accumulator registers never have to be cleared between tiles
    auto mma_one = [&](const Frags& f, int x, bool fresh) __attribute__((always_inline)) {
        const int i = x / TN, j = x % TN;
        const v8i fa = __builtin_shufflevector(f.h[frag_a<TN>(i)], f.h[frag_a<TN>(i) + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        const v8i fb = __builtin_shufflevector(f.h[frag_b(j)], f.h[frag_b(j) + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb, fa, fresh ? zero : acc[i][j], BLGP_B, CBSZ_A, 0, 0,
                                                                     0, 0);
    };

    // ---- prologue: stages of steps 0 and 1, fragments of step 0 ----------------------------------------
    const bool any_work = ld_a != nullptr;  // uniform
    if (any_work) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
#pragma unroll
            for (int x = 0; x < 2 * NLD; ++x) dma_one(ld_a, ld_b, s, x);
            advance_load_cursor();
        }
    }
    Frags f0, f1;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct loads have landed
    __syncthreads();
#pragma unroll
    for (int x = 0; x < NH; ++x) read_one(f0, xa00, xb00, 0, x);

    int step = 0;
    for (int cp_tile = 0; cp_tile < my_tiles; ++cp_tile) {
        const TileDesc td = my_tile(cp_tile);
        // One 128-byte K step.  `fresh`: the tile's first step, whose phase A starts the accumulators from 0.
        // The first step is written out separately from the loop (not as a branch inside it) so that the two
        // copies share no hoisted address registers.
        auto k_step = [&](bool fresh) __attribute__((always_inline)) {
            const int cur = step & 1;
            const uint32_t pa_cur = xa00 + cur * STAGE, pb_cur = xb00 + cur * STAGE;
            const uint32_t pa_nxt = xa00 + (cur ^ 1) * STAGE, pb_nxt = xb00 + (cur ^ 1) * STAGE;
            // Fragment reads trail the MFMAs: with 8 MFMAs per phase two reads follow MFMAs 1..6 (any earlier and
            // the 256-register budget overflows), with 16 MFMAs two reads follow each of the first eight.
            auto reads_after = [&](Frags& f, uint32_t pa, uint32_t pb_, int s, int x) __attribute__((always_inline)) {
                if constexpr (TN == 2) {
                    if (x >= 1 && x < 7) {
                        read_one(f, pa, pb_, s, 2 * x - 2);
                        read_one(f, pa, pb_, s, 2 * x - 1);
                    }
                } else {
                    if (x < 8) {
                        read_one(f, pa, pb_, s, 2 * x);
                        read_one(f, pa, pb_, s, 2 * x + 1);
                    }
                }
            };
            // phase A: its MFMAs touch each accumulator tile once
#pragma unroll
            for (int x = 0; x < L::kMmas; ++x) {
                mma_one(f0, x, fresh);
                reads_after(f1, pa_cur, pb_cur, 1, x);
                __builtin_amdgcn_sched_barrier(0);
            }
            // the compiler does not track direct-to-LDS loads across a barrier: wait for this wave's
            // outstanding ones (the next step's stage) before telling the others they have landed
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            __syncthreads();
            if constexpr (kResident) flip_read_stage(cur ^ 1);
            // phase B
#pragma unroll
            for (int x = 0; x < L::kMmas; ++x) {
                mma_one(f1, x, false);
                reads_after(f0, pa_nxt, pb_nxt, 0, x);
                dma_one(ld_a, ld_b, cur, x);  // kMmas == 2 * kLoads: one direct load per MFMA (bunching them up is slower)
                __builtin_amdgcn_sched_barrier(0);
            }
            advance_load_cursor();
            ++step;
        };
        // (with eight waves the ragged-M instantiation compiles to slower code when the first step is peeled)
        constexpr bool kPeel = Problem::kPeelFirstStep || WN == 2;
        if constexpr (kPeel) {
            if (td.nk > 0) {
                k_step(true);
                for (int kt = 1; kt < td.nk; ++kt) k_step(false);
            }
        } else {
            clear_acc();
            for (int kt = 0; kt < td.nk; ++kt) k_step(false);
        }

        // ---- tile finished: epilogue -------------------------------------------------------------------
        // acc[i][j][e] of lane l is C[row = 32 i + l%32][col = 32 j + 8*(e/4) + 4*(l/32) + e%4] of the wave tile.
        // A single scale is inverted with an IEEE division, scale vectors with v_rcp_f32 (exact for the
        // power-of-two scales of the axiswise recipes, within 1 ulp otherwise).
        if (kPeel && td.nk == 0) clear_acc();  // nothing was accumulated (empty group)
        // The wave's output goes through its private staging area 32 rows x 64 columns at a time (4 KB, pitch 128
        // bytes), i.e. one row group of MFMA tiles and two tile columns per pass.
        uint8_t* stg = lds + 2 * STAGE + wave * 4096;
        const bool zero_tile = td.nk == 0;  // nothing accumulated; the scales may be unset
        const float isb_scalar = Problem::kVecScales ? 1.0f : 1.0f / td.sb[0];
        const int ldc_bytes = (int)pb.ldc * 2;
        __amdgpu_buffer_rsrc_t c_rows;
        if constexpr (Problem::kMaskRows)
            c_rows = __builtin_amdgcn_make_buffer_rsrc(td.c + (int64_t)td.row_lo * pb.ldc, 0,
                                                       (td.row_hi - td.row_lo) * ldc_bytes, 0x00020000);
#pragma unroll
        for (int jh = 0; jh < TN / 2; ++jh) {
            float isb[2][4][4];
            if constexpr (Problem::kVecScales) {
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float4 s4 =
                            *reinterpret_cast<const float4*>(td.sb + wn * WTN + (2 * jh + j) * 32 + 8 * q + 4 * half);
                        isb[j][q][0] = zero_tile ? 0.0f : __builtin_amdgcn_rcpf(s4.x);
                        isb[j][q][1] = zero_tile ? 0.0f : __builtin_amdgcn_rcpf(s4.y);
                        isb[j][q][2] = zero_tile ? 0.0f : __builtin_amdgcn_rcpf(s4.z);
                        isb[j][q][3] = zero_tile ? 0.0f : __builtin_amdgcn_rcpf(s4.w);
                    }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int rt = wm * WTM + i * 32;  // first tile row of this pass
                // A single scale is re-read (volatile) in every pass: the pass then depends on a load, as it does
                // with scale vectors; with a loop-invariant multiplier the compiler forms the products of the
                // whole tile up front and spills accumulators.
                float mult = Problem::kVecScales ? __builtin_amdgcn_rcpf(td.sa[rt + l32])
                                                 : 1.0f / *reinterpret_cast<const volatile float*>(td.sa);
                mult = zero_tile ? 0.0f : mult * isb_scalar;
                // the 16-byte chunk index is XORed with (row >> 1) & 7 so that 16 consecutive rows cover all banks
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int cw = j * 32 + 8 * q + 4 * half;  // column inside the 64-column pass, multiple of 4
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            v[e] = acc[i][2 * jh + j][4 * q + e] * mult;
                            if constexpr (Problem::kVecScales) v[e] *= isb[j][q][e];
                        }
                        uint2 o;
                        o.x = pack_bf16x2(v[0], v[1]);
                        o.y = pack_bf16x2(v[2], v[3]);
                        const int chunk = (cw >> 3) ^ ((l32 >> 1) & 7);
                        *reinterpret_cast<uint2*>(stg + l32 * 128 + chunk * 16 + (cw & 4) * 2) = o;
                    }
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
                __builtin_amdgcn_wave_barrier();
                v4i staged[4];  // (an ext-vector type: arrays of HIP's uint4 struct end up in scratch)
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int rw = it * 8 + (lane >> 3);
                    staged[it] = *reinterpret_cast<const v4i*>(stg + rw * 128 + (((lane & 7) ^ ((rw >> 1) & 7)) << 4));
                }
                if constexpr (Problem::kMaskRows) {
                    // Only rows [row_lo, row_hi) of the tile belong to this tile's group.  The stores go through a
                    // buffer descriptor that spans exactly those rows: a lane whose row lies outside gets an
                    // offset below zero (huge when read as unsigned) or past the end, and the hardware drops its
                    // store - no divergent branches around the stores.
                    const int voff = (rt + (lane >> 3) - td.row_lo) * ldc_bytes + (wn * WTN + jh * 64 + (lane & 7) * 8) * 2;
#pragma unroll
                    for (int it = 0; it < 4; ++it)
                        __builtin_amdgcn_raw_buffer_store_b128(staged[it], c_rows, voff + it * 8 * ldc_bytes, 0, 0);
                } else {
                    uint16_t* crow = td.c + (int64_t)(rt + (lane >> 3)) * pb.ldc + wn * WTN + jh * 64 + (lane & 7) * 8;
#pragma unroll
                    for (int it = 0; it < 4; ++it) *reinterpret_cast<v4i*>(crow + (int64_t)(it * 8) * pb.ldc) = staged[it];
                }
                __builtin_amdgcn_s_waitcnt(0xc07f);  // the reads are done before the next pass overwrites
                __builtin_amdgcn_wave_barrier();
            }
        }
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

// persistent: one workgroup per CU walks a static share of the tiles (right when all tiles cost the same);
// otherwise one workgroup per tile, handed to free CUs by the hardware dispatcher (tiles of unequal cost).
template <typename Problem, int WN, int CBSZ_A, int BLGP_B>
int launch(const Problem& pb, int max_tiles, bool persistent, hipStream_t st)
{
    auto kern = gemm_fp8_dma8_kernel<Problem, WN, CBSZ_A, BLGP_B>;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        if (e != hipSuccess) {
            set_error("mi8 direct-to-LDS GEMM: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(e));
            return MI8_ERR_LAUNCH;
        }
        configured = true;
    }
    // Persistent: one workgroup per compute unit, or, for fewer tiles, as many as the tiles need - rounded up to
    // a multiple of 8, because every XCD takes an eighth of the tiles (rounded up) and needs that many
    // workgroups to finish in one round (43 tiles on 43 workgroups: XCDs with 5 workgroups for 6 tiles).
    int blocks = persistent ? num_cus() : max_tiles;
    const int wanted = persistent ? (max_tiles + 7) / 8 * 8 : max_tiles;
    if (blocks > wanted) blocks = wanted;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(Layout<WN>::kThreads), LDS_BYTES, st, pb);
    return launch_status("mi8 direct-to-LDS GEMM (8 waves)");
}

template <typename Problem, int WN = 4>
int launch_typed(const Problem& pb, int max_tiles, bool persistent, int a_dtype, int b_dtype, hipStream_t st)
{
    if (a_dtype == MI8_E4M3)
        return b_dtype == MI8_E4M3 ? launch<Problem, WN, 0, 0>(pb, max_tiles, persistent, st)
                                   : launch<Problem, WN, 0, 1>(pb, max_tiles, persistent, st);
    return b_dtype == MI8_E4M3 ? launch<Problem, WN, 1, 0>(pb, max_tiles, persistent, st)
                               : launch<Problem, WN, 1, 1>(pb, max_tiles, persistent, st);
}

}  // namespace

int launch_dma8(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st)
{
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    if (g.sa_vec) {
        DenseProblem<true> pb{g, g.lda, g.ldb, g.ldc};
        return launch_typed(pb, g.tiles_m * g.tiles_n, true, a_dtype, b_dtype, st);
    }
    DenseProblem<false> pb{g, g.lda, g.ldb, g.ldc};
    return launch_typed(pb, g.tiles_m * g.tiles_n, true, a_dtype, b_dtype, st);
}

int launch_dma4(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st)
{
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    if (g.sa_vec) {
        DenseProblem<true> pb{g, g.lda, g.ldb, g.ldc};
        return launch_typed<DenseProblem<true>, 2>(pb, g.tiles_m * g.tiles_n, true, a_dtype, b_dtype, st);
    }
    DenseProblem<false> pb{g, g.lda, g.ldb, g.ldc};
    return launch_typed<DenseProblem<false>, 2>(pb, g.tiles_m * g.tiles_n, true, a_dtype, b_dtype, st);
}

}  // namespace gemm
}  // namespace mi8
