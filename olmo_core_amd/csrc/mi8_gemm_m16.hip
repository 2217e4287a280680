// Persistent fp8 GEMM on 16x16x128 MFMAs: four waves of 128 x 128 per 256 x 256 workgroup tile, direct
// global->LDS loads of full 128-byte rows; for full 256 x 256 tiles, K % 128 == 0, bf16 output.
//
// Why this MFMA shape: an MI355X running fp8 MFMAs on random operands is power limited (it clocks down to
// 1.7-1.9 GHz), so throughput follows energy per flop, and v_mfma_f32_16x16x128_f8f6f4 needs less of it than
// v_mfma_f32_32x32x64_f8f6f4: back-to-back MFMAs on random bytes, nothing else running, measured 4.35 PFLOP/s
// against 4.0 PFLOP/s (both 4.97 PFLOP/s on all-zero operands, where the clock stays up).
//
// A 128-byte K step of a wave is 8 x 8 MFMAs (A tile i: 16 rows, B tile j: 16 columns, 4 accumulator registers
// each: 256 in all).  The step is split along M so that only half of the A fragments are double buffered:
//
//     barrier (every wave has issued its LDS reads of the previous phase B)
//     phase A   32 x { MFMA (A tiles 0-3) x (B tiles 0-7) }; LDS reads of A tiles 4-7 of this step; 8 direct loads:
//               the B rows of step s+2 into the stage of step s, whose B rows are no longer needed
//     wait for this wave's loads of step s+1 (all but the eight just issued), barrier
//     phase B   32 x { MFMA (A tiles 4-7) x (B tiles 0-7), B tile by B tile }; LDS reads of step s+1: A tiles 0-3
//               and each B tile as soon as its four MFMAs are issued; 8 direct loads: the A rows of step s+2
//
// Fragment registers: 32 (A 0-3) + 32 (A 4-7) + 64 (B) = 128.
//
// LDS: two 64 KB operand stages [row][128 B]; 16-byte chunk position c of row r holds global chunk c ^ swz16(r)
// (bank-conflict free for the fragment reads, see swz16).  The swizzle of a fragment row does not depend on the
// tile it belongs to, so two address registers per operand serve all eight tiles through the instruction's
// offset field.
#include <type_traits>

#include "mi8_gemm_tiles.h"
#include "mi8_swiglu.h"

namespace mi8 {
namespace gemm {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
typedef const __attribute__((address_space(3))) v4i* lfrag_t;

constexpr int STAGE = (BM + BN) * BK;        // 64 KB
constexpr int OUT_STAGING = 4 * 4096;        // 4 KB of output staging per wave
constexpr int SCALE_SLOT = 2 * 256 * 4;      // one tile's 256 row scales and 256 column scales
constexpr int SCALE_SLOTS = 4;
// Tile timeline (only in the diagnostics library, which compiles this file with -DMI8_TILE_TIMELINE): wave 0 of every
// workgroup records the shader clock at fixed points of each of its tiles - K loop start, after three K steps, epilogue
// start, every epilogue pass, last store issued, tile end - in 1 KB of LDS of its own and copies them out when the
// kernel ends.  A stamp costs one s_memtime and its wait (placed where nothing else the wave waits for is in flight).
#ifdef MI8_TILE_TIMELINE
constexpr int TIMELINE_BYTES = 1024;
constexpr int TIMELINE_STAMPS = 13;          // per tile
constexpr int TIMELINE_TILES = 16;           // tiles recorded per workgroup (later tiles overwrite the last record)
__device__ uint32_t* g_timeline = nullptr;   // [workgroups][256]: TIMELINE_TILES x TIMELINE_STAMPS, [254], [255]: 100 MHz clock at start / end
#define MI8_TL(k) tl_stamp(k)
#define MI8_TL_NEXT_TILE() (tl_ev += tl_ev < TIMELINE_STAMPS * (TIMELINE_TILES - 1) ? TIMELINE_STAMPS : 0)
#else
constexpr int TIMELINE_BYTES = 0;
#define MI8_TL(k) ((void)0)
#define MI8_TL_NEXT_TILE() ((void)0)
#endif
constexpr int LDS_BYTES = 2 * STAGE + OUT_STAGING + SCALE_SLOTS * SCALE_SLOT + TIMELINE_BYTES;
constexpr int kThreads = 256;
constexpr int WT = 128;                      // wave tile edge
constexpr int NT = WT / 16;                  // MFMA tiles per wave tile edge
constexpr int kLoads = 8;                    // direct loads per operand, step and wave (8 rows each)

// The 16-byte chunk index of row r is XORed with swz16(r).  A fragment read has lane l at row l % 16, chunk
// 2 (l / 16) + q, i.e. four lanes per 128-byte row.  Which swizzles the LDS of gfx950 serves without bank conflicts
// was found by timing all 4096 GF(2)-linear maps row -> 3 bits in a loop of ds_read_b128 from four waves: a third
// of them run at the rate of a contiguous read, this is the one with the fewest terms; (r >> 1) & 7, which
// would be conflict free if 16 consecutive lanes were served together over 64 banks, measured 28 % slower
// (SQ_LDS_BANK_CONFLICT: half of the LDS cycles of the GEMM).
__device__ __forceinline__ int swz16(int r) { return ((r >> 2) & 1) | (((r >> 1) & 1) << 2); }

// Maximum over every aligned group of eight lanes, of two independent 16-bit halves per register, by DPP moves (no
// LDS traffic: an LDS instruction the compiler knows of would make it wait for the direct-to-LDS loads in flight);
// all eight lanes end up with the result.
__device__ __forceinline__ uint32_t dpp_pk_umax16_over8(uint32_t v)
{
    v = pk_umax16(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v = pk_umax16(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v = pk_umax16(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true));  // row_half_mirror
    return v;
}

// Output stores.  A tile's 128 KB are written once and read by a later kernel; left in the L2 as ordinary dirty lines
// they displace the operand panels the XCD's 32 tiles share, and their write-back competes with the next tile's
// first operand loads.  Marked write-through and streaming (sc0 sc1 nt) they pass through: the K steps after an
// epilogue run at the rate of the others (K = 1024: 2350 instead of 2650 cycles per step, the GEMM -9 %), at the price of
// a few hundred cycles more in the epilogue itself; whole steps of the benchmark configurations gain 1-2 %.
// All output stores are buffer stores through the compiler's builtin, which takes these bits.  (Not inline asm: the
// hardware reads a store's data registers after the instruction has issued, and only for stores it knows of does the
// compiler keep later writes to those registers at a distance - an asm store followed by address arithmetic that
// reused its data registers wrote garbage.)
constexpr int kOutStoreAux = 1 | 2 | 16;  // sc0, nt, sc1
// descriptor of `bytes` bytes at p (raw buffer, 32-bit offsets; an offset at or past `bytes` drops the lane's store)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t out_rows(void* p, int bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(p, 0, bytes, 0x00020000);
}

template <typename Problem, int CBSZ_A, int BLGP_B>
__global__ __launch_bounds__(kThreads, 1) void gemm_fp8_m16_kernel(Problem pb)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int r16 = lane & 15, kb = lane >> 4;  // fragment row inside a tile; 32-byte K block of the lane
#ifdef MI8_TILE_TIMELINE
    uint32_t* const tl_out = g_timeline;
    int tl_ev = 0;
    const uint32_t tl_lds = (uint32_t)(uintptr_t)(lptr_t)(lds + LDS_BYTES - TIMELINE_BYTES);
    auto tl_put = [&](int slot, uint64_t t) __attribute__((always_inline)) {
        const uint32_t at = tl_lds + (uint32_t)(slot * 4);
        asm volatile("ds_write_b32 %0, %1" ::"v"(at), "v"((uint32_t)t) : "memory");
    };
    auto tl_stamp = [&](int k) __attribute__((always_inline)) {
        if (tl_out != nullptr && wave == 0) {  // (uniform)
            uint64_t t;
            asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t)::"memory");
            tl_put(tl_ev + k, t);
        }
    };
    if (tl_out != nullptr && wave == 0) {
        for (int i = lane; i < 256; i += 64) tl_put(i, 0);
        uint64_t t;
        asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t)::"memory");
        tl_put(254, t);
    }
#endif

    // ---- fragment read addresses of the stage being read (half q of the lane's 32 K bytes); tile t adds 2048 t
    uint32_t ra[2], rb[2];
    {
        const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)lds;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t chunk = (uint32_t)((2 * kb + q) ^ swz16(r16));
            ra[q] = lds0 + (uint32_t)((wm * WT + r16) * BK) + (chunk << 4);
            rb[q] = lds0 + (uint32_t)(BM * BK + (wn * WT + r16) * BK) + (chunk << 4);
        }
    }
    auto flip_read_stage = [&](int to_stage) __attribute__((always_inline)) {
        const uint32_t delta = to_stage ? (uint32_t)STAGE : (uint32_t)(-STAGE);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            ra[q] += delta;
            rb[q] += delta;
        }
    };
    auto read_a = [&](v4i (&f)[2], int tile, int q) __attribute__((always_inline)) {
        f[q] = *reinterpret_cast<lfrag_t>((uintptr_t)(ra[q] + tile * 16 * BK));
    };
    auto read_b = [&](v4i (&f)[2], int tile, int q) __attribute__((always_inline)) {
        f[q] = *reinterpret_cast<lfrag_t>((uintptr_t)(rb[q] + tile * 16 * BK));
    };

    // ---- direct loads: wave w fills rows [64 w + 8 p, +8) of each operand, p = 0..7; lane -> row 64 w + 8 p + lr
    // (lr = lane / 8), position lane % 8, which holds global chunk (lane % 8) ^ swz16(row); swz16(row) depends on
    // lr only.  The load's lane offset is a resident register per operand and parity of p (row lr of
    // the operand plus the chunk) plus a uniform row offset: one vector add next to the load, and few registers
    // (this kernel runs at the 256-register limit, and a reload from scratch waits on the in-order vector memory
    // counter, i.e. on every store and direct load before it).
    const int lr = lane >> 3;
    uint32_t dv[4];  // [operand][p & 1]
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t ld = k < 2 ? pb.lda : pb.ldb;
        dv[k] = (uint32_t)((int64_t)lr * ld) + ((uint32_t)((lane & 7) ^ swz16(8 * (k & 1) + lr)) << 4);
    }
    // x in 0..15: the first eight -> A rows 8 x, the rest -> B rows 8 (x - 8)
    auto dma_one = [&](const uint8_t* a_origin, const uint8_t* b_origin, int stage, int x) __attribute__((always_inline)) {
        const bool is_a = x < kLoads;
        const int p = x % kLoads;
        uint32_t rows = (uint32_t)((int64_t)(wave * 64 + 8 * p) * (is_a ? pb.lda : pb.ldb));
        asm volatile("" : "+s"(rows));  // opaque: the sum stays one add at the load instead of sixteen resident registers
        const uint32_t o = dv[(is_a ? 0 : 2) + (p & 1)] + rows;
        const uint8_t* src = (is_a ? a_origin : b_origin) + o;
        uint8_t* dst = lds + stage * STAGE + (is_a ? 0 : BM * BK) + (wave * 64 + 8 * (x % kLoads)) * BK;
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)dst, 16, 0, 0);
    };

    // ---- scales.  Nothing in the epilogue may wait on a global load: such a wait also covers the stores of the
    // previous pass and the operand loads in flight for the next tile (one in-order counter).  Single scales are
    // read here, once; scale vectors travel through LDS like the operands: when the load cursor reaches a tile,
    // each wave fetches its 64 row and 64 column scales into the next of four slots with two direct loads, and the
    // waits and barriers of the K steps in between make them visible before the tile's epilogue.  Slots are
    // counted over tiles that have K steps (the cursor skips the others, however many): the cursor is at most
    // two steps, hence two such tiles, ahead of the epilogue that reads a slot.
    // (two-segment problems: a slot holds the four scale vectors of a tile, and two slots are enough - a tile has at
    // least four K steps, so the load cursor is never more than one tile ahead of the tile whose slot is still read)
    constexpr int kSlotBytes = Problem::kTwoSegments ? 2 * SCALE_SLOT : SCALE_SLOT;
    constexpr int kSlotMask = Problem::kTwoSegments ? 1 : SCALE_SLOTS - 1;
    float inv_single = 1.0f;
    if constexpr (Problem::kSwiglu) {
        // The fused problem has two multipliers (x1, x3) and a running maximum of |h| per lane.  They live in the
        // scale-slot area of LDS (unused with single scales), not in registers: the K loop has none to spare.
        float* aux = reinterpret_cast<float*>(lds + 2 * STAGE + OUT_STAGING);
        if (tid == 0) {
            aux[0] = (1.0f / pb.single_sa()) * (1.0f / pb.single_sb());
            aux[1] = (1.0f / pb.single_sa()) * (1.0f / pb.sb3[0]);
        }
        reinterpret_cast<uint32_t*>(aux)[64 + tid] = 0;
    } else if constexpr (!Problem::kVecScales) {
        inv_single = (1.0f / pb.single_sa()) * (1.0f / pb.single_sb());
        asm volatile("" ::"v"(inv_single));  // the value is complete before the first direct load is issued
    }
    int ld_seq = 0, cp_seq = 0;  // tiles with K steps seen by the load cursor / by the epilogue
    auto scale_dma = [&](const TileDesc& d) __attribute__((always_inline)) {
        if constexpr (Problem::kVecScales) {
            uint8_t* slot = lds + 2 * STAGE + OUT_STAGING + (ld_seq & kSlotMask) * kSlotBytes + wave * 256;
            __builtin_amdgcn_global_load_lds((gptr_t)(d.sa + wave * 64 + lane), (lptr_t)slot, 4, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(d.sb + wave * 64 + lane), (lptr_t)(slot + 1024), 4, 0, 0);
            if constexpr (Problem::kTwoSegments) {
                __builtin_amdgcn_global_load_lds((gptr_t)(d.sa2 + wave * 64 + lane), (lptr_t)(slot + 2048), 4, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr_t)(d.sb2 + wave * 64 + lane), (lptr_t)(slot + 3072), 4, 0, 0);
            }
        }
        ++ld_seq;
    };

    // ---- this workgroup's tiles.  Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2: for tiles
    // of equal cost every XCD takes a contiguous range of the tile order (neighbouring tiles share operand panels),
    // its workgroups striding through it; tiles of unequal cost are strided over the whole grid instead
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
    if (my_tiles == 0) {
        if constexpr (Problem::kSwiglu)
            if (lane == 0) pb.h_slots[(int)blockIdx.x * 4 + wave] = 0;
        return;
    }
    auto my_tile = [&](int idx) __attribute__((always_inline)) { return pb.tile(first_tile + idx * tile_stride, cache); };

    // Fused SwiGLU problem: LDS B rows [64 w, 64 w + 64), the rows this wave fetches, are rows 64 (w / 2) .. of B1
    // (even w) or of B3 (odd w); folded into the wave's B cursor once per tile.
    int64_t b_wave_shift = 0;
    if constexpr (Problem::kSwiglu)
        b_wave_shift = (int64_t)(wave & 1) * pb.b3_offset + (int64_t)((wave >> 1) * 64 - wave * 64) * pb.ldb;
    // load cursor: the K step whose stage is fetched next (two steps ahead of the compute cursor); it skips
    // tiles without K steps and, past the last tile, keeps fetching valid data nobody reads
    int ld_tile = -1, ld_kt = 0, ld_nk = 0;
    const uint8_t* ld_a = nullptr;
    const uint8_t* ld_b = nullptr;
    // (two-segment problems) where the cursor continues after step ld_nk1 - 1 of the tile
    int ld_nk1 = 0;
    const uint8_t* ld_a2 = nullptr;
    const uint8_t* ld_b2 = nullptr;
    auto next_load_tile = [&]() __attribute__((always_inline)) {
        while (ld_tile + 1 < my_tiles) {
            ++ld_tile;
            const TileDesc d = my_tile(ld_tile);
            if (d.nk > 0 && d.c != nullptr) {
                ld_a = d.a;
                ld_b = d.b + b_wave_shift;
                ld_nk = d.nk;
                ld_kt = 0;
                if constexpr (Problem::kTwoSegments) {
                    ld_nk1 = d.nk1;
                    ld_a2 = d.a2;
                    ld_b2 = d.b2;
                }
                scale_dma(d);
                return;
            }
        }
        if (ld_a) {  // no further tile with work: rewind to the start of the current one (of its current segment)
            const int back = Problem::kTwoSegments ? ld_kt - ld_nk1 : ld_kt;
            ld_a -= (int64_t)back * BK;
            ld_b -= (int64_t)back * BK;
            ld_kt -= back;
        }
    };
    auto advance_load_cursor = [&]() __attribute__((always_inline)) {
        ++ld_kt;
        ld_a += BK;
        ld_b += BK;
        if constexpr (Problem::kTwoSegments) {
            if (ld_kt == ld_nk1) {  // (uniform) the first pair of operands is used up
                ld_a = ld_a2;
                ld_b = ld_b2;
            }
        }
        if (ld_kt >= ld_nk) next_load_tile();
    };
    next_load_tile();

    v4f acc[NT][NT];
    // D' = B . A^T : the first MFMA operand is the B fragment (its type code goes to cbsz).  `fresh`: the tile's
    // first touch of this accumulator; the MFMA then takes the constant 0 as its addend, so the accumulators
    // never have to be cleared between tiles.
    // kMfmaScale: power-of-two scale vectors are applied inside the MFMAs as block scales - an exponent byte per
    // operand row, 2^(byte - 127), the same for a row's four 32-byte K blocks; the bytes of four tiles share a register
    // and the instruction selects one (ia, jb: the A and B tile of the wave tile).  Scaling every product of an output
    // element by one power of two scales every partial sum alike: the bits are those of scaling the finished sum.
    int ea_lo = 0, ea_hi = 0, eb_lo = 0, eb_hi = 0;
    bool ms_tile = false;  // (wave-uniform) this tile's scales are applied by the MFMAs: the epilogue does not multiply
    auto mma = [&](const v4i (&a)[2], const v4i (&b)[2], v4f& c, bool fresh, int ia, int jb) __attribute__((always_inline)) {
        const v8i fa = __builtin_shufflevector(a[0], a[1], 0, 1, 2, 3, 4, 5, 6, 7);
        const v8i fb = __builtin_shufflevector(b[0], b[1], 0, 1, 2, 3, 4, 5, 6, 7);
        const v4f zero = {0, 0, 0, 0};
        if constexpr (Problem::kMfmaScale) {
            // Written as instructions of their own with the accumulator tied to the result: left to the register
            // allocator, a share of the scaled MFMAs do not accumulate in place, and with all 256 accumulator registers
            // in use the moves that follow end in spills.  (op_sel / op_sel_hi: bits 0 / 1 of the byte each scale
            // register is read at; first the B fragment's, which is the instruction's first matrix operand.)
            const int sca = ia < 4 ? ea_lo : ea_hi, scb = jb < 4 ? eb_lo : eb_hi;
#define MI8_MS_ASM(JB, IA)                                                                                                  \
    case JB * 4 + IA:                                                                                                      \
        if (fresh)                                                                                                         \
            asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel:[" #JB "&1," #IA "&1,0] "        \
                         "op_sel_hi:[" #JB ">>1," #IA ">>1,0] cbsz:%5 blgp:%6"                                             \
                         : "=a"(c)                                                                                         \
                         : "v"(fb), "v"(fa), "v"(scb), "v"(sca), "n"(BLGP_B), "n"(CBSZ_A));                                \
        else                                                                                                               \
            asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[" #JB "&1," #IA "&1,0] "       \
                         "op_sel_hi:[" #JB ">>1," #IA ">>1,0] cbsz:%5 blgp:%6"                                             \
                         : "+a"(c)                                                                                         \
                         : "v"(fb), "v"(fa), "v"(scb), "v"(sca), "n"(BLGP_B), "n"(CBSZ_A));                                \
        break;
            switch ((jb & 3) * 4 + (ia & 3)) {
                MI8_MS_ASM(0, 0) MI8_MS_ASM(0, 1) MI8_MS_ASM(0, 2) MI8_MS_ASM(0, 3)
                MI8_MS_ASM(1, 0) MI8_MS_ASM(1, 1) MI8_MS_ASM(1, 2) MI8_MS_ASM(1, 3)
                MI8_MS_ASM(2, 0) MI8_MS_ASM(2, 1) MI8_MS_ASM(2, 2) MI8_MS_ASM(2, 3)
                MI8_MS_ASM(3, 0) MI8_MS_ASM(3, 1) MI8_MS_ASM(3, 2) MI8_MS_ASM(3, 3)
            }
#undef MI8_MS_ASM
        } else {
            c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, fresh ? zero : c, BLGP_B, CBSZ_A, 0, 0, 0, 0);
        }
    };

    // ---- prologue: stages of steps 0 and 1, fragments of step 0 ----------------------------------------
    if (ld_a != nullptr) {  // uniform
#pragma unroll
        for (int s = 0; s < 2; ++s) {
#pragma unroll
            for (int x = 0; x < 2 * kLoads; ++x) dma_one(ld_a, ld_b, s, x);
            advance_load_cursor();
        }
    }
    // A tiles 0-3, A tiles 4-7, and two sets of B tiles 0-7: a step multiplies from one set while the next step's B
    // fragments are read into the other
    v4i fa_lo[4][2], fa_hi[4][2], fb[2][NT][2];
    // fragments a step's phase A starts from: A tiles 0-3 and all B tiles of the stage the read addresses point at
    auto read_step_head = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            read_a(fa_lo[t], t, 0);
            read_a(fa_lo[t], t, 1);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            read_b(fb[0][t], t, 0);
            read_b(fb[0][t], t, 1);
        }
    };
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct loads have landed
    __syncthreads();
    read_step_head();

    int step = 0;
    for (int cp_tile = 0; cp_tile < my_tiles; ++cp_tile) {
        const TileDesc td = my_tile(cp_tile);
        if (td.c == nullptr) continue;  // (uniform) a grid slot without a tile
        // (kMfmaScale) The tile's scale vectors are in its LDS slot by now (fetched when the load cursor reached the tile,
        // at least two K steps - each with a wait that covers them and a barrier - ago).  Every scale of the wave's 128
        // rows and 128 columns a normal power of two: their inverses go into the MFMAs as exponent bytes.  Anything
        // else (a mantissa, zero, infinity, NaN): the MFMAs run unscaled (byte 127) and the epilogue multiplies.
        // Two-segment problems have no such way out (two sets of scales meet in one accumulator): they read every
        // scale as the power of two its exponent field names.  seg: which pair of vectors of the slot.
        auto load_exponents = [&](int seg) __attribute__((always_inline)) {
            ms_tile = Problem::kTwoSegments;
            ea_lo = ea_hi = eb_lo = eb_hi = 0x7F7F7F7F;
            if (td.nk > 0) {  // (uniform)
                const uint8_t* slot = lds + 2 * STAGE + OUT_STAGING + (cp_seq & kSlotMask) * kSlotBytes + seg * 2048;
                uint32_t pa[2] = {0, 0}, pq[2] = {0, 0}, other = 0;
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const uint32_t ua = *reinterpret_cast<const uint32_t*>(slot + (wm * WT + 16 * t + r16) * 4);
                    const uint32_t ub = *reinterpret_cast<const uint32_t*>(slot + 1024 + (wn * WT + 16 * t + r16) * 4);
                    pa[t >> 2] |= ((254u - (ua >> 23)) & 0xFFu) << (8 * (t & 3));  // 1 / 2^k as an exponent byte
                    pq[t >> 2] |= ((254u - (ub >> 23)) & 0xFFu) << (8 * (t & 3));
                    other |= (ua & 0x7FFFFFu) | (ub & 0x7FFFFFu);
                    other |= (uint32_t)((ua >> 23) - 1u > 253u) | (uint32_t)((ub >> 23) - 1u > 253u);
                }
                if constexpr (!Problem::kTwoSegments) ms_tile = __builtin_amdgcn_ballot_w64(other != 0) == 0;
                if (ms_tile) {
                    ea_lo = (int)pa[0];
                    ea_hi = (int)pa[1];
                    eb_lo = (int)pq[0];
                    eb_hi = (int)pq[1];
                }
            }
        };
        if constexpr (Problem::kMfmaScale) load_exponents(0);
        MI8_TL(0);
        // One 128-byte K step.  `fresh`: the tile's first step; phase A touches the accumulators of A tiles 0-3,
        // phase B those of A tiles 4-7, so both start from 0 then.  The first step is written out separately
        // from the loop, not as a branch inside it.
        // S (a compile-time 0 or 1): the set of B fragments this step multiplies from; the next step's go into the other
        // one.  With a single set, a B tile's next copy could only be requested once its last MFMA of the step was
        // issued, the last tile's at the very end of the step - and the first MFMA of the next step then waited out the
        // LDS latency (the wait at a loop head covers every read in flight).  Now all reads of a step are issued in the
        // first three quarters of phase B.
        auto k_step = [&](bool fresh, auto set_tag) __attribute__((always_inline)) {
            constexpr int S = decltype(set_tag)::value;
            const int cur = step & 1;
            // every wave has issued its reads of this stage's B rows and A tiles 0-3 (previous phase B)
            asm volatile("s_barrier" ::: "memory");
            // phase A: this step's A tiles 4-7 are read behind the first eight MFMAs; the B half of step + 2 is
            // fetched into the B rows of this stage
#pragma unroll
            for (int x = 0; x < 32; ++x) {
                const int j = x >> 2, i = x & 3;
                mma(fa_lo[i], fb[S][j], acc[i][j], fresh, i, j);
                if (x < 8) read_a(fa_hi[x >> 1], 4 + (x >> 1), x & 1);
                if (x >= 8 && x % 3 == 2) dma_one(ld_a, ld_b, cur, kLoads + (x - 8) / 3);
                __builtin_amdgcn_sched_barrier(0);
            }
            // All but this phase's eight loads have landed: the other stage (step + 1) is complete.  (The
            // compiler does not track direct-to-LDS loads across a barrier.)
            // A tile's first step follows the previous tile's epilogue, whose 32 stores (40 with row-segment codes, 48
            // or 52 of the fused SwiGLU problem) are younger than the loads waited for here (one in-order counter):
            // they may stay outstanding as well.
            if (fresh) {
                if constexpr (Problem::kSwiglu) {
                    if (pb.x_codes)  // (uniform)
                        __builtin_amdgcn_s_waitcnt(0xCF7C);  // vmcnt(60): 8 loads, 48 + 4 stores
                    else
                        __builtin_amdgcn_s_waitcnt(0xCF78);  // vmcnt(56)
                } else {
                    __builtin_amdgcn_s_waitcnt(Problem::kOutCodes ? 0xCF70 : 0x8F78);  // vmcnt(48) / vmcnt(40)
                }
            } else
                __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8)
            asm volatile("s_barrier" ::: "memory");
            flip_read_stage(cur ^ 1);
            // phase B: the next step's fragments - all B tiles (into the other set), then A tiles 0-3 - are read
            // behind the first 24 MFMAs; the A half of step + 2 is fetched into the A rows of this stage
#pragma unroll
            for (int x = 0; x < 32; ++x) {
                const int j = x >> 2, i = x & 3;
                mma(fa_hi[i], fb[S][j], acc[4 + i][j], fresh, 4 + i, j);
                if (x < 16) read_b(fb[S ^ 1][x >> 1], x >> 1, x & 1);
                if (x >= 16 && x < 24) read_a(fa_lo[(x - 16) >> 1], (x - 16) >> 1, x & 1);
                if (i == 1) dma_one(ld_a, ld_b, cur, x >> 2);
                __builtin_amdgcn_sched_barrier(0);
            }
            advance_load_cursor();
            ++step;
        };
        if (td.nk > 0) {
            // a tile starts from set 0 (read_step_head) and alternates; what the last step prefetched for the next
            // tile is read again after the epilogue, into set 0
            const std::integral_constant<int, 0> set0;
            const std::integral_constant<int, 1> set1;
            if constexpr (Problem::kTwoSegments) {
                // both segments have an even number of steps: the switch to the second pair's scales falls between
                // two pairs of steps (the fragments of step nk1 were read from the second pair's bytes already)
                k_step(true, set0);
                k_step(false, set1);
                for (int kt = 2; kt < td.nk; kt += 2) {
                    if (kt == td.nk1) load_exponents(1);
                    k_step(false, set0);
                    k_step(false, set1);
                }
            } else {
            k_step(true, set0);
            int kt = 1;
            for (; kt + 1 < td.nk; kt += 2) {
                k_step(false, set1);
                k_step(false, set0);
                if (kt == 1) MI8_TL(1);
            }
            if (kt < td.nk) k_step(false, set1);
            }
        } else {  // nothing is accumulated (empty group): the tile is all zeros
#pragma unroll
            for (int i = 0; i < NT; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j) acc[i][j] = (v4f){0, 0, 0, 0};
        }

        // ---- tile finished: epilogue -------------------------------------------------------------------
        // acc[i][j][e] of lane l is C[row = 16 i + l%16][col = 16 j + 4 (l/16) + e] of the wave tile.
        // A single scale is inverted with an IEEE division, scale vectors with v_rcp_f32 (exact for the
        // power-of-two scales of the axiswise recipes, within 1 ulp otherwise).
        // The wave's output goes through its private staging area 32 rows x 64 columns at a time (4 KB, pitch 128
        // bytes, 16-byte chunk index XORed with (row >> 1) & 7), i.e. two A tiles by four B tiles per pass.
        // (the copies below are opaque to the compiler's hazard handling: the last MFMA has retired after these)
        MI8_TL(2);
        asm volatile("s_nop 15\n\ts_nop 15");
        uint8_t* stg = lds + 2 * STAGE + wave * 4096;
        const uint32_t stg_lds = (uint32_t)(uintptr_t)(lptr_t)stg;
        const bool zero_tile = td.nk == 0;  // nothing accumulated; the scales may be unset
        const uint8_t* sc_slot = lds + 2 * STAGE + OUT_STAGING + (cp_seq & kSlotMask) * kSlotBytes;
        if (!zero_tile) ++cp_seq;
        const int ldc_bytes = (int)pb.ldc * 2;
        const uint32_t c_lane_off = (uint32_t)((lane >> 3) * ldc_bytes + (lane & 7) * 16);
        __amdgpu_buffer_rsrc_t c_rows;
        if constexpr (Problem::kMaskRows)
            c_rows = out_rows(td.c + (int64_t)td.row_lo * pb.ldc, (td.row_hi - td.row_lo) * ldc_bytes);
        // The passes are software pipelined: the staged rows of a pass are read back into registers, and go to
        // memory only after the arithmetic of the next pass, so that each pass exposes one LDS round trip instead
        // of two.
        v4i staged[4];  // (an ext-vector type: arrays of HIP's uint4 struct end up in scratch)
        // Accumulating problems (C += product): what C holds at the addresses of a pass is fetched one pass ahead
        // of the stores that replace it, with the same coalesced 16-byte accesses, and added to the staged rows as
        // an elementwise bf16 add would (float32 sum of the two bf16 values, one rounding).
        v4i held[4];
        auto load_held = [&](int jq, int ih) __attribute__((always_inline)) {
            const int rt = wm * WT + ih * 32;
            if constexpr (Problem::kMaskRows) {
                const int voff = (rt + (lane >> 3) - td.row_lo) * ldc_bytes + (wn * WT + jq * 64 + (lane & 7) * 8) * 2;
#pragma unroll
                for (int it = 0; it < 4; ++it)  // (rows outside the group read as zeros and are not stored)
                    held[it] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(c_rows, voff + it * 8 * ldc_bytes, 0, 2));  // (nt: read once)
            } else {
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const uint8_t* base = reinterpret_cast<const uint8_t*>(td.c + (int64_t)(rt + it * 8) * pb.ldc + wn * WT + jq * 64);
                    uint32_t o = c_lane_off;
                    asm volatile("" : "+v"(o));
                    held[it] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(base + o));  // (read once)
                }
            }
        };
        auto add_held = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int it = 0; it < 4; ++it) staged[it] = add_bf16x8(staged[it], held[it]);
        };
        // Row-segment codes (kOutCodes, and the x codes of the fused SwiGLU problem): a pass holds 32 row segments of
        // 64 columns, eight lanes each (staged[it]: row 8 it + lane / 8).  A lane's eight values give one code per
        // row; a DPP butterfly over the eight lanes leaves the segment's code in all of them; lane j < 4 of every
        // group of eight then stores the code of row 8 j + lane / 8, so the pass writes its 32 codes (64 contiguous
        // bytes) with one store instruction.
        const int code_lane = (lane & 7) * 8 + (lane >> 3);
        auto lane_codes = [&](uint32_t& c01, uint32_t& c23) __attribute__((always_inline)) {
            c01 = (max_code8((uint32_t)staged[0][0], (uint32_t)staged[0][1], (uint32_t)staged[0][2], (uint32_t)staged[0][3]) & 0xFFFFu) |
                  (max_code8((uint32_t)staged[1][0], (uint32_t)staged[1][1], (uint32_t)staged[1][2], (uint32_t)staged[1][3]) & 0xFFFF0000u);
            c23 = (max_code8((uint32_t)staged[2][0], (uint32_t)staged[2][1], (uint32_t)staged[2][2], (uint32_t)staged[2][3]) & 0xFFFFu) |
                  (max_code8((uint32_t)staged[3][0], (uint32_t)staged[3][1], (uint32_t)staged[3][2], (uint32_t)staged[3][3]) & 0xFFFF0000u);
        };
        auto store_codes = [&](uint16_t* codes, int64_t rows_total, int col_block, int ih, uint32_t c01, uint32_t c23)
                               __attribute__((always_inline)) {
            c01 = dpp_pk_umax16_over8(c01);
            c23 = dpp_pk_umax16_over8(c23);
            const uint32_t w = (lane & 2) ? c23 : c01;
            const uint16_t code = (uint16_t)((lane & 1) ? (w >> 16) : (w & 0xFFFFu));
            if ((lane & 7) < 4) codes[(int64_t)col_block * rows_total + td.m0 + wm * WT + ih * 32 + code_lane] = code;
        };
        auto record_codes = [&](int p) __attribute__((always_inline)) {  // p = 4 * jq + ih: the pass whose rows are staged
            if constexpr (Problem::kOutCodes) {
                uint32_t c01, c23;
                lane_codes(c01, c23);
                store_codes(pb.codes, pb.g.M, td.n0 / 64 + wn * 2 + (p >> 2), p & 3, c01, c23);
            }
        };
        auto store_staged = [&](int jq, int ih) __attribute__((always_inline)) {
            const int rt = wm * WT + ih * 32;  // first tile row of the pass
            if constexpr (Problem::kMaskRows) {
                // Only rows [row_lo, row_hi) of the tile belong to this tile's group.  The stores go through a
                // buffer descriptor that spans exactly those rows: a lane whose row lies outside gets an offset
                // below zero (huge when read as unsigned) or past the end, and the hardware drops its store - no
                // divergent branches around the stores.
                const int voff = (rt + (lane >> 3) - td.row_lo) * ldc_bytes + (wn * WT + jq * 64 + (lane & 7) * 8) * 2;
#pragma unroll
                for (int it = 0; it < 4; ++it)
                    __builtin_amdgcn_raw_buffer_store_b128(staged[it], c_rows, voff + it * 8 * ldc_bytes, 0, kOutStoreAux);
            } else {
                // the tile's 256 rows as one buffer: a uniform offset per instruction + one lane offset shared by all passes
                const __amdgpu_buffer_rsrc_t c_tile = out_rows(td.c, 256 * ldc_bytes);
#pragma unroll
                for (int it = 0; it < 4; ++it)
                    __builtin_amdgcn_raw_buffer_store_b128(staged[it], c_tile, c_lane_off,
                                                           (rt + it * 8) * ldc_bytes + (wn * WT + jq * 64) * 2, kOutStoreAux);
            }
        };
        if constexpr (Problem::kSwiglu) {
            // Fused SwiGLU epilogue: the wave holds x1 (B tiles 0-3) and x3 (B tiles 4-7) of the same 128 rows x 64
            // columns.  Per 32 rows: x1 is scaled, rounded and staged; x3 likewise; h = silu(x1) * x3 is formed from
            // the rounded values (the arithmetic of the stand-alone pointwise kernel) and staged; the three outputs
            // leave through the same pipelined staging area as any other tile, twelve passes instead of eight.
            const float* aux = reinterpret_cast<const float*>(lds + 2 * STAGE + OUT_STAGING);
            uint32_t hmax = 0;
            auto store_out = [&](int which, int ih) __attribute__((always_inline)) {
                const int rt = wm * WT + ih * 32;
                const int64_t shift = which == 0 ? 0 : (which == 1 ? pb.x3_offset : pb.h_offset);
                const __amdgpu_buffer_rsrc_t c_tile = out_rows(td.c + shift, 256 * ldc_bytes);
#pragma unroll
                for (int it = 0; it < 4; ++it)
                    __builtin_amdgcn_raw_buffer_store_b128(staged[it], c_tile, c_lane_off, (rt + it * 8) * ldc_bytes + wn * 64 * 2,
                                                           kOutStoreAux);
            };
            // stage one pass (32 rows x 64 columns held as o[t][jj]); the pass before it goes to memory first
            auto stage = [&](const uint2 (&o)[2][4], int prev_which, int prev_ih) __attribute__((always_inline)) {
                asm volatile("" ::: "memory");
                if (prev_which >= 0) {
                    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the previous pass's rows are in registers
                    store_out(prev_which, prev_ih);
                }
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        const int row = 16 * t + r16;
                        const int cw = 16 * jj + 4 * kb;
                        const int chunk = (cw >> 3) ^ ((row >> 1) & 7);
                        const uint32_t saddr = stg_lds + (uint32_t)(row * 128 + chunk * 16 + (cw & 4) * 2);
                        asm volatile("ds_write_b64 %0, %1" ::"v"(saddr), "v"(o[t][jj]) : "memory");
                    }
                __builtin_amdgcn_s_waitcnt(0xc07f);
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int rw = it * 8 + (lane >> 3);
                    staged[it] = *reinterpret_cast<const v4i*>(stg + rw * 128 + (((lane & 7) ^ ((rw >> 1) & 7)) << 4));
                }
                asm volatile("" ::: "memory");
            };
            auto scaled = [&](uint2 (&o)[2][4], int ih, int j0, float mult_in) __attribute__((always_inline)) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    float mult = mult_in;
                    asm volatile("" : "+v"(mult));  // (a loop-invariant multiplier makes the compiler hoist all products)
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            float a_;
                            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a_) : "a"(acc[2 * ih + t][j0 + jj][e]));
                            v[e] = a_ * mult;
                        }
                        o[t][jj].x = pack_bf16x2(v[0], v[1]);
                        o[t][jj].y = pack_bf16x2(v[2], v[3]);
                    }
                }
            };
#pragma unroll
            for (int ih = 0; ih < 4; ++ih) {
                uint2 o1[2][4], o3[2][4], oh[2][4];
                scaled(o1, ih, 0, aux[0]);
                stage(o1, ih == 0 ? -1 : 2, ih - 1);
                uint32_t cx01 = 0, cx23 = 0;  // codes of the x1 rows now staged
                if (pb.x_codes) lane_codes(cx01, cx23);
                scaled(o3, ih, 4, aux[1]);
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        oh[t][jj] = swiglu_fwd4(o1[t][jj], o3[t][jj]);
                        hmax = umax32(hmax, (oh[t][jj].x & 0x7FFFu) << 16);
                        hmax = umax32(hmax, oh[t][jj].x & 0x7FFF0000u);
                        hmax = umax32(hmax, (oh[t][jj].y & 0x7FFFu) << 16);
                        hmax = umax32(hmax, oh[t][jj].y & 0x7FFF0000u);
                    }
                stage(o3, 0, ih);
                if (pb.x_codes) {  // (uniform) the x3 rows are staged: the larger of the two codes per row segment
                    uint32_t c01, c23;
                    lane_codes(c01, c23);
                    store_codes(pb.x_codes, pb.g.M, td.n0 / 64 + wn, ih, pk_umax16(c01, cx01), pk_umax16(c23, cx23));
                }
                stage(oh, 1, ih);
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);
            store_out(2, 3);
            {   // fold this tile's maximum into the lane's slot (an LDS atomic the compiler need not order against
                // the direct loads in flight)
                const uint32_t maddr = (uint32_t)(uintptr_t)(lptr_t)(lds + 2 * STAGE + OUT_STAGING) + (64 + tid) * 4;
                asm volatile("ds_max_u32 %0, %1" ::"v"(maddr), "v"(hmax) : "memory");
            }
        } else {
        // no_mul: the scales were applied inside the MFMAs (kMfmaScale problems, decided per tile)
        auto passes = [&](auto no_mul) __attribute__((always_inline)) {
        constexpr bool kNoMul = decltype(no_mul)::value;
#pragma unroll
        for (int jq = 0; jq < 2; ++jq) {
            float isb[4][4];
            if constexpr (Problem::kVecScales && !kNoMul) {
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const float4 s4 =
                        *reinterpret_cast<const float4*>(sc_slot + 1024 + (wn * WT + jq * 64 + 16 * jj + 4 * kb) * 4);
                    isb[jj][0] = zero_tile ? 0.0f : __builtin_amdgcn_rcpf(s4.x);
                    isb[jj][1] = zero_tile ? 0.0f : __builtin_amdgcn_rcpf(s4.y);
                    isb[jj][2] = zero_tile ? 0.0f : __builtin_amdgcn_rcpf(s4.z);
                    isb[jj][3] = zero_tile ? 0.0f : __builtin_amdgcn_rcpf(s4.w);
                }
            }
#pragma unroll
            for (int ih = 0; ih < 4; ++ih) {
                const int rt = wm * WT + ih * 32;  // first tile row of this pass
                uint2 o[2][4];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    // A single scale is made opaque in every pass: with a loop-invariant multiplier the compiler
                    // forms the products of the whole tile up front and spills accumulators.
                    float mult = inv_single;
                    if constexpr (kNoMul)
                        mult = 1.0f;
                    else if constexpr (Problem::kVecScales)
                        mult = __builtin_amdgcn_rcpf(*reinterpret_cast<const float*>(sc_slot + (rt + 16 * t + r16) * 4));
                    else
                        asm volatile("" : "+v"(mult));
                    if constexpr (!kNoMul) mult = zero_tile ? 0.0f : mult;
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            // The copy out of the accumulator file is an instruction of its own, ordered with the
                            // LDS stores of the passes before it: left to the scheduler, all 256 copies move to
                            // the top of the epilogue and the kernel spills.
                            float a_;
                            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a_) : "a"(acc[2 * ih + t][4 * jq + jj][e]));
                            if constexpr (kNoMul) {
                                v[e] = a_;
                            } else {
                                v[e] = a_ * mult;
                                if constexpr (Problem::kVecScales) v[e] *= isb[jj][e];
                            }
                        }
                        o[t][jj].x = pack_bf16x2(v[0], v[1]);
                        o[t][jj].y = pack_bf16x2(v[2], v[3]);
                    }
                }
                asm volatile("" ::: "memory");  // the stores below stay behind the arithmetic above
                if (jq + ih > 0) {
                    // the previous pass's rows have arrived in registers (so its staging area is free again)
                    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
                    if constexpr (Problem::kAccumulate) add_held();
                    record_codes(4 * jq + ih - 1);
                }
                // (this pass's old C values are requested before the previous pass's stores are issued: the wait for
                // them, one pass later, then leaves those stores outstanding)
                if constexpr (Problem::kAccumulate) load_held(jq, ih);
                if (jq + ih > 0) store_staged(ih == 0 ? jq - 1 : jq, ih == 0 ? 3 : ih - 1);
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        const int row = 16 * t + r16;
                        const int cw = 16 * jj + 4 * kb;  // column inside the 64-column pass, multiple of 4
                        const int chunk = (cw >> 3) ^ ((row >> 1) & 7);
                        // Written as an instruction of its own: before an LDS store it knows of, the compiler
                        // waits for every direct-to-LDS load in flight (it cannot tell that they target other
                        // addresses), i.e. for the operand loads already issued for the next tile.
                        const uint32_t saddr = stg_lds + (uint32_t)(row * 128 + chunk * 16 + (cw & 4) * 2);
                        asm volatile("ds_write_b64 %0, %1" ::"v"(saddr), "v"(o[t][jj]) : "memory");
                    }
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
                MI8_TL(3 + 4 * jq + ih);
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int rw = it * 8 + (lane >> 3);
                    staged[it] = *reinterpret_cast<const v4i*>(stg + rw * 128 + (((lane & 7) ^ ((rw >> 1) & 7)) << 4));
                }
                asm volatile("" ::: "memory");
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        if constexpr (Problem::kAccumulate) add_held();
        record_codes(7);
        store_staged(1, 3);
        MI8_TL(11);
        };
        if constexpr (Problem::kTwoSegments) {
            passes(std::true_type{});
        } else if constexpr (Problem::kMfmaScale) {
            if (ms_tile)
                passes(std::true_type{});
            else
                passes(std::false_type{});
        } else {
            passes(std::false_type{});
        }
        }
        // The last step's phase B has read the next tile's first fragments like any other step; reading them
        // again here makes those 96 registers free during the epilogue, which otherwise spills (and every
        // reload from scratch waits on the in-order vector memory counter, i.e. on the stores above).
        __builtin_amdgcn_sched_barrier(0);  // (or the scheduler moves these reads up into the epilogue)
        read_step_head();
        MI8_TL(12);
        MI8_TL_NEXT_TILE();
    }
    // direct loads issued for steps past the end must have landed before the LDS allocation is released
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    __syncthreads();
#ifdef MI8_TILE_TIMELINE
    if (tl_out != nullptr && wave == 0) {
        uint64_t t;
        asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t)::"memory");
        tl_put(255, t);
        __builtin_amdgcn_s_waitcnt(0xc07f);
        for (int i = lane; i < 256; i += 64)
            tl_out[(int)blockIdx.x * 256 + i] = reinterpret_cast<const uint32_t*>(lds + LDS_BYTES - TIMELINE_BYTES)[i];
    }
#endif
    if constexpr (Problem::kSwiglu) {  // one partial maximum of |h| per wave
        uint32_t m = reinterpret_cast<const uint32_t*>(lds + 2 * STAGE + OUT_STAGING)[64 + tid];
        m = wave_umax(m);
        if (lane == 0) pb.h_slots[(int)blockIdx.x * 4 + wave] = m;
    }
}

// Workgroups of a persistent launch: one per compute unit, or, for fewer tiles, as many as the tiles need - rounded
// up to a multiple of 8, because every XCD takes an eighth of the tiles (rounded up) and needs that many workgroups
// to finish in one round (43 tiles on 43 workgroups: XCDs with 5 workgroups for 6 tiles).
int persistent_blocks(int max_tiles)
{
    const int blocks = num_compute_units();
    const int wanted = (max_tiles + 7) / 8 * 8;
    return blocks > wanted ? wanted : blocks;
}

// persistent: one workgroup per CU walks a static share of the tiles; otherwise one workgroup per tile, handed to
// free CUs by the hardware dispatcher.
template <typename Problem, int CBSZ_A, int BLGP_B>
int launch(const Problem& pb, int max_tiles, bool persistent, hipStream_t st)
{
    auto kern = gemm_fp8_m16_kernel<Problem, CBSZ_A, BLGP_B>;
    // the output stores address the 256 rows of a tile with 32-bit byte offsets
    MI8_REQUIRE(pb.ldc > 0 && pb.ldc < (1 << 22), MI8_ERR_UNSUPPORTED, "mi8 16x16x128 GEMM: output row pitch %lld outside (0, 2^22) elements",
                (long long)pb.ldc);
    static std::atomic<uint64_t> configured{0};
    if (int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), LDS_BYTES, configured, "mi8 16x16x128 GEMM"))
        return rc;
    const int blocks = persistent ? persistent_blocks(max_tiles) : max_tiles;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(kThreads), LDS_BYTES, st, pb);
    return launch_status("mi8 16x16x128 GEMM");
}

template <typename Problem>
int launch_typed(const Problem& pb, int max_tiles, bool persistent, int a_dtype, int b_dtype, hipStream_t st)
{
    if (a_dtype == MI8_E4M3)
        return b_dtype == MI8_E4M3 ? launch<Problem, 0, 0>(pb, max_tiles, persistent, st)
                                   : launch<Problem, 0, 1>(pb, max_tiles, persistent, st);
    return b_dtype == MI8_E4M3 ? launch<Problem, 1, 0>(pb, max_tiles, persistent, st)
                               : launch<Problem, 1, 1>(pb, max_tiles, persistent, st);
}

}  // namespace

int launch_m16(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st)
{
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const int tiles = g.tiles_m * g.tiles_n;
    if (g.sa_vec) {
        if (g.accumulate) return launch_typed(DenseProblem<true, true>{g, g.lda, g.ldb, g.ldc}, tiles, true, a_dtype, b_dtype, st);
        return launch_typed(DenseProblem<true>{g, g.lda, g.ldb, g.ldc}, tiles, true, a_dtype, b_dtype, st);
    }
    if (g.accumulate) return launch_typed(DenseProblem<false, true>{g, g.lda, g.ldb, g.ldc}, tiles, true, a_dtype, b_dtype, st);
    return launch_typed(DenseProblem<false>{g, g.lda, g.ldb, g.ldc}, tiles, true, a_dtype, b_dtype, st);
}

int launch_m16_codes(GemmArgs& g, uint16_t* codes, int a_dtype, int b_dtype, hipStream_t st)
{
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    DenseProblem<false, false, true> pb{g, g.lda, g.ldb, g.ldc};
    pb.codes = codes;
    return launch_typed(pb, g.tiles_m * g.tiles_n, true, a_dtype, b_dtype, st);
}

int launch_m16_swiglu(GemmArgs& g, const uint8_t* b3, const float* sb3, uint16_t* x3, uint16_t* h, uint32_t* h_slots,
                      int* n_slots, uint16_t* x_codes, int a_dtype, int b_dtype, hipStream_t st)
{
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + 127) / 128;
    SwigluProblem pb{g, g.lda, g.ldb, g.ldc, (int64_t)(b3 - g.B), (int64_t)(x3 - reinterpret_cast<uint16_t*>(g.C)),
                     (int64_t)(h - reinterpret_cast<uint16_t*>(g.C)), sb3, h_slots, x_codes};
    const int tiles = g.tiles_m * g.tiles_n;
    *n_slots = 4 * persistent_blocks(tiles);  // one partial maximum per wave of the grid launch() forms from `tiles`
    return launch_typed(pb, tiles, true, a_dtype, b_dtype, st);
}

int launch_m16_grouped(const uint8_t* a, int a_dtype, int64_t lda, const uint8_t* b, int b_dtype, int64_t ldb,
                       int64_t b_group_stride, const int64_t* sizes, int E, int64_t T, int N, int K, const float* sa,
                       const float* sb, int64_t sb_group_stride, uint16_t* out, int64_t ldc, bool accumulate,
                       hipStream_t st)
{
    const int tiles_n = (N + BN - 1) / BN;
    const int64_t max_tiles64 = ((T + BM - 1) / BM + E) * tiles_n;
    const int max_tiles = max_tiles64 > (1 << 30) ? (1 << 30) : (int)max_tiles64;
    if (accumulate) {
        GroupedProblem<true> pb{a, b, out, lda, ldb, ldc, b_group_stride, sb_group_stride, sizes, E, T, N, K, tiles_n, sa, sb};
        return launch_typed(pb, max_tiles, true, a_dtype, b_dtype, st);
    }
    GroupedProblem<false> pb{a, b, out, lda, ldb, ldc, b_group_stride, sb_group_stride, sizes, E, T, N, K, tiles_n, sa, sb};
    return launch_typed(pb, max_tiles, true, a_dtype, b_dtype, st);
}

int launch_m16_grouped_dual(const uint8_t* a1, const uint8_t* a2, int a_dtype, int64_t lda, const uint8_t* b1,
                            const uint8_t* b2, int b_dtype, int64_t ldb, int64_t b_group_stride, const int64_t* sizes, int E,
                            int64_t T, int N, int K1, int K2, const float* sa1, const float* sa2, const float* sb1,
                            const float* sb2, int64_t sb_group_stride, uint16_t* out, int64_t ldc, hipStream_t st)
{
    const int tiles_n = (N + BN - 1) / BN;
    const int64_t max_tiles64 = ((T + BM - 1) / BM + E) * tiles_n;
    const int max_tiles = max_tiles64 > (1 << 30) ? (1 << 30) : (int)max_tiles64;
    GroupedDualProblem pb{{a1, b1, out, lda, ldb, ldc, b_group_stride, sb_group_stride, sizes, E, T, N, K1, tiles_n, sa1, sb1},
                          lda, ldb, ldc, a2, b2, sa2, sb2, K2};
    return launch_typed(pb, max_tiles, true, a_dtype, b_dtype, st);
}

int launch_m16_grouped_wgrad(const uint8_t* a_t, int a_dtype, const uint8_t* b_t, int b_dtype, int64_t ld_t,
                             const int64_t* sizes, int E, int64_t T, int N, int Kl, const float* sa, const float* sb,
                             uint16_t* out, hipStream_t st)
{
    const int tiles_n = (N + BM - 1) / BM, tiles_k = (Kl + BN - 1) / BN;
    GroupedWgradProblem pb{a_t, b_t, out, ld_t, ld_t, Kl, sizes, E, T, N, Kl, tiles_n, tiles_k, sa, sb};
    // persistent: workgroup b walks slots b, b + grid, ... - on its XCD (b % 8 is kept by a stride that is a multiple
    // of 8) these are the same tile position of one group after the other, so the XCD's workgroups stay in step
    return launch_typed(pb, GroupedWgradProblem::grid_tiles(E, tiles_n * tiles_k), true, a_dtype, b_dtype, st);
}

}  // namespace gemm
}  // namespace mi8

#ifdef MI8_TILE_TIMELINE
#include "../../include/mi8_diag.h"
// (declared in mi8_diag.h) One plain GEMM launch, single scales, bf16 output, with the tile timeline recorded.
extern "C" int mi8_diag_gemm_tile_timeline(const void* a, const float* sa, const void* b, const float* sb, void* out, int64_t M,
                                           int64_t N, int64_t K, int a_dtype, int b_dtype, uint32_t* stamps, void* stream)
{
    using namespace mi8;
    MI8_REQUIRE(a && b && sa && sb && out && stamps, MI8_ERR_ARG, "mi8_diag_gemm_tile_timeline: null pointer");
    MI8_REQUIRE(M >= 256 && N >= 256 && K >= 128 && K % 128 == 0 && N % 8 == 0 && M <= (1 << 30) && N <= (1 << 30) && K <= (1 << 30),
                MI8_ERR_UNSUPPORTED, "mi8_diag_gemm_tile_timeline: needs M, N >= 256, K a multiple of 128, N a multiple of 8");
    MI8_REQUIRE((a_dtype == MI8_E4M3 || a_dtype == MI8_E5M2) && (b_dtype == MI8_E4M3 || b_dtype == MI8_E5M2), MI8_ERR_ARG,
                "mi8_diag_gemm_tile_timeline: operand types must be MI8_E4M3 or MI8_E5M2");
    hipStream_t st = (hipStream_t)stream;
    gemm::GemmArgs g{(const uint8_t*)a, (const uint8_t*)b, out, 0, K, K, N, (int)M, (int)N, (int)K, sa, sb, 0, 0, 0, 0, 0};
    // the pointer is a device global of this library: set for this launch only, between stream synchronisations
    MI8_REQUIRE(hipStreamSynchronize(st) == hipSuccess &&
                    hipMemcpyToSymbol(HIP_SYMBOL(gemm::g_timeline), &stamps, sizeof(stamps)) == hipSuccess,
                MI8_ERR_LAUNCH, "mi8_diag_gemm_tile_timeline: could not set the timeline pointer");
    const int rc = gemm::launch_m16(g, a_dtype, b_dtype, st);
    uint32_t* none = nullptr;
    MI8_REQUIRE(hipStreamSynchronize(st) == hipSuccess &&
                    hipMemcpyToSymbol(HIP_SYMBOL(gemm::g_timeline), &none, sizeof(none)) == hipSuccess,
                MI8_ERR_LAUNCH, "mi8_diag_gemm_tile_timeline: launch or reset failed");
    return rc;
}
#endif
