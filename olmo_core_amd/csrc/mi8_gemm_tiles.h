// Problem policies of the persistent direct-to-LDS fp8 GEMM kernels: how a linear tile index maps to operand
// panels, scales and output rows for the dense problem and for the ragged grouped problems (forward /
// grad_input and grad_weight of a dropless-MoE expert layer).
#pragma once
#include "mi8_gemm.h"
#include "mi8_groups.h"

namespace mi8 {
namespace gemm {
namespace {

constexpr int BM = 256, BN = 256;  // output tile of one workgroup

// ---- what a workgroup needs to know about one output tile ---------------------------------------------
struct TileDesc {
    const uint8_t* a;  // first A row of the tile (K offset 0 of the tile's contraction range)
    const uint8_t* b;  // first B row of the tile
    int nk;            // 128-byte K steps (0: the tile is all zeros)
    const float* sa;   // scale of the tile's first row (or the single scale)
    const float* sb;   // scale of the tile's first column (or the single scale)
    uint16_t* c;       // C element (first row, first column) of the tile; null: the slot holds no tile
    int row_lo, row_hi;  // rows [row_lo, row_hi) of the 256 are stored
    int m0, n0;          // (problems that record row-segment codes) first row and column of the tile
    // (two-segment problems) the contraction continues, after nk1 steps, over a second pair of operands with scales
    // of their own
    const uint8_t* a2;
    const uint8_t* b2;
    const float* sa2;
    const float* sb2;
    int nk1;
};

struct NoCache {};

// Dense problem: C[M, N] = A[M, K] . B[N, K]^T.  The last tile row / column is shifted back so that every tile
// is full (M, N >= 256): the overlap is recomputed with the same K order and rewritten with identical values.
// CODES: the epilogue also records, per row segment (64 consecutive columns of a row) of C, the largest magnitude it
// wrote as a 16-bit code (mi8_swiglu.h; codes[(column / 64) * M + row], N % 64 == 0: shifted tiles then start on
// segment boundaries).
template <bool VEC, bool ACC = false, bool CODES = false>
struct DenseProblem {
    GemmArgs g;
    int64_t lda, ldb, ldc;
    uint16_t* codes = nullptr;  // (CODES)
    static constexpr bool kVecScales = VEC;  // both scales are vectors (per row / per column) or both single
    static constexpr bool kAccumulate = ACC;  // C += the rounded product
    static constexpr bool kOutCodes = CODES;
    // (scale vectors applied inside the MFMAs, as the grouped problems do, change nothing here: the K = 4096 rowwise GEMMs
    // of an attention block ran in 3.00-3.02 ms per step either way - under the power limit a shorter epilogue is paid
    // back by a lower clock)
    static constexpr bool kSwiglu = false, kMfmaScale = false, kTwoSegments = false;
    static constexpr bool kMaskRows = false, kXcdRanges = true;
    using Cache = NoCache;
    __device__ __forceinline__ Cache prepare() const { return Cache{}; }
    __device__ __forceinline__ int total_tiles(const Cache&) const { return g.tiles_m * g.tiles_n; }
    // (single-scale problems only) the two scales, the same for every tile
    __device__ __forceinline__ float single_sa() const { return g.sa[0]; }
    __device__ __forceinline__ float single_sb() const { return g.sb[0]; }
    __device__ __forceinline__ TileDesc tile(int t, const Cache&) const
    {
        int tm, tn;
        tile_coords(g, t, tm, tn);
        const int m0 = (tm * BM + BM <= g.M) ? tm * BM : g.M - BM;
        const int n0 = (tn * BN + BN <= g.N) ? tn * BN : g.N - BN;
        TileDesc d;
        d.a = g.A + (int64_t)m0 * g.lda;
        d.b = g.B + (int64_t)n0 * g.ldb;
        d.nk = g.K / BK;
        d.sa = g.sa + (VEC ? m0 : 0);
        d.sb = g.sb + (VEC ? n0 : 0);
        d.c = reinterpret_cast<uint16_t*>(g.C) + (int64_t)m0 * g.ldc + n0;
        d.row_lo = 0;
        d.row_hi = BM;
        d.m0 = m0;
        d.n0 = n0;
        return d;
    }
};

// The two input projections of a SwiGLU feed-forward block in one problem: x1 = A . B1^T, x3 = A . B3^T and
// h = silu(x1) * x3, all [M, H] bf16, single scales.  A 256 x 256 workgroup tile covers 128 columns of H: its B rows
// are, per 128-row half (one half per wave column), 64 rows of B1 followed by the same 64 rows of B3, so that a wave's
// accumulators for B tiles j and j + 4 hold x1 and x3 of the same elements and the epilogue can form h in registers.
// Tiles are shifted back at the ends like the dense problem's (M >= 256, H >= 128).
struct SwigluProblem {
    GemmArgs g;             // A, B = B1, C = x1; N = H; tiles_n counts 128-column tiles; sa, sb = scale of A, of B1
    int64_t lda, ldb, ldc;
    int64_t b3_offset;      // bytes from B1 to B3
    int64_t x3_offset;      // elements from x1 to x3 and to h (same pitch ldc)
    int64_t h_offset;
    const float* sb3;       // scale of B3
    uint32_t* h_slots;      // [4 * workgroups] partial maxima of |h| (float32 bit patterns)
    uint16_t* x_codes;      // null, or [H / 64][M] codes of the larger of x1 and x3 per row segment (H % 64 == 0)
    static constexpr bool kVecScales = false, kAccumulate = false, kSwiglu = true, kOutCodes = false;
    static constexpr bool kMaskRows = false, kXcdRanges = true, kMfmaScale = false, kTwoSegments = false;
    using Cache = NoCache;
    __device__ __forceinline__ Cache prepare() const { return Cache{}; }
    __device__ __forceinline__ int total_tiles(const Cache&) const { return g.tiles_m * g.tiles_n; }
    __device__ __forceinline__ float single_sa() const { return g.sa[0]; }
    __device__ __forceinline__ float single_sb() const { return g.sb[0]; }
    __device__ __forceinline__ TileDesc tile(int t, const Cache&) const
    {
        int tm, tn;
        tile_coords(g, t, tm, tn);
        const int m0 = (tm * BM + BM <= g.M) ? tm * BM : g.M - BM;
        const int n0 = (tn * 128 + 128 <= g.N) ? tn * 128 : g.N - 128;
        TileDesc d;
        d.a = g.A + (int64_t)m0 * g.lda;
        d.b = g.B + (int64_t)n0 * g.ldb;
        d.nk = g.K / BK;
        d.sa = g.sa;
        d.sb = g.sb;
        d.c = reinterpret_cast<uint16_t*>(g.C) + (int64_t)m0 * g.ldc + n0;
        d.row_lo = 0;
        d.row_hi = BM;
        d.m0 = m0;
        d.n0 = n0;
        return d;
    }
};

// Up to 64 groups: the prefix sums live in four registers of every wave for the whole kernel (lane e holds
// group e), and a lookup is a ballot and three lane reads, with no memory access inside the K loop.
struct GroupCache {
    int start, m, ubefore, uend;  // per lane: first row, clamped size, units before, units up to and including
    bool valid;                   // wave-uniform: E <= 64 (otherwise lookups go to memory)
};

template <int U>
__device__ __forceinline__ GroupCache build_group_cache(const int64_t* sizes, int E, int64_t T)
{
    GroupCache c{0, 0, 0, 0, E <= 64};
    if (!c.valid) return c;
    const int lane = (int)threadIdx.x & 63;
    int64_t m = (lane < E) ? sizes[lane] : 0;
    m = m < 0 ? 0 : (m > T ? T : m);
    int64_t end = wave_inclusive_sum(m, lane);
    int64_t start = end - m;
    end = end < T ? end : T;
    start = start < T ? start : T;
    const int64_t me = end - start;
    const int64_t un = (me + U - 1) / U;
    const int64_t uend = wave_inclusive_sum(un, lane);
    c.start = (int)start;  // T < 2^30 is checked on the host
    c.m = (int)me;
    c.ubefore = (int)(uend - un);
    c.uend = (int)uend;
    return c;
}

template <int U, bool BY_UNIT>
__device__ __forceinline__ GroupSpan locate_group_cached(const GroupCache& c, const int64_t* sizes, int E, int64_t T,
                                                         int64_t key)
{
    if (!c.valid) return locate_group<U, BY_UNIT>(sizes, E, T, key);
    int src;
    if constexpr (BY_UNIT) {
        const uint64_t mask = __ballot((int64_t)c.uend > key);
        if (mask == 0) return GroupSpan{E, T, 0, __builtin_amdgcn_readlane(c.uend, 63)};
        src = __ffsll((unsigned long long)mask) - 1;
    } else {
        src = (int)key;
    }
    GroupSpan r;
    r.e = src;
    r.rows_before = __builtin_amdgcn_readlane(c.start, src);
    r.m = __builtin_amdgcn_readlane(c.m, src);
    r.units_before = __builtin_amdgcn_readlane(c.ubefore, src);
    return r;
}

// Ragged-M grouped problem (dropless-MoE forward / grad_input): rows of A form consecutive groups, group e
// multiplies B_e = B + e * b_group_stride.  A tile covers up to 256 rows of ONE group; it always loads a full
// 256-row window (shifted back at the end of the matrix, T >= 256) and stores only its group's rows.
// Scale vectors that are exact powers of two (the axiswise recipes round theirs) are applied inside the MFMAs as block
// scales (kMfmaScale): with K of one or two thousand the vector-scale epilogue - two multiplications per element on a
// wave that has its SIMD to itself - is a third to a half of a tile's time, and this takes the multiplications out.
template <bool ACC = false>
struct GroupedProblem {
    static constexpr bool kAccumulate = ACC;
    static constexpr bool kSwiglu = false, kOutCodes = false, kMfmaScale = true, kTwoSegments = false;
    const uint8_t* A;
    const uint8_t* B;
    uint16_t* C;
    int64_t lda, ldb, ldc, b_group_stride, sb_group_stride;
    const int64_t* sizes;
    int E;
    int64_t T;
    int N, K, tiles_n;
    const float* sa;
    const float* sb;
    static constexpr bool kVecScales = true, kMaskRows = true, kXcdRanges = true;
    using Cache = GroupCache;
    __device__ __forceinline__ Cache prepare() const { return build_group_cache<BM>(sizes, E, T); }
    __device__ __forceinline__ int total_tiles(const Cache& c) const
    {
        const GroupSpan s = locate_group_cached<BM, true>(c, sizes, E, T, (int64_t)1 << 60);
        return (int)s.units_before * tiles_n;
    }
    __device__ __forceinline__ TileDesc tile(int t, const Cache& c) const
    {
        const int mt = t / tiles_n, nt = t % tiles_n;
        const GroupSpan s = locate_group_cached<BM, true>(c, sizes, E, T, mt);
        const int64_t want0 = s.rows_before + (mt - s.units_before) * BM;  // first row this tile is responsible for
        int64_t want1 = want0 + BM;
        const int64_t group_end = s.rows_before + s.m;
        want1 = want1 < group_end ? want1 : group_end;                     // ... up to the group's end
        const int64_t m0 = (want0 + BM <= T) ? want0 : T - BM;             // loaded window
        const int n0 = (nt * BN + BN <= N) ? nt * BN : N - BN;
        TileDesc d;
        d.a = A + m0 * lda;
        d.b = B + (int64_t)s.e * b_group_stride + (int64_t)n0 * ldb;
        d.nk = K / BK;
        d.sa = sa + m0;
        d.sb = sb + (int64_t)s.e * sb_group_stride + n0;
        d.c = C + m0 * ldc + n0;
        d.row_lo = (int)(want0 - m0);
        d.row_hi = (int)(want1 - m0);
        return d;
    }
};

// The sum of two ragged-M grouped products in one accumulation (the grad_input of an expert layer whose input feeds
// two projections: gx = g1 . W1 + g2 . W3): out[rows of e] = A1 . B1_e^T + A2 . B2_e^T, a contraction over K1 + K2 whose
// load cursor moves from the first pair of operands to the second after K1 / 128 steps.  The two products carry
// different scales per row and per column, all exact powers of two (the scale vectors are read as such: only their
// exponents are used), applied inside the MFMAs - so both terms meet in one float32 accumulator and are rounded once:
// no second launch, no read-modify-write of the output.  A1, A2 share a row pitch, B1, B2 a row pitch and group stride,
// the column scales a group stride; K1, K2 are multiples of 256 (an even number of steps each).
struct GroupedDualProblem {
    static constexpr bool kAccumulate = false, kSwiglu = false, kOutCodes = false, kMfmaScale = true, kTwoSegments = true;
    static constexpr bool kVecScales = true, kMaskRows = true, kXcdRanges = true;
    GroupedProblem<false> first;  // A1, B1, C, pitches, sizes, N, K = K1, sa1, sb1
    int64_t lda, ldb, ldc;        // (copies of first's, under the names the kernel reads)
    const uint8_t* A2;
    const uint8_t* B2;
    const float* sa2;
    const float* sb2;
    int K2;
    using Cache = GroupCache;
    __device__ __forceinline__ Cache prepare() const { return first.prepare(); }
    __device__ __forceinline__ int total_tiles(const Cache& c) const { return first.total_tiles(c); }
    __device__ __forceinline__ TileDesc tile(int t, const Cache& c) const
    {
        TileDesc d = first.tile(t, c);
        // the same window of rows, columns and group in the second pair of operands
        d.a2 = A2 + (d.a - first.A);
        d.b2 = B2 + (d.b - first.B);
        d.sa2 = sa2 + (d.sa - first.sa);
        d.sb2 = sb2 + (d.sb - first.sb);
        d.nk1 = d.nk;
        d.nk = d.nk1 + K2 / BK;
        return d;
    }
};

// Ragged-K grouped problem (dropless-MoE grad_weight): out[e] = A_t[:, S_e] . B_t[:, S_e]^T over group e's
// 128-aligned segment S_e of the padded token axis; N, Kl >= 256.  An empty group gives nk = 0: its tiles are
// written as zeros and its scales (never produced) are ignored.
//
// Tile order.  The tiles of one group share its operand panels (tiles_n of A_t, tiles_k of B_t) and cost the same;
// tiles of different groups share nothing and differ in cost by orders of magnitude.  Slot t of the tile order
// belongs to XCD t % 8 (workgroup b runs on XCD b % 8 and walks slots b, b + grid, ...): all tiles of a group are
// given to ONE XCD, whose workgroups run them side by side (its L2 serves every panel to all of them) and move on to
// the XCD's next group together, so a static walk is balanced inside an XCD.  Groups are dealt to the XCDs largest
// first in boustrophedon order (ranks 0..7 to XCDs 0..7, ranks 8..15 to XCDs 7..0, ...), which evens out the XCDs'
// loads for skewed sizes.  The ranks are computed by every wave from the sizes in its registers (E <= 64; more
// groups: in index order).
struct WgradCache {
    GroupCache g;
    int group_at_rank;  // lane p: the group whose size has rank p (ties broken by index)
};

struct GroupedWgradProblem {
    const uint8_t* At;
    const uint8_t* Bt;
    uint16_t* C;
    int64_t lda, ldb, ldc;  // lda = ldb = padded token pitch, ldc = Kl
    const int64_t* sizes;
    int E;
    int64_t T;
    int N, Kl, tiles_n, tiles_k;
    const float* sa;  // [E, N]
    const float* sb;  // [E, Kl]
    static constexpr bool kVecScales = true, kMaskRows = false, kXcdRanges = false;
    static constexpr bool kAccumulate = false, kSwiglu = false, kOutCodes = false, kMfmaScale = false, kTwoSegments = false;
    using Cache = WgradCache;
    __device__ __forceinline__ Cache prepare() const
    {
        Cache c{build_group_cache<128>(sizes, E, T), 0};
        const int lane = (int)threadIdx.x & 63;
        c.group_at_rank = lane;
        if (c.g.valid) {
            const int m = lane < E ? c.g.m : -1;
            int rank = 0;
            for (int j = 0; j < E; ++j) {
                const int mj = __builtin_amdgcn_readlane(c.g.m, j);
                rank += (mj > m || (mj == m && j < lane)) ? 1 : 0;
            }
            for (int j = 0; j < E; ++j)
                if (__builtin_amdgcn_readlane(rank, j) == lane) c.group_at_rank = j;
        }
        return c;
    }
    // slots of the launch grid: 8 XCDs x ceil(E / 8) groups x tiles per group (slots past the last group do nothing)
    __host__ __device__ __forceinline__ static int grid_tiles(int E, int per_group) { return 8 * ((E + 7) / 8) * per_group; }
    __device__ __forceinline__ int total_tiles(const Cache&) const { return grid_tiles(E, tiles_n * tiles_k); }
    __device__ __forceinline__ TileDesc tile(int t, const Cache& c) const
    {
        const int per_group = tiles_n * tiles_k;
        const int xcd = t & 7, slot = t >> 3;
        const int k = slot / per_group, rem = slot % per_group;  // the XCD's k-th group, tile rem of it
        const int rank = (k & 1) ? 8 * k + 7 - xcd : 8 * k + xcd;
        TileDesc d{};
        if (rank >= E) return d;  // d.c == nullptr: nothing to do
        const int e = c.g.valid ? __builtin_amdgcn_readlane(c.group_at_rank, rank) : rank;
        const int tn = rem / tiles_k, tk = rem % tiles_k;
        const GroupSpan s = locate_group_cached<128, false>(c.g, sizes, E, T, e);
        const int64_t seg0 = 128 * s.units_before;
        int64_t seg = 128 * ((s.m + 127) / 128);
        if (seg0 + seg > lda) seg = 0;
        const int n0 = (tn * BM + BM <= N) ? tn * BM : N - BM;
        const int k0 = (tk * BN + BN <= Kl) ? tk * BN : Kl - BN;
        d.a = At + (int64_t)n0 * lda + seg0;
        d.b = Bt + (int64_t)k0 * ldb + seg0;
        d.nk = (int)(seg / BK);
        d.sa = sa + (int64_t)e * N + n0;
        d.sb = sb + (int64_t)e * Kl + k0;
        d.c = C + ((int64_t)e * N + n0) * ldc + k0;
        d.row_lo = 0;
        d.row_hi = BM;
        return d;
    }
};

}  // namespace
}  // namespace gemm
}  // namespace mi8
