// amax reductions and saturating float8 casts (tensorwise, per-row, per-column with transposed output).
// All kernels are HBM-bound streaming kernels: 16-byte loads per lane, wave-shuffle reductions, an
// LDS-staged byte transpose for the transposed copy.
#include <mutex>

#include "mi8_groups.h"
#include "mi8_swiglu.h"

namespace mi8 {
namespace {

constexpr int kThreads = 256;

// ------------------------------------------------------------------------------------------------
// tensorwise amax -> per-workgroup partial maxima
// ------------------------------------------------------------------------------------------------

typedef unsigned short us2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_absmax_u16(uint32_t acc, uint32_t v)
{
    // two bf16 per dword: clear both sign bits, packed unsigned 16-bit max (v_pk_max_u16)
    us2 a = __builtin_bit_cast(us2, acc);
    us2 b = __builtin_bit_cast(us2, v & 0x7FFF7FFFu);
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}

template <int HP>
__device__ __forceinline__ void absmax_accumulate(uint4 v, uint32_t (&acc)[4])
{
    if constexpr (HP == MI8_BF16) {
        acc[0] = pk_absmax_u16(acc[0], v.x);
        acc[1] = pk_absmax_u16(acc[1], v.y);
        acc[2] = pk_absmax_u16(acc[2], v.z);
        acc[3] = pk_absmax_u16(acc[3], v.w);
    } else {
        acc[0] = umax32(acc[0], v.x & 0x7FFFFFFFu);
        acc[1] = umax32(acc[1], v.y & 0x7FFFFFFFu);
        acc[2] = umax32(acc[2], v.z & 0x7FFFFFFFu);
        acc[3] = umax32(acc[3], v.w & 0x7FFFFFFFu);
    }
}

// fold the four accumulators into one float32 |x| bit pattern
template <int HP>
__device__ __forceinline__ uint32_t absmax_fold(const uint32_t (&acc)[4])
{
    if constexpr (HP == MI8_BF16) {
        uint32_t m = pk_absmax_u16(pk_absmax_u16(acc[0], acc[1]), pk_absmax_u16(acc[2], acc[3]));
        uint32_t hi = m >> 16, lo = m & 0xFFFFu;
        return umax32(hi, lo) << 16;
    } else {
        return umax32(umax32(acc[0], acc[1]), umax32(acc[2], acc[3]));
    }
}

__device__ __forceinline__ uint32_t block_umax(uint32_t v, uint32_t* smem /* >= 4 words */)
{
    v = wave_umax(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) smem[wave] = v;
    __syncthreads();
    v = umax32(umax32(smem[0], smem[1]), umax32(smem[2], smem[3]));
    __syncthreads();
    return v;
}

template <int HP>
__global__ __launch_bounds__(kThreads) void amax_partials_kernel(const uint4* __restrict__ x, int64_t nvec,
                                                                 const void* __restrict__ tail, int ntail,
                                                                 uint32_t* __restrict__ slots)
{
    __shared__ uint32_t smem[4];
    uint32_t acc[4] = {0, 0, 0, 0};
    // Every workgroup streams one contiguous range of the tensor, 16 KB per iteration (four independent 16-byte
    // loads in flight per lane): measured 7.0 TB/s against 6.2 TB/s for a grid-stride walk of the same loads.
    const BlockRange r = block_range(nvec);
    int64_t i = r.lo + threadIdx.x;
    for (; i + 3 * kThreads < r.hi; i += 4 * kThreads) {
        uint4 v0 = x[i], v1 = x[i + kThreads], v2 = x[i + 2 * kThreads], v3 = x[i + 3 * kThreads];
        absmax_accumulate<HP>(v0, acc);
        absmax_accumulate<HP>(v1, acc);
        absmax_accumulate<HP>(v2, acc);
        absmax_accumulate<HP>(v3, acc);
    }
    for (; i < r.hi; i += kThreads) absmax_accumulate<HP>(x[i], acc);
    uint32_t m = absmax_fold<HP>(acc);
    if (blockIdx.x == 0 && (int)threadIdx.x < ntail) {
        if constexpr (HP == MI8_BF16)
            m = umax32(m, ((uint32_t) reinterpret_cast<const uint16_t*>(tail)[threadIdx.x] & 0x7FFFu) << 16);
        else
            m = umax32(m, reinterpret_cast<const uint32_t*>(tail)[threadIdx.x] & 0x7FFFFFFFu);
    }
    m = block_umax(m, smem);
    if (threadIdx.x == 0) slots[blockIdx.x] = m;
}

// The same for up to MI8_AMAX_BATCH tensors in one launch (a feed-forward block's input and weights: four launches of
// 20-27 us each spend a third of their time filling and draining the chip).  Tensor t owns workgroups
// [first[t], first[t + 1]) and the slots [t][0 .. first[t + 1] - first[t]).
struct AmaxBatchArgs {
    const void* x[MI8_AMAX_BATCH];
    int64_t n[MI8_AMAX_BATCH];
    int32_t first[MI8_AMAX_BATCH + 1];
    int32_t count;
    uint32_t* slots;
};

template <int HP>
__global__ __launch_bounds__(kThreads) void amax_partials_batch_kernel(AmaxBatchArgs a)
{
    __shared__ uint32_t smem[4];
    int t = 0;
#pragma unroll
    for (int i = 1; i < MI8_AMAX_BATCH; ++i)
        if (i < a.count && (int)blockIdx.x >= a.first[i]) t = i;
    const int block = (int)blockIdx.x - a.first[t], blocks = a.first[t + 1] - a.first[t];
    constexpr int kPerVec = HP == MI8_BF16 ? 8 : 4;
    const uint4* x = reinterpret_cast<const uint4*>(a.x[t]);
    const int64_t nvec = a.n[t] / kPerVec;
    uint32_t acc[4] = {0, 0, 0, 0};
    const BlockRange r = block_range(nvec, block, blocks);
    int64_t i = r.lo + threadIdx.x;
    for (; i + 3 * kThreads < r.hi; i += 4 * kThreads) {
        uint4 v0 = x[i], v1 = x[i + kThreads], v2 = x[i + 2 * kThreads], v3 = x[i + 3 * kThreads];
        absmax_accumulate<HP>(v0, acc);
        absmax_accumulate<HP>(v1, acc);
        absmax_accumulate<HP>(v2, acc);
        absmax_accumulate<HP>(v3, acc);
    }
    for (; i < r.hi; i += kThreads) absmax_accumulate<HP>(x[i], acc);
    uint32_t m = absmax_fold<HP>(acc);
    const int ntail = (int)(a.n[t] % kPerVec);
    if (block == 0 && (int)threadIdx.x < ntail) {
        if constexpr (HP == MI8_BF16)
            m = umax32(m, ((uint32_t) reinterpret_cast<const uint16_t*>(a.x[t])[nvec * kPerVec + threadIdx.x] & 0x7FFFu) << 16);
        else
            m = umax32(m, reinterpret_cast<const uint32_t*>(a.x[t])[nvec * kPerVec + threadIdx.x] & 0x7FFFFFFFu);
    }
    m = block_umax(m, smem);
    if (threadIdx.x == 0) a.slots[(int64_t)t * MI8_AMAX_SLOTS + block] = m;
}

template <int FP8>
__global__ __launch_bounds__(kThreads) void scale_from_partials_kernel(const uint32_t* __restrict__ slots,
                                                                       int n_slots, bool pow2,
                                                                       float* __restrict__ out)
{
    __shared__ uint32_t smem[4];
    uint32_t m = 0;
    for (int i = threadIdx.x; i < n_slots; i += kThreads) m = umax32(m, slots[i]);
    m = block_umax(m, smem);
    if (threadIdx.x == 0) {
        out[0] = scale_from_amax_bits<FP8>(m, pow2);
        out[1] = bits_to_f32(m);
    }
}

// ------------------------------------------------------------------------------------------------
// tile cast: 128 x 128 elements per workgroup, optional row-major output, optional transposed output
// ------------------------------------------------------------------------------------------------

constexpr int kTile = 128;

enum ScaleMode { kScalarFromSlots = 0, kScalarFromPtr = 1, kPerColumnFromWorkspace = 2 };

struct TileCastArgs {
    const void* x;
    int64_t rows, cols;
    const uint32_t* slots;  // kScalarFromSlots: partial maxima; kPerColumnFromWorkspace: [n_slots][cols]
    int n_slots;
    const float* scale_in;
    bool pow2;
    uint8_t* out;    // [rows, ld_out] or null
    int64_t ld_out;
    uint8_t* out_t;  // [cols, ld_t] or null
    int64_t ld_t;
    float* scale_out;  // scalar modes: [1]; per-column mode: [cols]; may be null
};

// Source row of logical row r when the casts read their input through a token permutation (the rows of a
// dropless-MoE expert batch: row r is the token that owns slot gather[r], top_k slots per token); -1 for a slot
// index outside [0, src_rows * top_k) - a dropped token, which reads as a row of zeros.
__device__ __forceinline__ int64_t gathered_row(const int32_t* gather, int top_k, int64_t src_rows, int64_t r, bool ok)
{
    if (!ok) return -1;
    const int64_t slot = gather[r];
    return (slot < 0 || slot >= src_rows * top_k) ? -1 : slot / top_k;
}

// Weight of the slot that logical row r holds (weighted gather: the row is the token's row times this weight, the
// product rounded to the element type as the gather kernel does); 1 without weights.
__device__ __forceinline__ float gathered_weight(const int32_t* gather, const void* w, int w_dtype, int64_t r, bool ok)
{
    if (!w || !ok) return 1.0f;
    const int64_t slot = gather[r];
    if (w_dtype == MI8_F32) return reinterpret_cast<const float*>(w)[slot];
    const uint16_t v = reinterpret_cast<const uint16_t*>(w)[slot];
    return w_dtype == MI8_BF16 ? bits_to_f32((uint32_t)v << 16) : (float)__builtin_bit_cast(_Float16, v);
}

template <int HP>
__device__ __forceinline__ float round_to_hp(float f)
{
    if constexpr (HP == MI8_BF16) return (float)(__bf16)f;
    return f;
}

// LDS holds the transposed tile as 128 columns x 128 row-bytes.  Two columns share a 256-byte line; the
// 16-byte chunk index inside the line is XORed with a function of the column's group of eight so that
// both the dword writes (lanes spread over 16 column groups x 4 row groups) and the 16-byte reads
// (lanes spread over 8 columns x 8 chunks) touch every bank once.
__device__ __forceinline__ int tile_lds_chunk(int col, int part /* 0..7: which 16 row-bytes */)
{
    const int grp = col >> 3;
    const int key = (((grp >> 3) & 1) << 3) | (grp & 7);
    return (col >> 1) * 16 + ((((col & 1) << 3) | part) ^ key);
}

// Quantise one 128 x 128 tile with the eight per-column scales of this lane (all equal for a tensorwise cast):
// rows [row0, row0 + 128) of x (rows >= row_end read as zero and produce zero bytes), columns [col0, col0 + 128).
// Row-major bytes go to out[r, c]; the transposed bytes go to out_t[c, dst0 + (r - row0)] as 16-byte chunks,
// chunks at or beyond dst_end are not written.
template <int HP, int FP8, bool SW>
__device__ __forceinline__ void tile_cast_body(const void* x, int64_t row_end, int64_t cols, int64_t row0, int64_t col0,
                                               const float (&sc)[8], uint8_t* out, int64_t ld_out, uint8_t* out_t, int64_t ld_t,
                                               int64_t dst0, int64_t dst_end, uint32_t* lds_t,
                                               uint8_t* out_r = nullptr, int64_t ld_r = 0, const float* row_scale = nullptr,
                                               int64_t row_scale_row0 = 0, const int32_t* gather = nullptr, int top_k = 1,
                                               int64_t src_rows = 0, const void* gather_w = nullptr, int gather_w_dtype = 0)
{
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int cl = lane & 15, g = lane >> 4;
    const int64_t c8 = col0 + 8 * cl;
    const bool col_ok = c8 < cols;
    const char* xb = reinterpret_cast<const char*>(x);

    float f[2][4][8];
#pragma unroll
    for (int it = 0; it < 2; ++it)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t r = row0 + 32 * wave + 16 * it + 4 * g + j;
            bool ok = col_ok && r < row_end;
            int64_t src = r;
            if (gather) {  // row r of the expert-sorted side is row gather[r] / top_k of x (uniform branch)
                src = gathered_row(gather, top_k, src_rows, r, r < row_end);
                ok = ok && src >= 0;
            }
            if (gather)  // (uniform) a token's row is read top_k times: it stays cached
                HpVec<HP>::load8(xb + (src * cols + c8) * HpVec<HP>::kBytes, ok, f[it][j]);
            else
                HpVec<HP>::template load8<true>(xb + (src * cols + c8) * HpVec<HP>::kBytes, ok, f[it][j]);
            if (gather_w) {  // (uniform) weighted gather: the product, rounded to the element type
                const float w = gathered_weight(gather, gather_w, gather_w_dtype, r, ok);
#pragma unroll
                for (int k = 0; k < 8; ++k) f[it][j][k] = round_to_hp<HP>(f[it][j][k] * w);
            }
        }

    // the rows' own scales, read ahead of the stores below (a read placed between them would wait for them)
    float srow[2][4];
#pragma unroll
    for (int it = 0; it < 2; ++it)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t r = row0 + 32 * wave + 16 * it + 4 * g + j;
            srow[it][j] = (out_r && r < row_end) ? row_scale[r - row_scale_row0] : 0.0f;  // (row_scale[0] = row row_scale_row0)
        }

#pragma unroll
    for (int it = 0; it < 2; ++it) {
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t r = row0 + 32 * wave + 16 * it + 4 * g + j;
            const bool ok = col_ok && r < row_end;
            const float* v = f[it][j];
            lo[j] = quant4<FP8, SW>(v[0], v[1], v[2], v[3], sc[0], sc[1], sc[2], sc[3]);
            hi[j] = quant4<FP8, SW>(v[4], v[5], v[6], v[7], sc[4], sc[5], sc[6], sc[7]);
            if (!ok) lo[j] = hi[j] = 0;  // padding is zero bytes whatever the scale is (0 * NaN is NaN)
            if (out && ok) store_stream8(out + r * ld_out + c8, lo[j], hi[j]);
            if (out_r && ok) {  // the same values quantised with the row's own scale
                const float sr = srow[it][j];
                const uint32_t rl = quant4<FP8, SW>(v[0], v[1], v[2], v[3], sr, sr, sr, sr);
                const uint32_t rh = quant4<FP8, SW>(v[4], v[5], v[6], v[7], sr, sr, sr, sr);
                store_stream8(out_r + r * ld_r + c8, rl, rh);
            }
        }
        if (out_t) {
            uint32_t t[8];
            transpose4x4_bytes(lo[0], lo[1], lo[2], lo[3], t[0], t[1], t[2], t[3]);
            transpose4x4_bytes(hi[0], hi[1], hi[2], hi[3], t[4], t[5], t[6], t[7]);
            const int rd = 8 * wave + 4 * it + g;  // which dword of the column's 32 row-dwords
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int col = 8 * cl + i;
                lds_t[tile_lds_chunk(col, rd >> 2) * 4 + (rd & 3)] = t[i];
            }
        }
    }

    if (out_t) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int q = tid + kThreads * i;
            const int col = q >> 3, part = q & 7;
            const uint4 v = reinterpret_cast<const uint4*>(lds_t)[tile_lds_chunk(col, part)];
            const int64_t c = col0 + col;
            const int64_t d = dst0 + 16 * part;
            if (c < cols && d < dst_end) store_stream16(out_t + c * ld_t + d, v);
        }
    }
}

template <int HP, int FP8, bool SW, int MODE>
__global__ __launch_bounds__(kThreads) void tile_cast_kernel(TileCastArgs a)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds_t[kTile * kTile / 4];
    __shared__ float s_scale[kTile];
    __shared__ uint32_t smem[4];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int cl = lane & 15, g = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * kTile;
    const int64_t col0 = (int64_t)blockIdx.x * kTile;

    // ---- scale(s) -------------------------------------------------------------------------
    float sc[8];
    if constexpr (MODE == kPerColumnFromWorkspace) {
        if (tid < kTile) {
            const int64_t c = col0 + tid;
            float s = 0.0f;
            if (c < a.cols) {
                uint32_t m = 0;
                for (int k = 0; k < a.n_slots; ++k) m = umax32(m, a.slots[(int64_t)k * a.cols + c]);
                s = scale_from_amax_bits<FP8>(m, a.pow2);
                if (blockIdx.y == 0 && a.scale_out) a.scale_out[c] = s;
            }
            s_scale[tid] = s;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; ++i) sc[i] = s_scale[8 * cl + i];
    } else {
        float s;
        if constexpr (MODE == kScalarFromSlots) {
            uint32_t m = 0;
            for (int i = tid; i < a.n_slots; i += kThreads) m = umax32(m, a.slots[i]);
            m = block_umax(m, smem);
            s = scale_from_amax_bits<FP8>(m, a.pow2);  // every lane: same bits in, same bits out
            if (a.scale_out && tid == 0 && blockIdx.x == 0 && blockIdx.y == 0) a.scale_out[0] = s;
        } else {
            s = a.scale_in[0];
            if (a.scale_out && tid == 0 && blockIdx.x == 0 && blockIdx.y == 0) a.scale_out[0] = s;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) sc[i] = s;
    }

    tile_cast_body<HP, FP8, SW>(a.x, a.rows, a.cols, row0, col0, sc, a.out, a.ld_out, a.out_t, a.ld_t, row0,
                                (a.rows + 15) / 16 * 16, lds_t);
}

// ------------------------------------------------------------------------------------------------
// per-column amax partials: workspace[chunk][col] = max |x[r, col]| over the chunk's rows
// ------------------------------------------------------------------------------------------------

template <int HP>
__global__ __launch_bounds__(kThreads) void colamax_kernel(const void* __restrict__ x, int64_t rows,
                                                           int64_t cols, int64_t rows_per_chunk,
                                                           uint32_t* __restrict__ ws)
{
    __shared__ uint32_t red[16][kTile + 1];
    const int tid = threadIdx.x;
    const int cl = tid & 15, rg = tid >> 4;
    const int64_t col0 = (int64_t)blockIdx.x * kTile;
    const int64_t c8 = col0 + 8 * cl;
    const bool col_ok = c8 < cols;
    const int64_t r_begin = (int64_t)blockIdx.y * rows_per_chunk;
    const int64_t r_end = (r_begin + rows_per_chunk < rows) ? r_begin + rows_per_chunk : rows;
    const char* xb = reinterpret_cast<const char*>(x);
    constexpr int NV = HpVec<HP>::kBytes == 2 ? 1 : 2;  // 16-byte vectors per 8 elements

    uint32_t acc[NV][4];
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[v][k] = 0;

    if (col_ok) {
        int64_t r = r_begin + rg;
        for (; r + 48 < r_end; r += 64) {
            uint4 v[4][NV];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int k = 0; k < NV; ++k)
                    v[u][k] = reinterpret_cast<const uint4*>(xb + ((r + 16 * u) * cols + c8) * HpVec<HP>::kBytes)[k];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int k = 0; k < NV; ++k) absmax_accumulate<HP>(v[u][k], acc[k]);
        }
        for (; r < r_end; r += 16) {
#pragma unroll
            for (int k = 0; k < NV; ++k)
                absmax_accumulate<HP>(reinterpret_cast<const uint4*>(xb + (r * cols + c8) * HpVec<HP>::kBytes)[k],
                                      acc[k]);
        }
    }
    // spread this lane's 8 columns into the reduction buffer as float32 |x| bit patterns
    if constexpr (HP == MI8_BF16) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            red[rg][8 * cl + 2 * k] = (acc[0][k] & 0xFFFFu) << 16;
            red[rg][8 * cl + 2 * k + 1] = acc[0][k] & 0xFFFF0000u;
        }
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            red[rg][8 * cl + k] = acc[0][k];
            red[rg][8 * cl + 4 + k] = acc[NV - 1][k];
        }
    }
    __syncthreads();
    if (tid < kTile && col0 + tid < cols) {
        uint32_t m = 0;
#pragma unroll
        for (int k = 0; k < 16; ++k) m = umax32(m, red[k][tid]);
        ws[(int64_t)blockIdx.y * cols + col0 + tid] = m;
    }
}

// ------------------------------------------------------------------------------------------------
// per-row cast: TPR lanes cooperate on one row, the whole row stays in registers between the amax and
// the conversion (single pass over HBM)
// ------------------------------------------------------------------------------------------------

template <int HP, int FP8, bool SW, int TPR /* 64 or 256 */, int NV /* 8-element vectors per lane */>
__global__ __launch_bounds__(kThreads) void rowwise_cast_kernel(const void* __restrict__ x, int64_t rows,
                                                                int64_t cols, bool pow2,
                                                                uint8_t* __restrict__ out, int64_t ld_out,
                                                                float* __restrict__ scale_out)
{
    __shared__ uint32_t smem[4];
    constexpr int ROWS_PER_BLOCK = kThreads / TPR;
    const int tid = threadIdx.x;
    const int sub = tid / TPR, lane = tid % TPR;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + sub;
    const bool row_ok = row < rows;
    const int nvec = (int)(cols >> 3);
    const char* xr = reinterpret_cast<const char*>(x) + row * cols * HpVec<HP>::kBytes;

    float f[NV][8];
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = lane + TPR * i;
        HpVec<HP>::template load8<true>(xr + (int64_t)v * 8 * HpVec<HP>::kBytes, row_ok && v < nvec, f[i]);
        m = umax32(m, absmax8_bits(f[i]));
    }
    if constexpr (TPR == 64)
        m = wave_umax(m);
    else
        m = block_umax(m, smem);
    const float s = scale_from_amax_bits<FP8>(m, pow2);
    if (row_ok && lane == 0) scale_out[row] = s;
    uint8_t* orow = out + row * ld_out;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = lane + TPR * i;
        if (row_ok && v < nvec) {
            const uint32_t lo = quant4<FP8, SW>(f[i][0], f[i][1], f[i][2], f[i][3], s, s, s, s);
            const uint32_t hi = quant4<FP8, SW>(f[i][4], f[i][5], f[i][6], f[i][7], s, s, s, s);
            store_stream8(orow + (int64_t)v * 8, lo, hi);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// grouped per-column cast: rows of x are split into consecutive groups (dropless-MoE experts); every
// group gets its own per-column scales and its transposed bytes start at a multiple of 128 in out_t
// ------------------------------------------------------------------------------------------------

struct GroupedCastArgs {
    const void* x;
    int64_t T, cols;
    const int64_t* sizes;
    int E;
    bool pow2;
    uint32_t* amax;  // [E, cols], zero on entry
    uint8_t* out_t;  // [cols, ld_t]
    int64_t ld_t;
    float* scale_out;  // [E, cols]
    // optional second product of the same two passes: the per-row cast of x (row-major), see
    // mi8_grouped_cast_rows_and_colwise_t
    uint32_t* row_amax;  // [T], zero on entry, or null
    uint8_t* out_r;      // [T, ld_r] or null
    int64_t ld_r;
    float* row_scale;    // [T]
    // optional token permutation in front of the cast (mi8_moe_gather_cast): row r of the [T, cols] input is row
    // gather[r] / top_k of x [src_rows, cols]
    const int32_t* gather;
    int top_k;
    int64_t src_rows;
    const void* gather_w;  // optional weight per slot (weighted gather), of element type gather_w_dtype
    int gather_w_dtype;
};

// Tile p of the padded row space (128 rows each; group e owns ceil(m_e / 128) consecutive tiles) -> its group,
// its rows [row0, row_end) in x (row_end = the group's end) and its destination column 128 p in out_t.
// Sizes are clamped so that nothing past row T is ever read.
// The search is a wave-wide prefix scan over the sizes (gemm::locate_group); walking the sizes one by one cost
// 35 us per launch at 64 groups, every step waiting for its own load.  All lanes return the same values; must be
// called by full waves in uniform control flow.
__device__ __forceinline__ bool locate_padded_tile(const int64_t* sizes, int E, int64_t T, int p, int& e,
                                                   int64_t& row0, int64_t& row_end)
{
    if (E <= 4) {  // a handful of groups (one: the dense two-product cast): walking them is cheaper than a scan
        int64_t before = 0;
        int tiles = 0;
        for (e = 0; e < E; ++e) {
            int64_t m = sizes[e];
            m = m < 0 ? 0 : m;
            m = before + m > T ? T - before : m;
            const int t = (int)((m + kTile - 1) / kTile);
            if (p < tiles + t) {
                row0 = before + (int64_t)kTile * (p - tiles);
                row_end = before + m;
                return true;
            }
            tiles += t;
            before += m;
        }
        return false;
    }
    const gemm::GroupSpan g = gemm::locate_group<kTile, true>(sizes, E, T, p);
    if (g.e >= E) return false;
    e = g.e;
    row0 = g.rows_before + (int64_t)kTile * (p - g.units_before);
    row_end = g.rows_before + g.m;
    return true;
}

// the 16 bytes of a row times the row's gather weight, each product rounded to the element type
template <int HP>
__device__ __forceinline__ uint4 scale_vec(uint4 v, float w)
{
    uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (HP == MI8_BF16) {
            const __bf16 lo = (__bf16)(bits_to_f32(d[i] << 16) * w), hi = (__bf16)(bits_to_f32(d[i] & 0xFFFF0000u) * w);
            d[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        } else {
            d[i] = f32_to_bits(bits_to_f32(d[i]) * w);
        }
    }
    return make_uint4(d[0], d[1], d[2], d[3]);
}

template <int HP>
__global__ __launch_bounds__(kThreads) void grouped_colamax_kernel(GroupedCastArgs a)
{
    __shared__ uint32_t red[16][kTile + 1];
    int e;
    int64_t row0, row_end;
    if (!locate_padded_tile(a.sizes, a.E, a.T, (int)blockIdx.y, e, row0, row_end)) return;
    const int tid = threadIdx.x;
    const int cl = tid & 15, rg = tid >> 4;
    const int64_t col0 = (int64_t)blockIdx.x * kTile;
    const int64_t c8 = col0 + 8 * cl;
    const char* xb = reinterpret_cast<const char*>(a.x);
    constexpr int NV = HpVec<HP>::kBytes == 2 ? 1 : 2;
    uint32_t acc[NV][4];
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[v][k] = 0;
#pragma unroll
    for (int i = 0; i < kTile / 16; ++i) {
        const int64_t r = row0 + rg + 16 * i;
        uint32_t rowacc[4] = {0, 0, 0, 0};
        const int64_t src = a.gather ? gathered_row(a.gather, a.top_k, a.src_rows, r, r < row_end) : r;
        if (c8 < a.cols && r < row_end && src >= 0) {
            const float w = gathered_weight(a.gather, a.gather_w, a.gather_w_dtype, r, true);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                uint4 v = reinterpret_cast<const uint4*>(xb + (src * a.cols + c8) * HpVec<HP>::kBytes)[k];
                if (a.gather_w) v = scale_vec<HP>(v, w);
                absmax_accumulate<HP>(v, acc[k]);
                if (a.row_amax) absmax_accumulate<HP>(v, rowacc);
            }
        }
        if (a.row_amax) {  // uniform; the 16 lanes that share this row fold their eight columns each
            uint32_t m = absmax_fold<HP>(rowacc);
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) m = umax32(m, (uint32_t)__shfl_xor((int)m, off, 16));
            if (cl == 0 && r < row_end && m) atomicMax(&a.row_amax[r], m);
        }
    }
    if constexpr (HP == MI8_BF16) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            red[rg][8 * cl + 2 * k] = (acc[0][k] & 0xFFFFu) << 16;
            red[rg][8 * cl + 2 * k + 1] = acc[0][k] & 0xFFFF0000u;
        }
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            red[rg][8 * cl + k] = acc[0][k];
            red[rg][8 * cl + 4 + k] = acc[NV - 1][k];
        }
    }
    __syncthreads();
    if (tid < kTile && col0 + tid < a.cols) {
        uint32_t m = 0;
#pragma unroll
        for (int k = 0; k < 16; ++k) m = umax32(m, red[k][tid]);
        atomicMax(&a.amax[(int64_t)e * a.cols + col0 + tid], m);  // integer max: order-independent, deterministic
    }
}

// Second pass of the SwiGLU backward of the dense feed-forward block when its two outputs are only ever needed
// in fp8: with the amax of g1 and g3 known (first pass: swiglu_bwd_kernel without outputs), the gradients are
// recomputed from x1, x3, gh tile by tile and go straight to their row-major and transposed fp8 copies - the bf16
// tensors g1 and g3 are never written or read back.  Same arithmetic as swiglu_bwd_kernel followed by
// tile_cast_kernel on each output (the values pass through the same bf16 rounding).
struct SwigluBwdCastArgs {
    const uint4* x1;
    const uint4* x3;
    const uint4* gh;
    int64_t rows, cols;
    const uint32_t* slots1;  // partial maxima of g1 / g3
    const uint32_t* slots3;
    int n_slots;
    bool pow2;
    uint8_t* out1;    // [rows, ld_out] or null
    uint8_t* out3;
    int64_t ld_out;
    uint8_t* out1_t;  // [cols, ld_t] or null
    uint8_t* out3_t;
    int64_t ld_t;
    float* scale_out1;  // [1]
    float* scale_out3;
};

template <int FP8, bool SW>
__global__ __launch_bounds__(kThreads) void swiglu_bwd_cast_kernel(SwigluBwdCastArgs a)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds_t[2][kTile * kTile / 4];
    __shared__ uint32_t smem[4];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int cl = lane & 15, g = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * kTile;
    const int64_t col0 = (int64_t)blockIdx.x * kTile;
    const int64_t c8 = col0 + 8 * cl;
    const bool col_ok = c8 < a.cols;
    const bool first = tid == 0 && blockIdx.x == 0 && blockIdx.y == 0;

    float sc[2];
    {
        uint32_t m1 = 0, m3 = 0;
        for (int i = tid; i < a.n_slots; i += kThreads) {
            m1 = umax32(m1, a.slots1[i]);
            m3 = umax32(m3, a.slots3[i]);
        }
        m1 = block_umax(m1, smem);
        __syncthreads();
        m3 = block_umax(m3, smem);
        sc[0] = scale_from_amax_bits<FP8>(m1, a.pow2);  // every lane: same bits in, same bits out
        sc[1] = scale_from_amax_bits<FP8>(m3, a.pow2);
        if (first) {
            a.scale_out1[0] = sc[0];
            a.scale_out3[0] = sc[1];
        }
    }
    uint8_t* const out[2] = {a.out1, a.out3};
    uint8_t* const out_t[2] = {a.out1_t, a.out3_t};
    const bool want_t = a.out1_t != nullptr;

#pragma unroll
    for (int it = 0; it < 2; ++it) {
        uint4 p[2][4];  // the two gradients of the thread's four rows, eight packed bf16 each
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t r = row0 + 32 * wave + 16 * it + 4 * g + j;
            p[0][j] = p[1][j] = make_uint4(0, 0, 0, 0);
            if (col_ok && r < a.rows) {
                const int64_t v = (r * a.cols + c8) >> 3;
                swiglu_bwd8(load_stream16(a.x1 + v), load_stream16(a.x3 + v), load_stream16(a.gh + v), p[0][j], p[1][j]);
            }
        }
#pragma unroll
        for (int o = 0; o < 2; ++o) {
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int64_t r = row0 + 32 * wave + 16 * it + 4 * g + j;
                const bool ok = col_ok && r < a.rows;
                float v[8];
                unpack8(p[o][j], v);
                lo[j] = quant4<FP8, SW>(v[0], v[1], v[2], v[3], sc[o], sc[o], sc[o], sc[o]);
                hi[j] = quant4<FP8, SW>(v[4], v[5], v[6], v[7], sc[o], sc[o], sc[o], sc[o]);
                if (!ok) lo[j] = hi[j] = 0;  // padding is zero bytes whatever the scale is (0 * NaN is NaN)
                if (out[o] && ok) store_stream8(out[o] + r * a.ld_out + c8, lo[j], hi[j]);
            }
            if (want_t) {
                uint32_t t[8];
                transpose4x4_bytes(lo[0], lo[1], lo[2], lo[3], t[0], t[1], t[2], t[3]);
                transpose4x4_bytes(hi[0], hi[1], hi[2], hi[3], t[4], t[5], t[6], t[7]);
                const int rd = 8 * wave + 4 * it + g;  // which dword of the column's 32 row-dwords
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int col = 8 * cl + i;
                    lds_t[o][tile_lds_chunk(col, rd >> 2) * 4 + (rd & 3)] = t[i];
                }
            }
        }
    }
    if (want_t) {
        __syncthreads();
        const int64_t dst_end = (a.rows + 15) / 16 * 16;
#pragma unroll
        for (int o = 0; o < 2; ++o)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int q = tid + kThreads * i;
                const int col = q >> 3, part = q & 7;
                const uint4 v = reinterpret_cast<const uint4*>(lds_t[o])[tile_lds_chunk(col, part)];
                const int64_t c = col0 + col;
                const int64_t d = row0 + 16 * part;
                if (c < a.cols && d < dst_end) store_stream16(out_t[o] + c * a.ld_t + d, v);
            }
    }
}

// SwiGLU of the dropless-MoE expert layer with the first pass of the two-product cast fused in: the kernel
// writes h = silu(x1) * x2 (or, backward, the gradients g1, g2 of it) in bf16 and takes, of what it writes, the
// amax per (group, column) and per row, exactly what grouped_colamax_kernel would compute in a pass of its own.
struct GroupedSwigluArgs {
    const uint4* x1;
    const uint4* x2;
    const uint4* gh;  // backward only
    uint4* o1;        // forward: h; backward: g1
    uint4* o2;        // backward: g2
    int64_t T, cols;
    const int64_t* sizes;
    int E;
    uint32_t* col_amax1;  // [E, cols], zero on entry
    uint32_t* row_amax1;  // [T], zero on entry
    uint32_t* col_amax2;  // backward only
    uint32_t* row_amax2;
};

template <bool BWD>
__global__ __launch_bounds__(kThreads) void grouped_swiglu_kernel(GroupedSwigluArgs a)
{
    constexpr int NO = BWD ? 2 : 1;
    __shared__ uint32_t red[NO][16][kTile + 1];
    int e;
    int64_t row0, row_end;
    if (!locate_padded_tile(a.sizes, a.E, a.T, (int)blockIdx.y, e, row0, row_end)) return;
    const int tid = threadIdx.x;
    const int cl = tid & 15, rg = tid >> 4;
    const int64_t col0 = (int64_t)blockIdx.x * kTile;
    const int64_t c8 = col0 + 8 * cl;
    uint32_t acc[NO][4];
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[o][k] = 0;
    uint32_t* const row_amax[2] = {a.row_amax1, a.row_amax2};
    uint32_t* const col_amax[2] = {a.col_amax1, a.col_amax2};
#pragma unroll
    for (int i = 0; i < kTile / 16; ++i) {
        const int64_t r = row0 + rg + 16 * i;
        uint32_t rowacc[NO][4];
#pragma unroll
        for (int o = 0; o < NO; ++o)
#pragma unroll
            for (int k = 0; k < 4; ++k) rowacc[o][k] = 0;
        if (c8 < a.cols && r < row_end) {
            const int64_t v = (r * a.cols + c8) >> 3;
            uint4 out[2];
            if constexpr (BWD) {
                swiglu_bwd8(load_stream16(a.x1 + v), load_stream16(a.x2 + v), load_stream16(a.gh + v), out[0], out[1]);
                a.o1[v] = out[0];
                a.o2[v] = out[1];
            } else {
                out[0] = swiglu_fwd8(load_stream16(a.x1 + v), load_stream16(a.x2 + v));
                a.o1[v] = out[0];
            }
#pragma unroll
            for (int o = 0; o < NO; ++o) {
                absmax_accumulate<MI8_BF16>(out[o], acc[o]);
                absmax_accumulate<MI8_BF16>(out[o], rowacc[o]);
            }
        }
#pragma unroll
        for (int o = 0; o < NO; ++o) {  // the 16 lanes that share this row fold their eight columns each
            uint32_t m = absmax_fold<MI8_BF16>(rowacc[o]);
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) m = umax32(m, (uint32_t)__shfl_xor((int)m, off, 16));
            if (cl == 0 && r < row_end && m) atomicMax(&row_amax[o][r], m);
        }
    }
#pragma unroll
    for (int o = 0; o < NO; ++o)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            red[o][rg][8 * cl + 2 * k] = (acc[o][k] & 0xFFFFu) << 16;
            red[o][rg][8 * cl + 2 * k + 1] = acc[o][k] & 0xFFFF0000u;
        }
    __syncthreads();
    if (tid < kTile && col0 + tid < a.cols) {
#pragma unroll
        for (int o = 0; o < NO; ++o) {
            uint32_t m = 0;
#pragma unroll
            for (int k = 0; k < 16; ++k) m = umax32(m, red[o][k][tid]);
            atomicMax(&col_amax[o][(int64_t)e * a.cols + col0 + tid], m);
        }
    }
}

template <int HP, int FP8, bool SW>
__global__ __launch_bounds__(kThreads) void grouped_tile_cast_kernel(GroupedCastArgs a)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds_t[kTile * kTile / 4];
    __shared__ float s_scale[kTile];
    __shared__ float s_row_scale[kTile];
    int e;
    int64_t row0, row_end;
    if (!locate_padded_tile(a.sizes, a.E, a.T, (int)blockIdx.y, e, row0, row_end)) return;
    const int tid = threadIdx.x;
    const int cl = tid & 15;
    const int64_t col0 = (int64_t)blockIdx.x * kTile;
    if (tid < kTile) {
        const int64_t c = col0 + tid;
        float s = 0.0f;
        if (c < a.cols) {
            s = scale_from_amax_bits<FP8>(a.amax[(int64_t)e * a.cols + c], a.pow2);
            a.scale_out[(int64_t)e * a.cols + c] = s;  // every tile of the group writes the same value
        }
        s_scale[tid] = s;
    } else if (a.out_r) {
        // the other half of the workgroup: the scales of the tile's rows from their amax (every column tile
        // derives the same values; the first one publishes them) - no separate launch for [T] scales
        const int64_t r = row0 + tid - kTile;
        float s = 0.0f;
        if (r < row_end) {
            s = scale_from_amax_bits<FP8>(a.row_amax[r], a.pow2);
            if (blockIdx.x == 0) a.row_scale[r] = s;
        }
        s_row_scale[tid - kTile] = s;
    }
    __syncthreads();
    float sc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sc[i] = s_scale[8 * cl + i];
    const int64_t dst0 = (int64_t)kTile * blockIdx.y;
    tile_cast_body<HP, FP8, SW>(a.x, row_end, a.cols, row0, col0, sc, nullptr, 0, a.out_t, a.ld_t, dst0, a.ld_t, lds_t,
                                a.out_r, a.ld_r, s_row_scale, row0, a.gather, a.top_k, a.src_rows, a.gather_w, a.gather_w_dtype);
}

// ---- dispatch helpers ------------------------------------------------------------------------------

template <int HP, int FP8, bool SW>
void launch_tile_cast(int mode, const TileCastArgs& a, dim3 grid, hipStream_t st)
{
    switch (mode) {
        case kScalarFromSlots:
            hipLaunchKernelGGL((tile_cast_kernel<HP, FP8, SW, kScalarFromSlots>), grid, dim3(kThreads), 0, st, a);
            break;
        case kScalarFromPtr:
            hipLaunchKernelGGL((tile_cast_kernel<HP, FP8, SW, kScalarFromPtr>), grid, dim3(kThreads), 0, st, a);
            break;
        default:
            hipLaunchKernelGGL((tile_cast_kernel<HP, FP8, SW, kPerColumnFromWorkspace>), grid, dim3(kThreads), 0,
                               st, a);
            break;
    }
}

void dispatch_tile_cast(int hp, int fp8, bool sw, int mode, const TileCastArgs& a, hipStream_t st)
{
    dim3 grid((unsigned)ceil_div(a.cols, kTile), (unsigned)ceil_div(a.rows, kTile));
#define MI8_TC(HP_, FP8_)                                       \
    if (sw)                                                     \
        launch_tile_cast<HP_, FP8_, true>(mode, a, grid, st);   \
    else                                                        \
        launch_tile_cast<HP_, FP8_, false>(mode, a, grid, st)
    if (hp == MI8_BF16) {
        if (fp8 == MI8_E4M3) { MI8_TC(MI8_BF16, MI8_E4M3); } else { MI8_TC(MI8_BF16, MI8_E5M2); }
    } else {
        if (fp8 == MI8_E4M3) { MI8_TC(MI8_F32, MI8_E4M3); } else { MI8_TC(MI8_F32, MI8_E5M2); }
    }
#undef MI8_TC
}

template <int HP, int FP8, bool SW>
int launch_rowwise(const void* x, int64_t rows, int64_t cols, bool pow2, uint8_t* out, int64_t ld_out, float* scale_out,
                   hipStream_t st)
{
    const int64_t nvec = cols / 8;
#define MI8_RW(TPR_, NV_)                                                                                    \
    hipLaunchKernelGGL((rowwise_cast_kernel<HP, FP8, SW, TPR_, NV_>), dim3((unsigned)ceil_div(rows, kThreads / TPR_)), \
                       dim3(kThreads), 0, st, x, rows, cols, pow2, out, ld_out, scale_out)
    if (nvec <= 64 * 2) { MI8_RW(64, 2); }
    else if (nvec <= 64 * 4) { MI8_RW(64, 4); }
    else if (nvec <= 64 * 8) { MI8_RW(64, 8); }
    else if (nvec <= 256 * 4) { MI8_RW(256, 4); }
    else if (nvec <= 256 * 8) { MI8_RW(256, 8); }
    else if (nvec <= 256 * 16) { MI8_RW(256, 16); }
    else if (nvec <= 256 * 32) { MI8_RW(256, 32); }
    else return MI8_ERR_UNSUPPORTED;
#undef MI8_RW
    return MI8_OK;
}

bool valid_hp(int v) { return v == MI8_BF16 || v == MI8_F32; }
bool valid_fp8(int v) { return v == MI8_E4M3 || v == MI8_E5M2; }

int64_t colamax_rows_per_chunk(int64_t rows)
{
    int64_t rpc = round_up(ceil_div(rows, 32), 16);
    return rpc < 256 ? 256 : rpc;
}

// ---- small tensors: amax, scale and cast in one launch --------------------------------------------------
// A few rows of activations (a generation step) are cast by ONE workgroup: every lane keeps its share of the
// tensor in registers between the amax reduction and the conversion, so the tensorwise cast is one launch
// instead of two and reads x once.  Same helpers as the two-kernel route: same scale, same bytes.
constexpr int kSmallThreads = 1024;
constexpr int kSmallVecs = 8;  // 8-element groups per lane
constexpr int64_t kSmallCastElems = (int64_t)kSmallThreads * kSmallVecs * 8;

template <int HP, int FP8, bool SW>
__global__ __launch_bounds__(kSmallThreads) void small_cast_kernel(const void* __restrict__ x, int64_t rows,
                                                                   int64_t cols, bool pow2, uint8_t* __restrict__ out,
                                                                   int64_t ld_out, float* __restrict__ scale_out)
{
    __shared__ uint32_t smem[kSmallThreads / 64];
    const int tid = threadIdx.x;
    const int64_t groups = rows * cols / 8;  // cols % 16 == 0
    const char* xb = reinterpret_cast<const char*>(x);
    float f[kSmallVecs][8];
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < kSmallVecs; ++i) {
        const int64_t g = tid + (int64_t)kSmallThreads * i;
        HpVec<HP>::load8(xb + g * 8 * HpVec<HP>::kBytes, g < groups, f[i]);  // zeros past the end
        m = umax32(m, absmax8_bits(f[i]));
    }
    m = wave_umax(m);
    if ((tid & 63) == 0) smem[tid >> 6] = m;
    __syncthreads();
    m = 0;
#pragma unroll
    for (int w = 0; w < kSmallThreads / 64; ++w) m = umax32(m, smem[w]);
    const float s = scale_from_amax_bits<FP8>(m, pow2);  // every lane: same bits in, same bits out
    if (tid == 0 && scale_out) scale_out[0] = s;
#pragma unroll
    for (int i = 0; i < kSmallVecs; ++i) {
        const int64_t g = tid + (int64_t)kSmallThreads * i;
        if (g >= groups) continue;
        const int64_t e = g * 8, r = e / cols, c = e % cols;
        const uint32_t lo = quant4<FP8, SW>(f[i][0], f[i][1], f[i][2], f[i][3], s, s, s, s);
        const uint32_t hi = quant4<FP8, SW>(f[i][4], f[i][5], f[i][6], f[i][7], s, s, s, s);
        *reinterpret_cast<uint2*>(out + r * ld_out + c) = make_uint2(lo, hi);
    }
}

template <int HP>
void launch_small_cast(int fp8_dtype, bool sw, const void* x, int64_t rows, int64_t cols, bool pow2, uint8_t* out,
                       int64_t ld_out, float* scale_out, hipStream_t st)
{
    const dim3 grid(1), block(kSmallThreads);
    if (fp8_dtype == MI8_E4M3) {
        if (sw) hipLaunchKernelGGL((small_cast_kernel<HP, MI8_E4M3, true>), grid, block, 0, st, x, rows, cols, pow2, out, ld_out, scale_out);
        else hipLaunchKernelGGL((small_cast_kernel<HP, MI8_E4M3, false>), grid, block, 0, st, x, rows, cols, pow2, out, ld_out, scale_out);
    } else {
        if (sw) hipLaunchKernelGGL((small_cast_kernel<HP, MI8_E5M2, true>), grid, block, 0, st, x, rows, cols, pow2, out, ld_out, scale_out);
        else hipLaunchKernelGGL((small_cast_kernel<HP, MI8_E5M2, false>), grid, block, 0, st, x, rows, cols, pow2, out, ld_out, scale_out);
    }
}

}  // namespace
}  // namespace mi8

using namespace mi8;

extern "C" int32_t mi8_amax_slots_for(int64_t n)
{
    if (n <= 0) return 1;
    // one workgroup per 256 lanes x 4 vectors x 8 (bf16) elements at least, capped by the workspace size
    int64_t blocks = ceil_div(n, (int64_t)kThreads * 4 * 8);
    if (blocks < 1) blocks = 1;
    if (blocks > MI8_AMAX_SLOTS) blocks = MI8_AMAX_SLOTS;
    return (int32_t)blocks;
}

extern "C" int mi8_amax_partials(const void* x, int hp_dtype, int64_t n, uint32_t* slots, int32_t* n_slots_used,
                                 void* stream)
{
    MI8_REQUIRE(x && slots, MI8_ERR_ARG, "mi8_amax_partials: null pointer");
    MI8_REQUIRE(valid_hp(hp_dtype), MI8_ERR_ARG, "mi8_amax_partials: unknown hp dtype %d", hp_dtype);
    MI8_REQUIRE(n > 0, MI8_ERR_ARG, "mi8_amax_partials: n must be positive (got %lld)", (long long)n);
    MI8_REQUIRE(aligned16(x), MI8_ERR_UNSUPPORTED, "mi8_amax_partials: x must be 16-byte aligned");
    const int per_vec = hp_dtype == MI8_BF16 ? 8 : 4;
    const int64_t nvec = n / per_vec;
    const int ntail = (int)(n % per_vec);
    const int esz = hp_dtype == MI8_BF16 ? 2 : 4;
    const void* tail = reinterpret_cast<const char*>(x) + nvec * per_vec * esz;
    const int32_t blocks = mi8_amax_slots_for(n);
    if (n_slots_used) *n_slots_used = blocks;
    hipStream_t st = (hipStream_t)stream;
    if (hp_dtype == MI8_BF16)
        hipLaunchKernelGGL((amax_partials_kernel<MI8_BF16>), dim3(blocks), dim3(kThreads), 0, st,
                           (const uint4*)x, nvec, tail, ntail, slots);
    else
        hipLaunchKernelGGL((amax_partials_kernel<MI8_F32>), dim3(blocks), dim3(kThreads), 0, st, (const uint4*)x,
                           nvec, tail, ntail, slots);
    return launch_status("mi8_amax_partials");
}

extern "C" int mi8_amax_partials_batch(const void* const* xs, const int64_t* ns, int32_t count, int hp_dtype,
                                       uint32_t* slots, int32_t* n_slots_used, void* stream)
{
    MI8_REQUIRE(xs && ns && slots, MI8_ERR_ARG, "mi8_amax_partials_batch: null pointer");
    MI8_REQUIRE(valid_hp(hp_dtype), MI8_ERR_ARG, "mi8_amax_partials_batch: unknown hp dtype %d", hp_dtype);
    MI8_REQUIRE(count > 0 && count <= MI8_AMAX_BATCH, MI8_ERR_ARG, "mi8_amax_partials_batch: %d tensors (1..%d)", count,
                MI8_AMAX_BATCH);
    AmaxBatchArgs a{};
    a.count = count;
    a.slots = slots;
    a.first[0] = 0;
    for (int t = 0; t < count; ++t) {
        MI8_REQUIRE(xs[t] != nullptr, MI8_ERR_ARG, "mi8_amax_partials_batch: tensor %d is null", t);
        MI8_REQUIRE(ns[t] > 0, MI8_ERR_ARG, "mi8_amax_partials_batch: tensor %d has %lld elements", t, (long long)ns[t]);
        MI8_REQUIRE(aligned16(xs[t]), MI8_ERR_UNSUPPORTED, "mi8_amax_partials_batch: tensor %d must be 16-byte aligned", t);
        a.x[t] = xs[t];
        a.n[t] = ns[t];
        const int32_t blocks = mi8_amax_slots_for(ns[t]);
        a.first[t + 1] = a.first[t] + blocks;
        if (n_slots_used) n_slots_used[t] = blocks;
    }
    for (int t = count; t < MI8_AMAX_BATCH; ++t) a.first[t + 1] = a.first[count];
    hipStream_t st = (hipStream_t)stream;
    if (hp_dtype == MI8_BF16)
        hipLaunchKernelGGL((amax_partials_batch_kernel<MI8_BF16>), dim3(a.first[count]), dim3(kThreads), 0, st, a);
    else
        hipLaunchKernelGGL((amax_partials_batch_kernel<MI8_F32>), dim3(a.first[count]), dim3(kThreads), 0, st, a);
    return launch_status("mi8_amax_partials_batch");
}

namespace mi8 {
namespace {

// amax of many tensors in one launch (the per-optimizer-step scale refresh of all float8 weights): block
// (chunk, tensor) folds its share of tensor `blockIdx.y` and merges it with an integer atomic maximum, which is
// order-independent, so the result is deterministic.  Tensors must be 16-byte aligned with numel % 8 == 0 (bf16)
// or % 4 == 0 (float32).
template <int HP>
__global__ __launch_bounds__(kThreads) void multi_amax_kernel(const void* const* __restrict__ ptrs,
                                                              const int64_t* __restrict__ numels,
                                                              uint32_t* __restrict__ amax_bits)
{
    __shared__ uint32_t smem[4];
    const int t = blockIdx.y;
    const uint4* x = reinterpret_cast<const uint4*>(ptrs[t]);
    const int64_t nvec = numels[t] / (HP == MI8_BF16 ? 8 : 4);
    uint32_t acc[4] = {0, 0, 0, 0};
    const BlockRange r = block_range(nvec);
    int64_t i = r.lo + threadIdx.x;
    for (; i + 3 * kThreads < r.hi; i += 4 * kThreads) {
        uint4 v0 = x[i], v1 = x[i + kThreads], v2 = x[i + 2 * kThreads], v3 = x[i + 3 * kThreads];
        absmax_accumulate<HP>(v0, acc);
        absmax_accumulate<HP>(v1, acc);
        absmax_accumulate<HP>(v2, acc);
        absmax_accumulate<HP>(v3, acc);
    }
    for (; i < r.hi; i += kThreads) absmax_accumulate<HP>(x[i], acc);
    uint32_t m = block_umax(absmax_fold<HP>(acc), smem);
    if (threadIdx.x == 0 && m) atomicMax(&amax_bits[t], m);
}

template <int FP8>
__global__ void multi_scale_kernel(const uint32_t* __restrict__ amax_bits, int n, bool pow2, float* __restrict__ scales)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) scales[i] = scale_from_amax_bits<FP8>(amax_bits[i], pow2);
}

__global__ void zero_u32_kernel(uint32_t* p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

}  // namespace
}  // namespace mi8

extern "C" int mi8_multi_tensor_scales(const void* const* ptrs, const int64_t* numels, int32_t n_tensors, int hp_dtype,
                                       int fp8_dtype, uint32_t flags, uint32_t* amax_workspace, float* scales_out,
                                       void* stream)
{
    MI8_REQUIRE(ptrs && numels && amax_workspace && scales_out, MI8_ERR_ARG, "mi8_multi_tensor_scales: null pointer");
    MI8_REQUIRE(valid_hp(hp_dtype) && valid_fp8(fp8_dtype), MI8_ERR_ARG, "mi8_multi_tensor_scales: unknown dtype");
    MI8_REQUIRE(n_tensors > 0 && n_tensors <= 65535, MI8_ERR_ARG, "mi8_multi_tensor_scales: %d tensors (1..65535)",
                n_tensors);
    hipStream_t st = (hipStream_t)stream;
    const unsigned nb = (unsigned)ceil_div(n_tensors, 256);
    hipLaunchKernelGGL(zero_u32_kernel, dim3(nb), dim3(256), 0, st, amax_workspace, n_tensors);
    const dim3 grid(64, (unsigned)n_tensors);
    if (hp_dtype == MI8_BF16)
        hipLaunchKernelGGL((multi_amax_kernel<MI8_BF16>), grid, dim3(kThreads), 0, st, ptrs, numels, amax_workspace);
    else
        hipLaunchKernelGGL((multi_amax_kernel<MI8_F32>), grid, dim3(kThreads), 0, st, ptrs, numels, amax_workspace);
    const bool pow2 = flags & MI8_FLAG_POW2_SCALE;
    if (fp8_dtype == MI8_E4M3)
        hipLaunchKernelGGL((multi_scale_kernel<MI8_E4M3>), dim3(nb), dim3(256), 0, st, amax_workspace, n_tensors, pow2,
                           scales_out);
    else
        hipLaunchKernelGGL((multi_scale_kernel<MI8_E5M2>), dim3(nb), dim3(256), 0, st, amax_workspace, n_tensors, pow2,
                           scales_out);
    return launch_status("mi8_multi_tensor_scales");
}

extern "C" int mi8_scale_from_partials(const uint32_t* slots, int32_t n_slots, int fp8_dtype, uint32_t flags,
                                       float* out, void* stream)
{
    MI8_REQUIRE(slots && out, MI8_ERR_ARG, "mi8_scale_from_partials: null pointer");
    MI8_REQUIRE(valid_fp8(fp8_dtype), MI8_ERR_ARG, "mi8_scale_from_partials: unknown fp8 dtype %d", fp8_dtype);
    MI8_REQUIRE(n_slots > 0 && n_slots <= MI8_AMAX_SLOTS, MI8_ERR_ARG, "mi8_scale_from_partials: n_slots %d out of range",
                n_slots);
    const bool pow2 = flags & MI8_FLAG_POW2_SCALE;
    hipStream_t st = (hipStream_t)stream;
    if (fp8_dtype == MI8_E4M3)
        hipLaunchKernelGGL((scale_from_partials_kernel<MI8_E4M3>), dim3(1), dim3(kThreads), 0, st, slots, n_slots,
                           pow2, out);
    else
        hipLaunchKernelGGL((scale_from_partials_kernel<MI8_E5M2>), dim3(1), dim3(kThreads), 0, st, slots, n_slots,
                           pow2, out);
    return launch_status("mi8_scale_from_partials");
}

extern "C" int mi8_cast_tensorwise(const void* x, int hp_dtype, int64_t rows, int64_t cols, const uint32_t* slots,
                                   int32_t n_slots, const float* scale_in, int fp8_dtype, uint32_t flags, void* out,
                                   int64_t ld_out, void* out_t, int64_t ld_t, float* scale_out, void* stream)
{
    MI8_REQUIRE(x, MI8_ERR_ARG, "mi8_cast_tensorwise: x is null");
    MI8_REQUIRE(out || out_t, MI8_ERR_ARG, "mi8_cast_tensorwise: no output requested");
    MI8_REQUIRE(valid_hp(hp_dtype) && valid_fp8(fp8_dtype), MI8_ERR_ARG, "mi8_cast_tensorwise: unknown dtype");
    MI8_REQUIRE(rows > 0 && cols > 0, MI8_ERR_ARG, "mi8_cast_tensorwise: empty input (%lld x %lld)", (long long)rows,
                (long long)cols);
    MI8_REQUIRE(!(slots && scale_in), MI8_ERR_ARG, "mi8_cast_tensorwise: give slots or scale_in, not both");
    const bool fused_amax = !slots && !scale_in;  // small tensors: amax taken by the cast kernel itself
    MI8_REQUIRE(!fused_amax || (rows * cols <= kSmallCastElems && out && !out_t), MI8_ERR_ARG,
                "mi8_cast_tensorwise: without slots or scale_in the tensor may have at most %lld elements and only "
                "the row-major output (%lld x %lld)",
                (long long)kSmallCastElems, (long long)rows, (long long)cols);
    MI8_REQUIRE(!slots || (n_slots > 0 && n_slots <= MI8_AMAX_SLOTS), MI8_ERR_ARG,
                "mi8_cast_tensorwise: n_slots %d out of range", n_slots);
    MI8_REQUIRE(cols % 16 == 0, MI8_ERR_UNSUPPORTED, "mi8_cast_tensorwise: cols (%lld) must be a multiple of 16",
                (long long)cols);
    MI8_REQUIRE(aligned16(x) && aligned16(out) && aligned16(out_t), MI8_ERR_UNSUPPORTED,
                "mi8_cast_tensorwise: pointers must be 16-byte aligned");
    if (out)
        MI8_REQUIRE(ld_out >= cols && ld_out % 16 == 0, MI8_ERR_UNSUPPORTED,
                    "mi8_cast_tensorwise: ld_out (%lld) must be a multiple of 16 and at least cols", (long long)ld_out);
    if (out_t)
        MI8_REQUIRE(ld_t >= rows && ld_t % 16 == 0, MI8_ERR_UNSUPPORTED,
                    "mi8_cast_tensorwise: ld_t (%lld) must be a multiple of 16 and at least rows", (long long)ld_t);
    if (fused_amax) {
        const bool sw = (flags & MI8_FLAG_SW_CVT) != 0, pow2 = (flags & MI8_FLAG_POW2_SCALE) != 0;
        if (hp_dtype == MI8_BF16)
            launch_small_cast<MI8_BF16>(fp8_dtype, sw, x, rows, cols, pow2, (uint8_t*)out, ld_out, scale_out, (hipStream_t)stream);
        else
            launch_small_cast<MI8_F32>(fp8_dtype, sw, x, rows, cols, pow2, (uint8_t*)out, ld_out, scale_out, (hipStream_t)stream);
        return launch_status("mi8_cast_tensorwise");
    }
    TileCastArgs a{x, rows, cols, slots, n_slots, scale_in, (flags & MI8_FLAG_POW2_SCALE) != 0,
                   (uint8_t*)out, ld_out, (uint8_t*)out_t, ld_t, scale_out};
    dispatch_tile_cast(hp_dtype, fp8_dtype, (flags & MI8_FLAG_SW_CVT) != 0, slots ? kScalarFromSlots : kScalarFromPtr,
                       a, (hipStream_t)stream);
    return launch_status("mi8_cast_tensorwise");
}

// ------------------------------------------------------------------------------------------------
// Tensorwise dynamic cast for callers that cannot allocate: the partial maxima live in a file-scope device
// array instead of a caller-owned workspace.
// ------------------------------------------------------------------------------------------------

static __device__ __align__(256) uint32_t scratch[MI8_AMAX_SLOTS];

namespace mi8 {
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
uint32_t* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each device, looked up once

// The device address of this device's copy of `scratch` (every GPU holds its own copy at its own address; the
// array's name is only a host-side handle for the lookup).
int scratch_for_current_device(uint32_t** out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("mi8_cast_tensorwise_static: cannot identify the current device (%s, device %d)",
                  hipGetErrorString(e), dev);
        return MI8_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_error("mi8_cast_tensorwise_static: hipGetSymbolAddress failed on device %d: %s", dev,
                      hipGetErrorString(e));
            return MI8_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = static_cast<uint32_t*>(p);
    }
    *out = g_scratch_ptr[dev];
    return MI8_OK;
}

}  // namespace
}  // namespace mi8

extern "C" int mi8_cast_tensorwise_static(const void* x, int hp_dtype, int64_t rows, int64_t cols, int fp8_dtype,
                                          uint32_t flags, void* out, int64_t ld_out, void* out_t, int64_t ld_t,
                                          float* scale_out, void* stream)
{
    MI8_REQUIRE(x, MI8_ERR_ARG, "mi8_cast_tensorwise_static: x is null");
    MI8_REQUIRE(valid_hp(hp_dtype), MI8_ERR_ARG, "mi8_cast_tensorwise_static: unknown hp dtype %d", hp_dtype);
    MI8_REQUIRE(rows > 0 && cols > 0, MI8_ERR_ARG, "mi8_cast_tensorwise_static: empty input (%lld x %lld)",
                (long long)rows, (long long)cols);
    MI8_REQUIRE(rows <= MI8_STATIC_CAST_MAX_DIM && cols <= MI8_STATIC_CAST_MAX_DIM &&
                    rows * cols <= MI8_STATIC_CAST_MAX_ELEMS,
                MI8_ERR_UNSUPPORTED,
                "mi8_cast_tensorwise_static: %lld x %lld is beyond the limit of this entry point (each dimension at "
                "most %lld, at most %lld elements); use mi8_amax_partials + mi8_cast_tensorwise with a workspace",
                (long long)rows, (long long)cols, (long long)MI8_STATIC_CAST_MAX_DIM,
                (long long)MI8_STATIC_CAST_MAX_ELEMS);
    uint32_t* slots = nullptr;
    if (int rc = scratch_for_current_device(&slots)) return rc;
    int32_t n_slots = 0;
    // every slot the cast reads is written by this amax pass: nothing has to start at zero
    if (int rc = mi8_amax_partials(x, hp_dtype, rows * cols, slots, &n_slots, stream)) return rc;
    return mi8_cast_tensorwise(x, hp_dtype, rows, cols, slots, n_slots, nullptr, fp8_dtype, flags, out, ld_out, out_t,
                               ld_t, scale_out, stream);
}

extern "C" int mi8_swiglu_bwd_cast(const void* x1, const void* x3, const void* gh, int64_t rows, int64_t cols,
                                   const uint32_t* slots_g1, const uint32_t* slots_g3, int32_t n_slots, int fp8_dtype,
                                   uint32_t flags, void* out1, void* out3, int64_t ld_out, void* out1_t, void* out3_t,
                                   int64_t ld_t, float* scale_out1, float* scale_out3, void* stream)
{
    MI8_REQUIRE(x1 && x3 && gh && slots_g1 && slots_g3 && scale_out1 && scale_out3, MI8_ERR_ARG,
                "mi8_swiglu_bwd_cast: null pointer");
    MI8_REQUIRE((out1 != nullptr) == (out3 != nullptr) && (out1_t != nullptr) == (out3_t != nullptr) && (out1 || out1_t),
                MI8_ERR_ARG, "mi8_swiglu_bwd_cast: request the same layouts (row-major and/or transposed) of both outputs");
    MI8_REQUIRE(valid_fp8(fp8_dtype), MI8_ERR_ARG, "mi8_swiglu_bwd_cast: unknown dtype");
    MI8_REQUIRE(rows > 0 && cols > 0, MI8_ERR_ARG, "mi8_swiglu_bwd_cast: empty input");
    MI8_REQUIRE(n_slots > 0 && n_slots <= MI8_AMAX_SLOTS, MI8_ERR_ARG, "mi8_swiglu_bwd_cast: n_slots %d out of range", n_slots);
    MI8_REQUIRE(cols % 16 == 0, MI8_ERR_UNSUPPORTED, "mi8_swiglu_bwd_cast: cols (%lld) must be a multiple of 16",
                (long long)cols);
    MI8_REQUIRE(aligned16(x1) && aligned16(x3) && aligned16(gh) && aligned16(out1) && aligned16(out3) && aligned16(out1_t) &&
                    aligned16(out3_t),
                MI8_ERR_UNSUPPORTED, "mi8_swiglu_bwd_cast: pointers must be 16-byte aligned");
    if (out1)
        MI8_REQUIRE(ld_out >= cols && ld_out % 16 == 0, MI8_ERR_UNSUPPORTED,
                    "mi8_swiglu_bwd_cast: ld_out (%lld) must be a multiple of 16 and at least cols", (long long)ld_out);
    if (out1_t)
        MI8_REQUIRE(ld_t >= rows && ld_t % 16 == 0, MI8_ERR_UNSUPPORTED,
                    "mi8_swiglu_bwd_cast: ld_t (%lld) must be a multiple of 16 and at least rows", (long long)ld_t);
    SwigluBwdCastArgs a{(const uint4*)x1, (const uint4*)x3, (const uint4*)gh, rows, cols, slots_g1, slots_g3, n_slots,
                        (flags & MI8_FLAG_POW2_SCALE) != 0, (uint8_t*)out1, (uint8_t*)out3, ld_out, (uint8_t*)out1_t,
                        (uint8_t*)out3_t, ld_t, scale_out1, scale_out3};
    const dim3 grid((unsigned)ceil_div(cols, kTile), (unsigned)ceil_div(rows, kTile));
    hipStream_t st = (hipStream_t)stream;
    const bool sw = flags & MI8_FLAG_SW_CVT;
    if (fp8_dtype == MI8_E4M3) {
        if (sw) hipLaunchKernelGGL((swiglu_bwd_cast_kernel<MI8_E4M3, true>), grid, dim3(kThreads), 0, st, a);
        else hipLaunchKernelGGL((swiglu_bwd_cast_kernel<MI8_E4M3, false>), grid, dim3(kThreads), 0, st, a);
    } else {
        if (sw) hipLaunchKernelGGL((swiglu_bwd_cast_kernel<MI8_E5M2, true>), grid, dim3(kThreads), 0, st, a);
        else hipLaunchKernelGGL((swiglu_bwd_cast_kernel<MI8_E5M2, false>), grid, dim3(kThreads), 0, st, a);
    }
    return launch_status("mi8_swiglu_bwd_cast");
}

extern "C" int mi8_cast_rowwise(const void* x, int hp_dtype, int64_t rows, int64_t cols, int fp8_dtype,
                                uint32_t flags, void* out, int64_t ld_out, float* scale_out, void* stream)
{
    MI8_REQUIRE(x && out && scale_out, MI8_ERR_ARG, "mi8_cast_rowwise: null pointer");
    MI8_REQUIRE(ld_out >= cols && ld_out % 16 == 0, MI8_ERR_UNSUPPORTED,
                "mi8_cast_rowwise: ld_out (%lld) must be a multiple of 16 and at least cols", (long long)ld_out);
    MI8_REQUIRE(valid_hp(hp_dtype) && valid_fp8(fp8_dtype), MI8_ERR_ARG, "mi8_cast_rowwise: unknown dtype");
    MI8_REQUIRE(rows > 0 && cols > 0, MI8_ERR_ARG, "mi8_cast_rowwise: empty input");
    MI8_REQUIRE(cols % 16 == 0 && cols <= 65536, MI8_ERR_UNSUPPORTED,
                "mi8_cast_rowwise: cols (%lld) must be a multiple of 16 and at most 65536", (long long)cols);
    MI8_REQUIRE(aligned16(x) && aligned16(out), MI8_ERR_UNSUPPORTED, "mi8_cast_rowwise: pointers must be 16-byte aligned");
    const bool pow2 = flags & MI8_FLAG_POW2_SCALE, sw = flags & MI8_FLAG_SW_CVT;
    hipStream_t st = (hipStream_t)stream;
    int rc;
#define MI8_ROW(HP_, FP8_) \
    rc = sw ? launch_rowwise<HP_, FP8_, true>(x, rows, cols, pow2, (uint8_t*)out, ld_out, scale_out, st) \
            : launch_rowwise<HP_, FP8_, false>(x, rows, cols, pow2, (uint8_t*)out, ld_out, scale_out, st)
    if (hp_dtype == MI8_BF16) {
        if (fp8_dtype == MI8_E4M3) { MI8_ROW(MI8_BF16, MI8_E4M3); } else { MI8_ROW(MI8_BF16, MI8_E5M2); }
    } else {
        if (fp8_dtype == MI8_E4M3) { MI8_ROW(MI8_F32, MI8_E4M3); } else { MI8_ROW(MI8_F32, MI8_E5M2); }
    }
#undef MI8_ROW
    MI8_REQUIRE(rc == MI8_OK, rc, "mi8_cast_rowwise: unsupported row length %lld", (long long)cols);
    return launch_status("mi8_cast_rowwise");
}

extern "C" int64_t mi8_colamax_workspace_slots(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0) return 0;
    return ceil_div(rows, colamax_rows_per_chunk(rows)) * cols;
}

extern "C" int mi8_cast_colwise_t(const void* x, int hp_dtype, int64_t rows, int64_t cols, int fp8_dtype,
                                  uint32_t flags, uint32_t* workspace, void* out_t, int64_t ld_t, float* scale_out,
                                  void* stream)
{
    MI8_REQUIRE(x && workspace && out_t && scale_out, MI8_ERR_ARG, "mi8_cast_colwise_t: null pointer");
    MI8_REQUIRE(valid_hp(hp_dtype) && valid_fp8(fp8_dtype), MI8_ERR_ARG, "mi8_cast_colwise_t: unknown dtype");
    MI8_REQUIRE(rows > 0 && cols > 0, MI8_ERR_ARG, "mi8_cast_colwise_t: empty input");
    MI8_REQUIRE(cols % 16 == 0, MI8_ERR_UNSUPPORTED, "mi8_cast_colwise_t: cols (%lld) must be a multiple of 16",
                (long long)cols);
    MI8_REQUIRE(ld_t >= rows && ld_t % 16 == 0, MI8_ERR_UNSUPPORTED,
                "mi8_cast_colwise_t: ld_t (%lld) must be a multiple of 16 and at least rows", (long long)ld_t);
    MI8_REQUIRE(aligned16(x) && aligned16(out_t), MI8_ERR_UNSUPPORTED,
                "mi8_cast_colwise_t: pointers must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const int64_t rpc = colamax_rows_per_chunk(rows);
    const int n_chunks = (int)ceil_div(rows, rpc);
    dim3 grid((unsigned)ceil_div(cols, kTile), (unsigned)n_chunks);
    if (hp_dtype == MI8_BF16)
        hipLaunchKernelGGL((colamax_kernel<MI8_BF16>), grid, dim3(kThreads), 0, st, x, rows, cols, rpc, workspace);
    else
        hipLaunchKernelGGL((colamax_kernel<MI8_F32>), grid, dim3(kThreads), 0, st, x, rows, cols, rpc, workspace);
    int rc = launch_status("mi8_cast_colwise_t(amax)");
    if (rc != MI8_OK) return rc;
    TileCastArgs a{x, rows, cols, workspace, n_chunks, nullptr, (flags & MI8_FLAG_POW2_SCALE) != 0,
                   nullptr, 0, (uint8_t*)out_t, ld_t, scale_out};
    dispatch_tile_cast(hp_dtype, fp8_dtype, (flags & MI8_FLAG_SW_CVT) != 0, kPerColumnFromWorkspace, a, st);
    return launch_status("mi8_cast_colwise_t(cast)");
}

extern "C" int64_t mi8_grouped_padded_rows(int64_t T, int32_t num_groups)
{
    if (T < 0 || num_groups < 0) return 0;
    // sum of ceil(m_e / 128) over groups whose sizes sum to at most T is at most ceil(T / 128) + num_groups - 1
    return round_up(T, kTile) + (int64_t)kTile * (num_groups > 0 ? num_groups - 1 : 0);
}

namespace mi8 {
namespace {

int grouped_cast_launch(const char* what, const void* x, int hp_dtype, int64_t T, int64_t cols, const int64_t* group_sizes,
                        int32_t num_groups, int fp8_dtype, uint32_t flags, uint32_t* amax_ws, void* out_t, int64_t ld_t,
                        float* scale_out, uint32_t* row_amax_ws, void* out_rows, int64_t ld_rows, float* row_scale_out,
                        void* stream, const int32_t* gather = nullptr, int32_t top_k = 1, int64_t src_rows = 0,
                        const void* gather_w = nullptr, int gather_w_dtype = 0)
{
    MI8_REQUIRE(x && group_sizes && amax_ws && out_t && scale_out, MI8_ERR_ARG, "%s: null pointer", what);
    MI8_REQUIRE(!gather || (top_k > 0 && src_rows > 0 && src_rows * top_k < ((int64_t)1 << 31)), MI8_ERR_ARG,
                "%s: a gathered input needs top_k > 0 and fewer than 2^31 token slots", what);
    MI8_REQUIRE(valid_hp(hp_dtype) && valid_fp8(fp8_dtype), MI8_ERR_ARG, "%s: unknown dtype", what);
    MI8_REQUIRE(T > 0 && cols > 0 && num_groups > 0, MI8_ERR_ARG, "%s: empty input", what);
    MI8_REQUIRE(cols % 16 == 0, MI8_ERR_UNSUPPORTED, "%s: cols (%lld) must be a multiple of 16", what, (long long)cols);
    MI8_REQUIRE(ld_t % 16 == 0 && ld_t >= mi8_grouped_padded_rows(T, num_groups), MI8_ERR_UNSUPPORTED,
                "%s: ld_t (%lld) must be a multiple of 16 and at least mi8_grouped_padded_rows() = %lld", what,
                (long long)ld_t, (long long)mi8_grouped_padded_rows(T, num_groups));
    MI8_REQUIRE(aligned16(x) && aligned16(out_t) && aligned16(out_rows), MI8_ERR_UNSUPPORTED,
                "%s: pointers must be 16-byte aligned", what);
    if (out_rows)
        MI8_REQUIRE(row_amax_ws && row_scale_out && ld_rows >= cols && ld_rows % 16 == 0, MI8_ERR_ARG,
                    "%s: the row output needs its workspace, its scale output and a pitch >= cols (multiple of 16)", what);
    const int64_t ptiles = ceil_div(T, kTile) + num_groups;
    MI8_REQUIRE(ptiles <= 65535, MI8_ERR_UNSUPPORTED, "%s: too many row tiles (%lld)", what, (long long)ptiles);
    const bool pow2 = (flags & MI8_FLAG_POW2_SCALE) != 0;
    GroupedCastArgs a{x, T, cols, group_sizes, num_groups, pow2, amax_ws, (uint8_t*)out_t, ld_t, scale_out,
                      out_rows ? row_amax_ws : nullptr, (uint8_t*)out_rows, ld_rows, row_scale_out, gather, top_k, src_rows, gather_w,
                      gather_w_dtype};
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)ceil_div(cols, kTile), (unsigned)ptiles);
    int rc = MI8_OK;
    if (!(flags & MI8_FLAG_AMAX_READY)) {  // otherwise the workspaces already hold the amax of x
        if (hp_dtype == MI8_BF16)
            hipLaunchKernelGGL((grouped_colamax_kernel<MI8_BF16>), grid, dim3(kThreads), 0, st, a);
        else
            hipLaunchKernelGGL((grouped_colamax_kernel<MI8_F32>), grid, dim3(kThreads), 0, st, a);
        rc = launch_status(what);
        if (rc != MI8_OK) return rc;
    }
    const bool sw = flags & MI8_FLAG_SW_CVT;
#define MI8_GC(HP_, FP8_)                                                                                   \
    if (sw)                                                                                                 \
        hipLaunchKernelGGL((grouped_tile_cast_kernel<HP_, FP8_, true>), grid, dim3(kThreads), 0, st, a);    \
    else                                                                                                    \
        hipLaunchKernelGGL((grouped_tile_cast_kernel<HP_, FP8_, false>), grid, dim3(kThreads), 0, st, a)
    if (hp_dtype == MI8_BF16) {
        if (fp8_dtype == MI8_E4M3) { MI8_GC(MI8_BF16, MI8_E4M3); } else { MI8_GC(MI8_BF16, MI8_E5M2); }
    } else {
        if (fp8_dtype == MI8_E4M3) { MI8_GC(MI8_F32, MI8_E4M3); } else { MI8_GC(MI8_F32, MI8_E5M2); }
    }
#undef MI8_GC
    return launch_status(what);
}

}  // namespace
}  // namespace mi8

extern "C" int mi8_grouped_cast_colwise_t(const void* x, int hp_dtype, int64_t T, int64_t cols,
                                          const int64_t* group_sizes, int32_t num_groups, int fp8_dtype,
                                          uint32_t flags, uint32_t* amax_ws, void* out_t, int64_t ld_t,
                                          float* scale_out, void* stream)
{
    return grouped_cast_launch("mi8_grouped_cast_colwise_t", x, hp_dtype, T, cols, group_sizes, num_groups, fp8_dtype,
                               flags, amax_ws, out_t, ld_t, scale_out, nullptr, nullptr, 0, nullptr, stream);
}

extern "C" int mi8_grouped_cast_rows_and_colwise_t(const void* x, int hp_dtype, int64_t T, int64_t cols,
                                                   const int64_t* group_sizes, int32_t num_groups, int fp8_dtype,
                                                   uint32_t flags, uint32_t* amax_ws, void* out_t, int64_t ld_t,
                                                   float* scale_out, uint32_t* row_amax_ws, void* out_rows,
                                                   int64_t ld_rows, float* row_scale_out, void* stream)
{
    MI8_REQUIRE(out_rows, MI8_ERR_ARG, "mi8_grouped_cast_rows_and_colwise_t: out_rows is null");
    return grouped_cast_launch("mi8_grouped_cast_rows_and_colwise_t", x, hp_dtype, T, cols, group_sizes, num_groups,
                               fp8_dtype, flags, amax_ws, out_t, ld_t, scale_out, row_amax_ws, out_rows, ld_rows,
                               row_scale_out, stream);
}

namespace mi8 {
namespace {

int grouped_swiglu_launch(const char* what, const GroupedSwigluArgs& a, bool bwd, void* stream)
{
    MI8_REQUIRE(a.x1 && a.x2 && a.o1 && a.sizes && a.col_amax1 && a.row_amax1, MI8_ERR_ARG, "%s: null pointer", what);
    if (bwd) MI8_REQUIRE(a.gh && a.o2 && a.col_amax2 && a.row_amax2, MI8_ERR_ARG, "%s: null pointer", what);
    MI8_REQUIRE(a.T > 0 && a.cols > 0 && a.E > 0, MI8_ERR_ARG, "%s: empty input", what);
    MI8_REQUIRE(a.cols % 16 == 0, MI8_ERR_UNSUPPORTED, "%s: cols (%lld) must be a multiple of 16", what, (long long)a.cols);
    MI8_REQUIRE(aligned16(a.x1) && aligned16(a.x2) && aligned16(a.gh) && aligned16(a.o1) && aligned16(a.o2),
                MI8_ERR_UNSUPPORTED, "%s: pointers must be 16-byte aligned", what);
    const int64_t ptiles = ceil_div(a.T, kTile) + a.E;
    MI8_REQUIRE(ptiles <= 65535, MI8_ERR_UNSUPPORTED, "%s: too many row tiles (%lld)", what, (long long)ptiles);
    dim3 grid((unsigned)ceil_div(a.cols, kTile), (unsigned)ptiles);
    if (bwd)
        hipLaunchKernelGGL((grouped_swiglu_kernel<true>), grid, dim3(kThreads), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((grouped_swiglu_kernel<false>), grid, dim3(kThreads), 0, (hipStream_t)stream, a);
    return launch_status(what);
}

}  // namespace
}  // namespace mi8

extern "C" int mi8_grouped_swiglu_fwd(const void* x1, const void* x2, int64_t T, int64_t cols, const int64_t* group_sizes,
                                      int32_t num_groups, void* h, uint32_t* amax_ws, uint32_t* row_amax_ws, void* stream)
{
    GroupedSwigluArgs a{(const uint4*)x1, (const uint4*)x2, nullptr, (uint4*)h, nullptr, T, cols, group_sizes, num_groups,
                        amax_ws, row_amax_ws, nullptr, nullptr};
    return grouped_swiglu_launch("mi8_grouped_swiglu_fwd", a, false, stream);
}

extern "C" int mi8_grouped_swiglu_bwd(const void* x1, const void* x2, const void* gh, int64_t T, int64_t cols,
                                      const int64_t* group_sizes, int32_t num_groups, void* g1, void* g2,
                                      uint32_t* amax_ws1, uint32_t* row_amax_ws1, uint32_t* amax_ws2,
                                      uint32_t* row_amax_ws2, void* stream)
{
    GroupedSwigluArgs a{(const uint4*)x1, (const uint4*)x2, (const uint4*)gh, (uint4*)g1, (uint4*)g2, T, cols, group_sizes,
                        num_groups, amax_ws1, row_amax_ws1, amax_ws2, row_amax_ws2};
    return grouped_swiglu_launch("mi8_grouped_swiglu_bwd", a, true, stream);
}

extern "C" int mi8_moe_gather_cast_rows_and_colwise_t(const void* x, int hp_dtype, int64_t tokens, int64_t cols,
                                                      const int32_t* indices, int32_t top_k, const void* weights,
                                                      int w_dtype, const int64_t* group_sizes,
                                                      int32_t num_groups, int fp8_dtype, uint32_t flags,
                                                      uint32_t* amax_ws, void* out_t, int64_t ld_t, float* scale_out,
                                                      uint32_t* row_amax_ws, void* out_rows, int64_t ld_rows,
                                                      float* row_scale_out, void* stream)
{
    MI8_REQUIRE(indices && out_rows, MI8_ERR_ARG, "mi8_moe_gather_cast_rows_and_colwise_t: null pointer");
    MI8_REQUIRE(tokens > 0 && top_k > 0, MI8_ERR_ARG, "mi8_moe_gather_cast_rows_and_colwise_t: empty input");
    MI8_REQUIRE(!(flags & MI8_FLAG_AMAX_READY), MI8_ERR_ARG,
                "mi8_moe_gather_cast_rows_and_colwise_t: the amax pass is part of this call");
    MI8_REQUIRE(!weights || w_dtype == MI8_BF16 || w_dtype == MI8_F16 || w_dtype == MI8_F32, MI8_ERR_ARG,
                "mi8_moe_gather_cast_rows_and_colwise_t: unknown weight dtype %d", w_dtype);
    return grouped_cast_launch("mi8_moe_gather_cast_rows_and_colwise_t", x, hp_dtype, tokens * top_k, cols, group_sizes,
                               num_groups, fp8_dtype, flags, amax_ws, out_t, ld_t, scale_out, row_amax_ws, out_rows,
                               ld_rows, row_scale_out, stream, indices, top_k, tokens, weights, w_dtype);
}
