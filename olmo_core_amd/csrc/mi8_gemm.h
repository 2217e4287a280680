// Shared pieces of the fp8 GEMM kernels (argument block, LDS swizzle, tile order).
#pragma once
#include "mi8_common.h"

namespace mi8 {
namespace gemm {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BK = 128;  // bytes of K per LDS stage

struct GemmArgs {
    const uint8_t* A;
    const uint8_t* B;
    void* C;
    int c_f32;
    int64_t lda, ldb, ldc;
    int M, N, K;
    const float* sa;
    const float* sb;
    int sa_vec, sb_vec;
    int tiles_m, tiles_n;
    int accumulate;  // add the rounded product to what C holds (the sum of two grad_input halves) instead of overwriting
};


__device__ __forceinline__ int swz(int r) { return (r ^ (r >> 3)) & 7; }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f)
{
    __bf16 h = (__bf16)f;  // round-to-nearest-even; v_cvt_pk_bf16_f32 on gfx950
    return __builtin_bit_cast(uint16_t, h);
}

// Two floats -> two bf16 (round-to-nearest-even) in one dword, low half first: a single v_cvt_pk_bf16_f32.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    const f32x2_t f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

// bf16(a) + bf16(b) for eight packed values, each sum formed in float32 and rounded once (what an elementwise add of
// two bf16 tensors computes)
__device__ __forceinline__ v4i add_bf16x8(v4i a, v4i b)
{
    v4i r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t x = (uint32_t)a[i], y = (uint32_t)b[i];
        const float lo = bits_to_f32(x << 16) + bits_to_f32(y << 16);
        const float hi = bits_to_f32(x & 0xFFFF0000u) + bits_to_f32(y & 0xFFFF0000u);
        r[i] = (int)pack_bf16x2(lo, hi);
    }
    return r;
}

// Linear tile index -> tile coordinates: tiles are walked in groups of 8 tile-rows (all columns of the group
// before the next group, walked from a group-dependent start column) so that tiles with neighbouring indices
// share A and B panels.
__device__ __forceinline__ void tile_coords(const GemmArgs& g, int t, int& tm, int& tn)
{
    constexpr int GROUP = 8;
    const int span = GROUP * g.tiles_n;
    const int first_m = (t / span) * GROUP;
    const int gsz = (g.tiles_m - first_m < GROUP) ? g.tiles_m - first_m : GROUP;
    const int in = t % span;
    tm = first_m + in % gsz;
    // Every group starts its column sweep somewhere else: groups that run at the same time on different XCDs
    // (one group per XCD when tiles_m = 64) would otherwise request the same B panels from memory in lockstep.
    tn = (in / gsz + (t / span) * ((g.tiles_n + GROUP - 1) / GROUP)) % g.tiles_n;
}

// Workgroup id -> output tile.  Consecutive workgroup ids are spread round-robin over the 8 XCDs, each with
// its own L2; give every XCD a contiguous range of tiles so that the workgroups resident on one XCD share A
// and B panels in its L2.
__device__ __forceinline__ bool tile_of_block(const GemmArgs& g, int& tm, int& tn)
{
    constexpr int XCDS = 8;
    const int total = g.tiles_m * g.tiles_n;
    const int per_xcd = (total + XCDS - 1) / XCDS;
    const int b = (int)blockIdx.x;
    const int t = (b % XCDS) * per_xcd + b / XCDS;
    if (t >= total) return false;
    tile_coords(g, t, tm, tn);
    return true;
}

// persistent direct-to-LDS kernel, four waves of 128 x 128 on 16x16x128 MFMAs (mi8_gemm_m16.hip); requires
// M, N >= 256, K % 128 == 0, N % 8 == 0, ldc % 8 == 0, a 16-byte aligned bf16 output
int launch_m16(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st);  // (honours g.accumulate)
// the same with single scales, also recording the row-segment codes of C (uint16 [N / 64][M], N % 64 == 0)
int launch_m16_codes(GemmArgs& g, uint16_t* codes, int a_dtype, int b_dtype, hipStream_t st);
// the two input projections of a SwiGLU block and h = silu(x1) * x3 in one launch (g: A, B = B1, C = x1, N = H,
// single scales sa, sb = scale of B1); writes 4 * workgroups partial maxima of |h| and their count
// (x_codes: null, or uint16 [H / 64][M] row-segment codes of the larger of x1 and x3, H % 64 == 0)
int launch_m16_swiglu(GemmArgs& g, const uint8_t* b3, const float* sb3, uint16_t* x3, uint16_t* h, uint32_t* h_slots,
                      int* n_slots, uint16_t* x_codes, int a_dtype, int b_dtype, hipStream_t st);
// a few rows of A (M <= kSkinnyMaxM) against all of B, bound by reading B once (mi8_gemm_skinny.hip): any N,
// K % 16 == 0, any mix of single scales and scale vectors, bf16 or fp32 output
constexpr int kSkinnyMaxM = 64;
int launch_skinny(GemmArgs& g, int a_dtype, int b_dtype, hipStream_t st);
// the same kernel over the ragged grouped problems (bf16 output, per-row / per-column scale vectors):
// forward / grad_input (T, N >= 256, K % 128 == 0) and grad_weight (N, Kl >= 256)
int launch_m16_grouped(const uint8_t* a, int a_dtype, int64_t lda, const uint8_t* b, int b_dtype, int64_t ldb,
                       int64_t b_group_stride, const int64_t* sizes, int E, int64_t T, int N, int K, const float* sa,
                       const float* sb, int64_t sb_group_stride, uint16_t* out, int64_t ldc, bool accumulate,
                       hipStream_t st);
// out[rows of e] = A1 . B1_e^T + A2 . B2_e^T in one accumulation (power-of-two scale vectors, applied inside the
// MFMAs); T, N >= 256, K1, K2 multiples of 256
int launch_m16_grouped_dual(const uint8_t* a1, const uint8_t* a2, int a_dtype, int64_t lda, const uint8_t* b1,
                            const uint8_t* b2, int b_dtype, int64_t ldb, int64_t b_group_stride, const int64_t* sizes, int E,
                            int64_t T, int N, int K1, int K2, const float* sa1, const float* sa2, const float* sb1,
                            const float* sb2, int64_t sb_group_stride, uint16_t* out, int64_t ldc, hipStream_t st);
int launch_m16_grouped_wgrad(const uint8_t* a_t, int a_dtype, const uint8_t* b_t, int b_dtype, int64_t ld_t,
                             const int64_t* sizes, int E, int64_t T, int N, int Kl, const float* sa, const float* sb,
                             uint16_t* out, hipStream_t st);

}  // namespace gemm
}  // namespace mi8
