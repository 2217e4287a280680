// Scaled float8 GEMM on CDNA4 matrix cores:  C[M,N] = bf16( (A[M,K] . B[N,K]^T) * (1/sa) * (1/sb) ).
//
// Both operands are K-contiguous ("TN"), which is what v_mfma_f32_32x32x64_f8f6f4 wants: every lane feeds 32
// consecutive K bytes of one row.  A workgroup owns a BM x BN tile of C, walks K in 128-byte steps through a
// double-buffered LDS stage, and each wave accumulates a (BM/WM) x (BN/WN) sub-tile in fp32 registers.
//
// LDS stage layout: [row][128 bytes]; the 16-byte chunk c of row r sits at chunk position c ^ swz(r),
// swz(r) = (r ^ (r >> 3)) & 7, so that the 16-byte fragment reads of 32 different rows spread over all banks
// while the stores (8 lanes per row) stay contiguous.
//
// This file holds that general tile kernel (any M, N; K % 16 == 0; bf16 or fp32 output), its split-K form for
// problems with few output tiles, and the entry points, which pick a kernel by shape: the persistent direct-to-LDS
// kernel of mi8_gemm_m16.hip for large problems, the weight-streaming kernel of mi8_gemm_skinny.hip for a few
// rows of A.
#include "mi8_gemm_body.h"

namespace mi8 {
using namespace gemm;
namespace {

template <int BM, int BN, int WM, int WN, int CBSZ, int BLGP>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm_fp8_kernel(GemmArgs g)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    int tm, tn;
    if (!tile_of_block(g, tm, tn)) return;
    gemm_tile_body<BM, BN, WM, WN, CBSZ, BLGP>(g, tm * BM, tn * BN, lds);
}

// ---- split K ---------------------------------------------------------------------------------------
// A problem with few output tiles and a long K leaves most compute units idle while every busy one pays a
// memory latency per 128-byte K step.  Here blockIdx.y cuts K into slices: every (tile, slice) workgroup runs
// the same tile routine on its slice (operand pointers moved along the rows, which are K-contiguous) and stores
// the raw fp32 sums into its own plane of a workspace; a second kernel adds the planes in a fixed order (the
// result does not depend on scheduling), applies the scales and rounds.

constexpr int kSplitTile = 128;

struct SplitArgs {
    GemmArgs g;          // the problem; C, ldc, scales describe the final output
    float* planes;       // [splits][M][ld_plane] fp32
    int64_t ld_plane;    // round_up(N, 4)
    int steps_per_split; // 128-byte K steps per slice; the last slice may be shorter, none is empty
    int splits;
};

template <int CBSZ, int BLGP>
__global__ __launch_bounds__(256, 1) void gemm_fp8_splitk_kernel(SplitArgs a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    GemmArgs g = a.g;
    int tm, tn;
    if (!tile_of_block(g, tm, tn)) return;
    const int split = (int)blockIdx.y;
    const int k0 = split * a.steps_per_split * BK;
    const int left = g.K - k0;
    g.A += k0;
    g.B += k0;
    g.K = left < a.steps_per_split * BK ? left : a.steps_per_split * BK;
    g.C = a.planes + (int64_t)split * g.M * a.ld_plane;
    g.c_f32 = 1;
    g.ldc = a.ld_plane;
    g.sa = g.sb = nullptr;
    g.sa_vec = g.sb_vec = 0;
    gemm_tile_body<kSplitTile, kSplitTile, 2, 2, CBSZ, BLGP>(g, tm * kSplitTile, tn * kSplitTile, lds);
}

// out[m][n] = round( (sum over planes, in plane order) * (1/sa) * (1/sb) ); four columns per thread
__global__ __launch_bounds__(256) void splitk_reduce_kernel(SplitArgs a)
{
    const GemmArgs& g = a.g;
    const int64_t quads_per_row = a.ld_plane / 4;
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= (int64_t)g.M * quads_per_row) return;
    const int m = (int)(q / quads_per_row);
    const int n = (int)(q % quads_per_row) * 4;
    const int64_t plane = (int64_t)g.M * a.ld_plane;
    const float* p = a.planes + (int64_t)m * a.ld_plane + n;
    float4 s = *reinterpret_cast<const float4*>(p);
    for (int i = 1; i < a.splits; ++i) {
        const float4 t = *reinterpret_cast<const float4*>(p + i * plane);
        s.x += t.x;
        s.y += t.y;
        s.z += t.z;
        s.w += t.w;
    }
    // same scale arithmetic as the tile routine's own epilogue
    const float isa = g.sa_vec ? __builtin_amdgcn_rcpf(g.sa[m]) : 1.0f / g.sa[0];
    const float isb_scalar = g.sb_vec ? 0.0f : 1.0f / g.sb[0];
    const float v[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (n + j >= g.N) break;
        const float isb = g.sb_vec ? __builtin_amdgcn_rcpf(g.sb[n + j]) : isb_scalar;
        const float r = v[j] * isa * isb;
        if (g.c_f32)
            reinterpret_cast<float*>(g.C)[(int64_t)m * g.ldc + n + j] = r;
        else
            reinterpret_cast<uint16_t*>(g.C)[(int64_t)m * g.ldc + n + j] = f32_to_bf16_bits(r);
    }
}

template <int CBSZ, int BLGP>
int launch_splitk_typed(const SplitArgs& a, hipStream_t st)
{
    auto kern = gemm_fp8_splitk_kernel<CBSZ, BLGP>;
    constexpr int lds_bytes = 2 * (kSplitTile + kSplitTile) * BK;
    static std::atomic<uint64_t> configured{0};
    if (int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured, "mi8_gemm_fp8_splitk"))
        return rc;
    const int total = a.g.tiles_m * a.g.tiles_n;
    hipLaunchKernelGGL(kern, dim3(((total + 7) / 8) * 8, a.splits), dim3(256), lds_bytes, st, a);
    const int64_t quads = (int64_t)a.g.M * (a.ld_plane / 4);
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, a);
    return launch_status("mi8_gemm_fp8_splitk");
}

// slices for a problem, 1 = do not split: aim at two workgroups per compute unit, at least four K steps a slice
int suggested_splits(int64_t M, int64_t N, int64_t K)
{
    const int64_t tiles = ((M + kSplitTile - 1) / kSplitTile) * ((N + kSplitTile - 1) / kSplitTile);
    const int64_t steps = (K + BK - 1) / BK;
    if (M <= 16 || tiles > 256 || steps < 8) return 1;  // (up to 16 rows: the few-rows kernel reads B once)
    int64_t s = 512 / tiles;
    if (s > steps / 4) s = steps / 4;
    if (s > 32) s = 32;
    if (s < 2) return 1;
    const int64_t per = (steps + s - 1) / s;
    return (int)((steps + per - 1) / per);  // no empty slice
}

// ---- variants --------------------------------------------------------------------------------------

struct Variant {
    const char* name;
    int bm, bn, threads;
};

constexpr Variant kVariants[] = {
    {"256x256_w2x2", 256, 256, 256},
    {"256x256_w2x4", 256, 256, 512},
    {"128x128_w2x2", 128, 128, 256},
    {"256x128_w2x2", 256, 128, 256},
    {"128x256_w2x2", 128, 256, 256},
    {"256x256_dma_w4x128_m16x128", 256, 256, 256},
    {"rows64x16_k8_m16x128", 64, 16, 512},
};
constexpr int kSmallTile = 2, kM16 = 5, kSkinny = 6;
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template <int BM, int BN, int WM, int WN, int CBSZ, int BLGP>
int launch_one(const GemmArgs& g, hipStream_t st)
{
    auto kern = gemm_fp8_kernel<BM, BN, WM, WN, CBSZ, BLGP>;
    constexpr int lds_bytes = 2 * (BM + BN) * BK;
    static std::atomic<uint64_t> configured{0};
    if (int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured, "mi8_gemm_fp8"))
        return rc;
    const int total = g.tiles_m * g.tiles_n;
    const int blocks = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(WM * WN * 64), lds_bytes, st, g);
    return launch_status("mi8_gemm_fp8");
}

template <int CBSZ, int BLGP>
int launch_variant(int variant, GemmArgs& g, hipStream_t st)
{
    const Variant& v = kVariants[variant];
    g.tiles_m = (g.M + v.bm - 1) / v.bm;
    g.tiles_n = (g.N + v.bn - 1) / v.bn;
    switch (variant) {
        case 0: return launch_one<256, 256, 2, 2, CBSZ, BLGP>(g, st);
        case 1: return launch_one<256, 256, 2, 4, CBSZ, BLGP>(g, st);
        case 2: return launch_one<128, 128, 2, 2, CBSZ, BLGP>(g, st);
        case 3: return launch_one<256, 128, 2, 2, CBSZ, BLGP>(g, st);
        case 4: return launch_one<128, 256, 2, 2, CBSZ, BLGP>(g, st);
    }
    set_error("mi8_gemm_fp8: unknown variant %d", variant);
    return MI8_ERR_ARG;
}

}  // namespace
}  // namespace mi8

using namespace mi8;

extern "C" int mi8_gemm_num_variants(void) { return kNumVariants; }

extern "C" const char* mi8_gemm_variant_name(int variant)
{
    return (variant >= 0 && variant < kNumVariants) ? kVariants[variant].name : nullptr;
}

namespace {
int gemm_fp8_entry(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb, int64_t M, int64_t N,
                   int64_t K, const float* sa, int sa_is_vector, const float* sb, int sb_is_vector, void* out,
                   int out_dtype, int64_t ldc, int variant, bool accumulate, void* stream)
{
    MI8_REQUIRE(a && b && sa && sb && out, MI8_ERR_ARG, "mi8_gemm_fp8: null pointer");
    MI8_REQUIRE((a_dtype == MI8_E4M3 || a_dtype == MI8_E5M2) && (b_dtype == MI8_E4M3 || b_dtype == MI8_E5M2),
                MI8_ERR_ARG, "mi8_gemm_fp8: unknown fp8 dtype");
    MI8_REQUIRE(M > 0 && N > 0 && K > 0, MI8_ERR_ARG, "mi8_gemm_fp8: empty problem %lld x %lld x %lld",
                (long long)M, (long long)N, (long long)K);
    MI8_REQUIRE(variant >= -1 && variant < kNumVariants, MI8_ERR_ARG, "mi8_gemm_fp8: unknown variant %d", variant);
    MI8_REQUIRE(K % 16 == 0 && lda % 16 == 0 && ldb % 16 == 0 && lda >= K && ldb >= K, MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8: K (%lld), lda (%lld), ldb (%lld) must be multiples of 16 with lda, ldb >= K",
                (long long)K, (long long)lda, (long long)ldb);
    MI8_REQUIRE(ldc >= N, MI8_ERR_UNSUPPORTED, "mi8_gemm_fp8: ldc (%lld) < N (%lld)", (long long)ldc, (long long)N);
    MI8_REQUIRE(aligned16(a) && aligned16(b), MI8_ERR_UNSUPPORTED, "mi8_gemm_fp8: operands must be 16-byte aligned");
    MI8_REQUIRE(M * lda < (int64_t)1 << 32 && N * ldb < (int64_t)1 << 32 && M < (1 << 30) && N < (1 << 30) &&
                    K < (1 << 30),
                MI8_ERR_UNSUPPORTED, "mi8_gemm_fp8: operand larger than 4 GiB");
    MI8_REQUIRE(out_dtype == MI8_BF16 || out_dtype == MI8_F32, MI8_ERR_ARG, "mi8_gemm_fp8: unknown output dtype %d",
                out_dtype);
    GemmArgs g{(const uint8_t*)a, (const uint8_t*)b, out, out_dtype == MI8_F32 ? 1 : 0, lda, ldb, ldc, (int)M, (int)N, (int)K,
               sa, sb, sa_is_vector ? 1 : 0, sb_is_vector ? 1 : 0, 0, 0, accumulate ? 1 : 0};
    hipStream_t st = (hipStream_t)stream;
    // (the persistent kernel shifts its last tile row / column back over the previous one when M or N is not a
    // multiple of 256 and rewrites the overlap with identical values: not possible when accumulating)
    // (its output stores address a tile's 256 rows with 32-bit byte offsets: ldc < 2^22)
    const bool dma_ok = (K % 128 == 0) && M >= 256 && N >= 256 && N % 8 == 0 && ldc % 8 == 0 && ldc < (1 << 22) && aligned16(out) &&
                        out_dtype == MI8_BF16 && (!sb_is_vector || aligned16(sb)) &&
                        (sa_is_vector != 0) == (sb_is_vector != 0) && (!accumulate || (M % 256 == 0 && N % 256 == 0));
    // measured on MI355X on the benchmark configurations' shapes: the four-wave layout beats the eight-wave one
    // by 0-14 %, and its 16x16x128 form beats its 32x32x64 form by 3-9 % (random operands, power-limited clocks).
    // Problems with few 256 x 256 tiles leave most compute units idle and pay one memory latency per K step:
    // 128 x 128 tiles put four times the workgroups to work (512 x 11008 x 4096: 42 us against 70 us), and a few
    // rows of A go to the kernel that streams B once.
    if (variant < 0) {
        const int64_t tiles256 = ((M + 255) / 256) * ((N + 255) / 256);
        if (M <= kSkinnyMaxM && !accumulate)
            variant = kSkinny;
        else if (dma_ok)
            variant = tiles256 <= 96 ? kSmallTile : kM16;  // (mi8_gemm_fp8_swiglu_matches_separate mirrors this)
        else
            variant = tiles256 <= 384 ? kSmallTile : 1;
    }
    MI8_REQUIRE(!(accumulate && variant == kSkinny), MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_accumulate: the few-rows variant does not accumulate");
    if (variant == kSkinny) return launch_skinny(g, a_dtype, b_dtype, st);
    if (variant == kM16) {
        MI8_REQUIRE(dma_ok, MI8_ERR_UNSUPPORTED,
                    "mi8_gemm_fp8: the direct-to-LDS variant needs M, N >= 256, K %% 128 == 0, N %% 8 == 0, ldc %% 8 == 0, "
                    "scales that are both single values or both vectors, and a 16-byte aligned bf16 output (M=%lld N=%lld K=%lld ldc=%lld)",
                    (long long)M, (long long)N, (long long)K, (long long)ldc);
        return launch_m16(g, a_dtype, b_dtype, st);
    }
    if (a_dtype == MI8_E4M3)
        return b_dtype == MI8_E4M3 ? launch_variant<0, 0>(variant, g, st) : launch_variant<0, 1>(variant, g, st);
    return b_dtype == MI8_E4M3 ? launch_variant<1, 0>(variant, g, st) : launch_variant<1, 1>(variant, g, st);
}
}  // namespace

extern "C" int mi8_gemm_fp8(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                            int64_t M, int64_t N, int64_t K, const float* sa, int sa_is_vector, const float* sb,
                            int sb_is_vector, void* out, int out_dtype, int64_t ldc, int variant, void* stream)
{
    return gemm_fp8_entry(a, a_dtype, lda, b, b_dtype, ldb, M, N, K, sa, sa_is_vector, sb, sb_is_vector, out, out_dtype,
                          ldc, variant, false, stream);
}

extern "C" int mi8_gemm_fp8_accumulate(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                                       int64_t M, int64_t N, int64_t K, const float* sa, int sa_is_vector,
                                       const float* sb, int sb_is_vector, void* out, int out_dtype, int64_t ldc,
                                       void* stream)
{
    return gemm_fp8_entry(a, a_dtype, lda, b, b_dtype, ldb, M, N, K, sa, sa_is_vector, sb, sb_is_vector, out, out_dtype,
                          ldc, -1, true, stream);
}

// 1 if mi8_gemm_fp8_swiglu takes the shape AND mi8_gemm_fp8 would run both projections on the same persistent
// kernel (then the fused launch reproduces the three-call route bit for bit; other tile kernels sum in another order)
extern "C" int mi8_gemm_fp8_swiglu_matches_separate(int64_t M, int64_t H, int64_t K)
{
    if (M < 256 || H < 256 || K <= 0 || K % 128 || H % 8) return 0;
    const int64_t tiles256 = ((M + 255) / 256) * ((H + 255) / 256);
    return tiles256 > 96 ? 1 : 0;
}

extern "C" int mi8_gemm_fp8_swiglu(const void* a, int a_dtype, int64_t lda, const void* b1, const void* b3, int b_dtype,
                                   int64_t ldb, int64_t M, int64_t H, int64_t K, const float* sa, const float* sb1,
                                   const float* sb3, void* x1, void* x3, void* h, int64_t ldc, uint32_t* slots_h,
                                   int32_t* n_slots_used, uint16_t* x_codes, void* stream)
{
    MI8_REQUIRE(a && b1 && b3 && sa && sb1 && sb3 && x1 && x3 && h && slots_h && n_slots_used, MI8_ERR_ARG,
                "mi8_gemm_fp8_swiglu: null pointer");
    MI8_REQUIRE((a_dtype == MI8_E4M3 || a_dtype == MI8_E5M2) && (b_dtype == MI8_E4M3 || b_dtype == MI8_E5M2),
                MI8_ERR_ARG, "mi8_gemm_fp8_swiglu: unknown fp8 dtype");
    MI8_REQUIRE(M >= 256 && H >= 128 && K > 0 && K % 128 == 0 && H % 8 == 0, MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_swiglu: needs M >= 256, H >= 128, H %% 8 == 0, K %% 128 == 0 (got %lld x %lld x %lld); use "
                "mi8_gemm_fp8 twice and mi8_swiglu_fwd",
                (long long)M, (long long)H, (long long)K);
    MI8_REQUIRE(lda % 16 == 0 && ldb % 16 == 0 && lda >= K && ldb >= K && ldc >= H && ldc % 8 == 0, MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_swiglu: lda, ldb must be multiples of 16 and >= K, ldc a multiple of 8 and >= H");
    MI8_REQUIRE(aligned16(a) && aligned16(b1) && aligned16(b3) && aligned16(x1) && aligned16(x3) && aligned16(h),
                MI8_ERR_UNSUPPORTED, "mi8_gemm_fp8_swiglu: operands and outputs must be 16-byte aligned");
    MI8_REQUIRE(M * lda < (int64_t)1 << 32 && H * ldb < (int64_t)1 << 32 && M < (1 << 30) && H < (1 << 30) &&
                    K < (1 << 30),
                MI8_ERR_UNSUPPORTED, "mi8_gemm_fp8_swiglu: operand larger than 4 GiB");
    MI8_REQUIRE(!x_codes || H % 64 == 0, MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_swiglu: row-segment codes need H (%lld) to be a multiple of 64", (long long)H);
    GemmArgs g{(const uint8_t*)a, (const uint8_t*)b1, x1, 0, lda, ldb, ldc, (int)M, (int)H, (int)K, sa, sb1, 0, 0, 0, 0, 0};
    int used = 0;
    const int rc = launch_m16_swiglu(g, (const uint8_t*)b3, sb3, (uint16_t*)x3, (uint16_t*)h, slots_h, &used, x_codes,
                                     a_dtype, b_dtype, (hipStream_t)stream);
    *n_slots_used = used;
    return rc;
}

// 1 if mi8_gemm_fp8_codes takes the shape: the shapes mi8_gemm_fp8 runs on the persistent tile kernel (so that the
// output has the bits of the plain call) whose row segments line up with the output tiles
extern "C" int mi8_gemm_fp8_codes_supported(int64_t M, int64_t N, int64_t K)
{
    if (M < 256 || N < 256 || K <= 0 || K % 128 || N % 64) return 0;
    const int64_t tiles256 = ((M + 255) / 256) * ((N + 255) / 256);
    return tiles256 > 96 ? 1 : 0;
}

extern "C" int mi8_gemm_fp8_codes(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb, int64_t M,
                                  int64_t N, int64_t K, const float* sa, const float* sb, void* out, int64_t ldc,
                                  uint16_t* codes, void* stream)
{
    MI8_REQUIRE(a && b && sa && sb && out && codes, MI8_ERR_ARG, "mi8_gemm_fp8_codes: null pointer");
    MI8_REQUIRE((a_dtype == MI8_E4M3 || a_dtype == MI8_E5M2) && (b_dtype == MI8_E4M3 || b_dtype == MI8_E5M2),
                MI8_ERR_ARG, "mi8_gemm_fp8_codes: unknown fp8 dtype");
    MI8_REQUIRE(mi8_gemm_fp8_codes_supported(M, N, K), MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_codes: needs N %% 64 == 0, K %% 128 == 0 and more than 96 tiles of 256 x 256 (got %lld x %lld x "
                "%lld); use mi8_gemm_fp8 and mi8_rowseg_max_codes",
                (long long)M, (long long)N, (long long)K);
    MI8_REQUIRE(lda % 16 == 0 && ldb % 16 == 0 && lda >= K && ldb >= K && ldc >= N && ldc % 8 == 0, MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_codes: lda, ldb must be multiples of 16 and >= K, ldc a multiple of 8 and >= N");
    MI8_REQUIRE(aligned16(a) && aligned16(b) && aligned16(out), MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_codes: operands and output must be 16-byte aligned");
    MI8_REQUIRE(M * lda < (int64_t)1 << 32 && N * ldb < (int64_t)1 << 32 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30),
                MI8_ERR_UNSUPPORTED, "mi8_gemm_fp8_codes: operand larger than 4 GiB");
    GemmArgs g{(const uint8_t*)a, (const uint8_t*)b, out, 0, lda, ldb, ldc, (int)M, (int)N, (int)K, sa, sb, 0, 0, 0, 0, 0};
    return launch_m16_codes(g, codes, a_dtype, b_dtype, (hipStream_t)stream);
}

extern "C" int mi8_gemm_splitk_suggest(int64_t M, int64_t N, int64_t K)
{
    if (M <= 0 || N <= 0 || K <= 0) return 1;
    return suggested_splits(M, N, K);
}

extern "C" int64_t mi8_gemm_splitk_workspace_bytes(int64_t M, int64_t N, int splits)
{
    if (M <= 0 || N <= 0 || splits <= 0) return 0;
    return (int64_t)splits * M * ((N + 3) / 4 * 4) * (int64_t)sizeof(float);
}

extern "C" int mi8_gemm_fp8_splitk(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                                   int64_t M, int64_t N, int64_t K, const float* sa, int sa_is_vector,
                                   const float* sb, int sb_is_vector, void* out, int out_dtype, int64_t ldc,
                                   int splits, void* workspace, int64_t workspace_bytes, void* stream)
{
    MI8_REQUIRE(a && b && sa && sb && out && workspace, MI8_ERR_ARG, "mi8_gemm_fp8_splitk: null pointer");
    MI8_REQUIRE((a_dtype == MI8_E4M3 || a_dtype == MI8_E5M2) && (b_dtype == MI8_E4M3 || b_dtype == MI8_E5M2),
                MI8_ERR_ARG, "mi8_gemm_fp8_splitk: unknown fp8 dtype");
    MI8_REQUIRE(M > 0 && N > 0 && K > 0, MI8_ERR_ARG, "mi8_gemm_fp8_splitk: empty problem %lld x %lld x %lld",
                (long long)M, (long long)N, (long long)K);
    MI8_REQUIRE(K % 16 == 0 && lda % 16 == 0 && ldb % 16 == 0 && lda >= K && ldb >= K, MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_splitk: K (%lld), lda (%lld), ldb (%lld) must be multiples of 16 with lda, ldb >= K",
                (long long)K, (long long)lda, (long long)ldb);
    MI8_REQUIRE(ldc >= N, MI8_ERR_UNSUPPORTED, "mi8_gemm_fp8_splitk: ldc (%lld) < N (%lld)", (long long)ldc,
                (long long)N);
    MI8_REQUIRE(aligned16(a) && aligned16(b) && aligned16(workspace), MI8_ERR_UNSUPPORTED,
                "mi8_gemm_fp8_splitk: operands and workspace must be 16-byte aligned");
    MI8_REQUIRE(M * lda < (int64_t)1 << 32 && N * ldb < (int64_t)1 << 32 && M < (1 << 30) && N < (1 << 30) &&
                    K < (1 << 30),
                MI8_ERR_UNSUPPORTED, "mi8_gemm_fp8_splitk: operand larger than 4 GiB");
    MI8_REQUIRE(out_dtype == MI8_BF16 || out_dtype == MI8_F32, MI8_ERR_ARG,
                "mi8_gemm_fp8_splitk: unknown output dtype %d", out_dtype);
    const int64_t steps = (K + BK - 1) / BK;
    MI8_REQUIRE(splits >= 1 && splits <= 64 && splits <= steps, MI8_ERR_ARG,
                "mi8_gemm_fp8_splitk: splits (%d) must be in 1..min(64, K steps = %lld)", splits, (long long)steps);
    const int64_t per = (steps + splits - 1) / splits;
    const int used = (int)((steps + per - 1) / per);  // slices that are not empty
    MI8_REQUIRE(workspace_bytes >= mi8_gemm_splitk_workspace_bytes(M, N, used), MI8_ERR_ARG,
                "mi8_gemm_fp8_splitk: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
                (long long)mi8_gemm_splitk_workspace_bytes(M, N, used));
    SplitArgs s{};
    s.g = GemmArgs{(const uint8_t*)a, (const uint8_t*)b, out, out_dtype == MI8_F32 ? 1 : 0, lda, ldb, ldc, (int)M,
                   (int)N, (int)K, sa, sb, sa_is_vector ? 1 : 0, sb_is_vector ? 1 : 0,
                   (int)((M + kSplitTile - 1) / kSplitTile), (int)((N + kSplitTile - 1) / kSplitTile)};
    s.planes = (float*)workspace;
    s.ld_plane = (N + 3) / 4 * 4;
    s.steps_per_split = (int)per;
    s.splits = used;
    hipStream_t st = (hipStream_t)stream;
    if (a_dtype == MI8_E4M3)
        return b_dtype == MI8_E4M3 ? launch_splitk_typed<0, 0>(s, st) : launch_splitk_typed<0, 1>(s, st);
    return b_dtype == MI8_E4M3 ? launch_splitk_typed<1, 0>(s, st) : launch_splitk_typed<1, 1>(s, st);
}
