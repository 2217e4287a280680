// Scaled float8 GEMM on CDNA4 matrix cores:  C[M,N] = bf16( (A[M,K] . B[N,K]^T) * (1/sa) * (1/sb) ).
//
// Both operands are K-contiguous ("TN"), which is what v_mfma_f32_32x32x64_f8f6f4 wants: every lane feeds 32
// consecutive K bytes of one row.  A workgroup owns a BM x BN tile of C, walks K in 128-byte steps through a
// double-buffered LDS stage, and each wave accumulates a (BM/WM) x (BN/WN) sub-tile in fp32 registers.
//
// LDS stage layout: [row][128 bytes]; the 16-byte chunk c of row r sits at chunk position c ^ swz(r),
// swz(r) = (r ^ (r >> 3)) & 7, so that the 16-byte fragment reads of 32 different rows spread over all banks
// while the stores (8 lanes per row) stay contiguous.
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
    {"256x256_dma_w4_k64x4", 256, 256, 256},
    {"256x256_dma_w8_k128x2", 256, 256, 512},
    {"256x256_dma_w4x128_k128x2", 256, 256, 256},
    {"256x256_dma_w4x128_m16x128", 256, 256, 256},
};
constexpr int kDma = 5, kDma8 = 6, kDma4 = 7, kM16 = 8;
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template <int BM, int BN, int WM, int WN, int CBSZ, int BLGP>
int launch_one(const GemmArgs& g, hipStream_t st)
{
    auto kern = gemm_fp8_kernel<BM, BN, WM, WN, CBSZ, BLGP>;
    constexpr int lds_bytes = 2 * (BM + BN) * BK;
    static bool configured = false;  // the attribute is per function; setting it twice is harmless
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) {
            set_error("mi8_gemm_fp8: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
            return MI8_ERR_LAUNCH;
        }
        configured = true;
    }
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

extern "C" int mi8_gemm_fp8(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                            int64_t M, int64_t N, int64_t K, const float* sa, int sa_is_vector, const float* sb,
                            int sb_is_vector, void* out, int out_dtype, int64_t ldc, int variant, void* stream)
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
               sa, sb, sa_is_vector ? 1 : 0, sb_is_vector ? 1 : 0, 0, 0};
    hipStream_t st = (hipStream_t)stream;
    const bool dma_ok = (K % 64 == 0) && M >= 256 && N >= 256 && N % 8 == 0 && ldc % 8 == 0 && aligned16(out) &&
                        out_dtype == MI8_BF16 && (!sb_is_vector || aligned16(sb)) &&
                        (sa_is_vector != 0) == (sb_is_vector != 0);
    // measured on MI355X on the benchmark configurations' shapes: the four-wave layout beats the eight-wave one
    // by 0-14 %, and its 16x16x128 form beats its 32x32x64 form by 3-9 % (random operands, power-limited clocks)
    if (variant < 0) variant = dma_ok ? (K % 128 == 0 ? kM16 : kDma) : 1;
    if (variant == kDma8 && dma_ok && K % 128 == 0) return launch_dma8(g, a_dtype, b_dtype, st);
    if (variant == kDma4 && dma_ok && K % 128 == 0) return launch_dma4(g, a_dtype, b_dtype, st);
    if (variant == kM16 && dma_ok && K % 128 == 0) return launch_m16(g, a_dtype, b_dtype, st);
    if (variant == kDma || variant == kDma8 || variant == kDma4 || variant == kM16) {
        MI8_REQUIRE(dma_ok && variant == kDma, MI8_ERR_UNSUPPORTED,
                    "mi8_gemm_fp8: the direct-to-LDS variant needs M, N >= 256, K %% 64 == 0 (8 waves: 128), N %% 8 == 0, ldc %% 8 == 0, "
                    "scales that are both single values or both vectors, and a 16-byte aligned bf16 output (M=%lld N=%lld K=%lld ldc=%lld)",
                    (long long)M, (long long)N, (long long)K, (long long)ldc);
        return launch_dma(g, a_dtype, b_dtype, st);
    }
    if (a_dtype == MI8_E4M3)
        return b_dtype == MI8_E4M3 ? launch_variant<0, 0>(variant, g, st) : launch_variant<0, 1>(variant, g, st);
    return b_dtype == MI8_E4M3 ? launch_variant<1, 0>(variant, g, st) : launch_variant<1, 1>(variant, g, st);
}
