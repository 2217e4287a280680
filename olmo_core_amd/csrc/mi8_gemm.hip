// Scaled float8 GEMM on CDNA4 matrix cores:  C[M,N] = bf16( (A[M,K] . B[N,K]^T) * (1/sa) * (1/sb) ).
//
// Both operands are K-contiguous ("TN"), which is what v_mfma_f32_32x32x64_f8f6f4 wants: every lane feeds 32
// consecutive K bytes of one row.  A workgroup owns a BM x BN tile of C, walks K in 128-byte steps through a
// double-buffered LDS stage, and each wave accumulates a (BM/WM) x (BN/WN) sub-tile in fp32 registers.
//
// LDS stage layout: [row][128 bytes]; the 16-byte chunk c of row r sits at chunk position c ^ swz(r),
// swz(r) = (r ^ (r >> 3)) & 7, so that the 16-byte fragment reads of 32 different rows spread over all banks
// while the stores (8 lanes per row) stay contiguous.
#include "mi8_gemm.h"

namespace mi8 {
using namespace gemm;
namespace {

template <int BM, int BN, int WM, int WN, int CBSZ, int BLGP>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm_fp8_kernel(GemmArgs g)
{
    constexpr int NT = WM * WN * 64;
    constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
    constexpr int TM = WTM / 32, TN = WTN / 32;  // 32x32 MFMA tiles per wave
    constexpr int ROWS_PER_PASS = NT / 8;        // 8 lanes x 16 bytes cover one 128-byte row
    constexpr int PA = BM / ROWS_PER_PASS, PB = BN / ROWS_PER_PASS;
    constexpr int STAGE = (BM + BN) * BK;
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile/threads mismatch");

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    int tm, tn;
    if (!tile_of_block(g, tm, tn)) return;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, half = lane >> 5;

    // ---- global -> register staging: this lane's rows and 16-byte chunk --------------------------
    const int ld_row = tid >> 3, ld_chunk = tid & 7;
    uint32_t a_off[PA], b_off[PB];
#pragma unroll
    for (int p = 0; p < PA; ++p) {
        int r = m0 + p * ROWS_PER_PASS + ld_row;
        r = r < g.M ? r : g.M - 1;  // rows past the edge re-read the last row; never stored
        a_off[p] = (uint32_t)((int64_t)r * g.lda + ld_chunk * 16);
    }
#pragma unroll
    for (int p = 0; p < PB; ++p) {
        int r = n0 + p * ROWS_PER_PASS + ld_row;
        r = r < g.N ? r : g.N - 1;
        b_off[p] = (uint32_t)((int64_t)r * g.ldb + ld_chunk * 16);
    }
    // LDS store position of this lane's chunk inside a stage (same for every pass up to the row offset)
    uint32_t st_off[(PA > PB ? PA : PB)];
#pragma unroll
    for (int p = 0; p < (PA > PB ? PA : PB); ++p) {
        const int r = p * ROWS_PER_PASS + ld_row;
        st_off[p] = (uint32_t)(r * BK + ((ld_chunk ^ swz(r)) << 4));
    }

    uint4 ra[PA], rb[PB];
    auto load_tile = [&](int kt) {
        const int k = kt * BK + ld_chunk * 16;
        const bool ok = k < g.K;
        const uint8_t* ap = g.A + (int64_t)kt * BK;
        const uint8_t* bp = g.B + (int64_t)kt * BK;
#pragma unroll
        for (int p = 0; p < PA; ++p)
            ra[p] = ok ? *reinterpret_cast<const uint4*>(ap + a_off[p]) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int p = 0; p < PB; ++p)
            rb[p] = ok ? *reinterpret_cast<const uint4*>(bp + b_off[p]) : make_uint4(0, 0, 0, 0);
    };
    auto store_tile = [&](int stage) {
        uint8_t* sa_ = lds + stage * STAGE;
        uint8_t* sb_ = sa_ + BM * BK;
#pragma unroll
        for (int p = 0; p < PA; ++p) *reinterpret_cast<uint4*>(sa_ + st_off[p]) = ra[p];
#pragma unroll
        for (int p = 0; p < PB; ++p) *reinterpret_cast<uint4*>(sb_ + st_off[p]) = rb[p];
    };

    // ---- fragment read offsets (row part; the chunk part depends on the k sub-step) --------------
    // lane l feeds row (l % 32) of a 32-row tile with K bytes [32*half, 32*half+32) of the 64-byte sub-step
    uint32_t fa_row[TM], fb_row[TN];
    int fa_swz[TM], fb_swz[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int r = wm * WTM + i * 32 + l32;
        fa_row[i] = (uint32_t)(r * BK);
        fa_swz[i] = swz(r);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int r = wn * WTN + j * 32 + l32;
        fb_row[j] = (uint32_t)(BM * BK + r * BK);
        fb_swz[j] = swz(r);
    }

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const int nk = (g.K + BK - 1) / BK;
    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) load_tile(kt + 1);
        const uint8_t* st = lds + cur * STAGE;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int c0 = 4 * kk + 2 * half;
            v8i fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const v4i lo = *reinterpret_cast<const v4i*>(st + fa_row[i] + (((c0) ^ fa_swz[i]) << 4));
                const v4i hi = *reinterpret_cast<const v4i*>(st + fa_row[i] + (((c0 + 1) ^ fa_swz[i]) << 4));
                fa[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const v4i lo = *reinterpret_cast<const v4i*>(st + fb_row[j] + (((c0) ^ fb_swz[j]) << 4));
                const v4i hi = *reinterpret_cast<const v4i*>(st + fb_row[j] + (((c0 + 1) ^ fb_swz[j]) << 4));
                fb[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], CBSZ, BLGP,
                                                                                 0, 0, 0, 0);
        }
        if (kt + 1 < nk) store_tile(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue: scale, round to bf16, store ------------------------------------------------------
    // accumulator element e of lane l is C[row = 8*(e/4) + 4*(l/32) + e%4][col = l%32] of its 32x32 tile
    const float isb_scalar = g.sb_vec ? 0.0f : 1.0f / g.sb[0];
    const float isa_scalar = g.sa_vec ? 0.0f : 1.0f / g.sa[0];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn * WTN + j * 32 + l32;
        const bool col_ok = col < g.N;
        const float isb = g.sb_vec ? (col_ok ? 1.0f / g.sb[col] : 0.0f) : isb_scalar;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + wm * WTM + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                if (col_ok && row < g.M) {
                    const float isa = g.sa_vec ? 1.0f / g.sa[row] : isa_scalar;
                    const float v = acc[i][j][e] * isa * isb;
                    if (g.c_f32)
                        reinterpret_cast<float*>(g.C)[(int64_t)row * g.ldc + col] = v;
                    else
                        reinterpret_cast<uint16_t*>(g.C)[(int64_t)row * g.ldc + col] = f32_to_bf16_bits(v);
                }
            }
        }
    }
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
};
constexpr int kDma = 5, kDma8 = 6;
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
                        out_dtype == MI8_BF16;
    if (variant < 0) variant = dma_ok ? (K % 128 == 0 ? kDma8 : kDma) : 1;
    if (variant == kDma8 && dma_ok && K % 128 == 0) return launch_dma8(g, a_dtype, b_dtype, st);
    if (variant == kDma || variant == kDma8) {
        MI8_REQUIRE(dma_ok && variant == kDma, MI8_ERR_UNSUPPORTED,
                    "mi8_gemm_fp8: the direct-to-LDS variant needs M, N >= 256, K %% 64 == 0 (8 waves: 128), N %% 8 == 0, ldc %% 8 == 0 "
                    "and a 16-byte aligned bf16 output (M=%lld N=%lld K=%lld ldc=%lld)",
                    (long long)M, (long long)N, (long long)K, (long long)ldc);
        return launch_dma(g, a_dtype, b_dtype, st);
    }
    if (a_dtype == MI8_E4M3)
        return b_dtype == MI8_E4M3 ? launch_variant<0, 0>(variant, g, st) : launch_variant<0, 1>(variant, g, st);
    return b_dtype == MI8_E4M3 ? launch_variant<1, 0>(variant, g, st) : launch_variant<1, 1>(variant, g, st);
}
