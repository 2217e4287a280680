// Ragged grouped fp8 GEMMs for the dropless-MoE expert layer: rows of the activation matrix are split into
// consecutive groups (one per expert, sizes known only on the device), every group multiplies its own weight.
//
//   grouped_gemm  : out[rows_e, :] = A[rows_e, :K] . B_e[:N, :K]^T      (forward and grad_input; ragged M)
//   grouped_wgrad : out[e]         = A_t[:, seg_e] . B_t[:, seg_e]^T     (grad_weight; ragged K, segments padded
//                                                                          to multiples of 128 with zero bytes)
//
// Each workgroup finds its group by walking the (at most a few hundred) group sizes, builds a per-group view of
// the operands and runs the general tile routine on it; workgroups beyond the real number of tiles exit.
#include "mi8_gemm_body.h"

namespace mi8 {
using namespace gemm;
namespace {

constexpr int GBM = 256, GBN = 256;  // 8 waves of 128 x 64: the best general-shape configuration measured
constexpr int GWM = 2, GWN = 4;
constexpr int kGroupedThreads = GWM * GWN * 64;
constexpr int kGroupedLds = 2 * (GBM + GBN) * BK;

struct GroupedArgs {
    const uint8_t* A;  // [T, lda]
    const uint8_t* B;  // group e starts at B + e * b_group_stride, rows N, pitch ldb
    void* C;           // [T, ldc]
    int c_f32;
    int64_t lda, ldb, ldc, b_group_stride, sb_group_stride;
    const int64_t* sizes;
    int E;
    int64_t T;
    int N, K;
    const float* sa;  // [T]
    const float* sb;  // group e: sb + e * sb_group_stride, N values
    int tiles_n;
    int accumulate;   // C += the rounded product
};

template <int CBSZ, int BLGP>
__global__ __launch_bounds__(kGroupedThreads, 1) void grouped_gemm_kernel(GroupedArgs a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int mt = (int)blockIdx.x / a.tiles_n, nt = (int)blockIdx.x % a.tiles_n;
    int64_t row0 = 0;
    int tiles_before = 0, e = 0, m_e = 0;
    bool found = false;
    for (e = 0; e < a.E; ++e) {
        int64_t m = a.sizes[e];
        m = m < 0 ? 0 : m;
        m = (row0 + m > a.T) ? a.T - row0 : m;  // never touch rows past the activation matrix
        const int t = (int)((m + GBM - 1) / GBM);
        if (mt < tiles_before + t) {
            m_e = (int)m;
            found = true;
            break;
        }
        tiles_before += t;
        row0 += m;
    }
    if (!found) return;
    GemmArgs g;
    g.A = a.A + row0 * a.lda;
    g.B = a.B + (int64_t)e * a.b_group_stride;
    g.C = reinterpret_cast<uint8_t*>(a.C) + row0 * a.ldc * (a.c_f32 ? 4 : 2);
    g.c_f32 = a.c_f32;
    g.lda = a.lda;
    g.ldb = a.ldb;
    g.ldc = a.ldc;
    g.M = m_e;
    g.N = a.N;
    g.K = a.K;
    g.sa = a.sa + row0;
    g.sb = a.sb + (int64_t)e * a.sb_group_stride;
    g.sa_vec = 1;
    g.sb_vec = 1;
    g.tiles_m = 0;
    g.tiles_n = a.tiles_n;
    g.accumulate = a.accumulate;
    gemm_tile_body<GBM, GBN, GWM, GWN, CBSZ, BLGP>(g, (mt - tiles_before) * GBM, nt * GBN, lds);
}

struct GroupedWgradArgs {
    const uint8_t* At;  // [N, ld_t]
    const uint8_t* Bt;  // [Kl, ld_t]
    int64_t ld_t;
    const int64_t* sizes;
    int E;
    int64_t T;
    int N, Kl;
    const float* sa;  // [E, N]
    const float* sb;  // [E, Kl]
    void* C;          // [E, N, Kl]
    int c_f32;
    int tiles_n, tiles_k;
};

template <int CBSZ, int BLGP>
__global__ __launch_bounds__(kGroupedThreads, 1) void grouped_wgrad_kernel(GroupedWgradArgs a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int per_group = a.tiles_n * a.tiles_k;
    const int e = (int)blockIdx.x / per_group;
    const int rem = (int)blockIdx.x % per_group;
    const int tn = rem / a.tiles_k, tk = rem % a.tiles_k;
    // segment of group e in the padded token axis: starts at 128 * (tiles of the groups before it)
    int64_t rows_before = 0, tiles_before = 0, m_e = 0;
    for (int i = 0; i <= e; ++i) {
        int64_t m = a.sizes[i];
        m = m < 0 ? 0 : m;
        m = (rows_before + m > a.T) ? a.T - rows_before : m;
        if (i == e) {
            m_e = m;
            break;
        }
        tiles_before += (m + 127) / 128;
        rows_before += m;
    }
    const int64_t seg0 = 128 * tiles_before;
    int64_t seg = 128 * ((m_e + 127) / 128);
    if (seg0 + seg > a.ld_t) seg = 0;
    GemmArgs g;
    g.A = a.At + seg0;
    g.B = a.Bt + seg0;
    g.C = reinterpret_cast<uint8_t*>(a.C) + (int64_t)e * a.N * a.Kl * (a.c_f32 ? 4 : 2);
    g.c_f32 = a.c_f32;
    g.lda = a.ld_t;
    g.ldb = a.ld_t;
    g.ldc = a.Kl;
    g.M = a.N;
    g.N = a.Kl;
    g.K = (int)seg;  // 0 for an empty group: the tile routine then writes zeros
    // an empty group has no scales (nothing was quantised): give the epilogue a finite stand-in
    static __device__ const float kOne = 1.0f;
    g.sa = seg ? a.sa + (int64_t)e * a.N : &kOne;
    g.sb = seg ? a.sb + (int64_t)e * a.Kl : &kOne;
    g.sa_vec = seg ? 1 : 0;
    g.sb_vec = seg ? 1 : 0;
    g.tiles_m = 0;
    g.tiles_n = a.tiles_k;
    g.accumulate = 0;
    gemm_tile_body<GBM, GBN, GWM, GWN, CBSZ, BLGP>(g, tn * GBM, tk * GBN, lds);
}

template <int CBSZ, int BLGP>
int launch_grouped(const GroupedArgs& a, int blocks, hipStream_t st)
{
    auto kern = grouped_gemm_kernel<CBSZ, BLGP>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), kGroupedLds, configured, "mi8_grouped_gemm_fp8"))
        return rc;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGroupedThreads), kGroupedLds, st, a);
    return launch_status("mi8_grouped_gemm_fp8");
}

template <int CBSZ, int BLGP>
int launch_wgrad(const GroupedWgradArgs& a, int blocks, hipStream_t st)
{
    auto kern = grouped_wgrad_kernel<CBSZ, BLGP>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), kGroupedLds, configured, "mi8_grouped_wgrad_fp8"))
        return rc;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGroupedThreads), kGroupedLds, st, a);
    return launch_status("mi8_grouped_wgrad_fp8");
}

bool fp8_code(int v) { return v == MI8_E4M3 || v == MI8_E5M2; }

}  // namespace
}  // namespace mi8

using namespace mi8;

namespace {
int grouped_gemm_entry(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                       int64_t b_group_stride, const int64_t* group_sizes, int32_t num_groups, int64_t T, int64_t N,
                       int64_t K, const float* sa, const float* sb, int64_t sb_group_stride, void* out, int out_dtype,
                       int64_t ldc, bool accumulate, void* stream)
{
    MI8_REQUIRE(a && b && group_sizes && sa && sb && out, MI8_ERR_ARG, "mi8_grouped_gemm_fp8: null pointer");
    MI8_REQUIRE(fp8_code(a_dtype) && fp8_code(b_dtype), MI8_ERR_ARG, "mi8_grouped_gemm_fp8: unknown fp8 dtype");
    MI8_REQUIRE(out_dtype == MI8_BF16 || out_dtype == MI8_F32, MI8_ERR_ARG, "mi8_grouped_gemm_fp8: unknown output dtype");
    MI8_REQUIRE(T > 0 && N > 0 && K > 0 && num_groups > 0, MI8_ERR_ARG, "mi8_grouped_gemm_fp8: empty problem");
    MI8_REQUIRE(K % 16 == 0 && lda % 16 == 0 && ldb % 16 == 0 && lda >= K && ldb >= K && b_group_stride % 16 == 0,
                MI8_ERR_UNSUPPORTED, "mi8_grouped_gemm_fp8: K, lda, ldb and the group stride must be multiples of 16, lda, ldb >= K");
    MI8_REQUIRE(ldc >= N, MI8_ERR_UNSUPPORTED, "mi8_grouped_gemm_fp8: ldc < N");
    MI8_REQUIRE(aligned16(a) && aligned16(b), MI8_ERR_UNSUPPORTED, "mi8_grouped_gemm_fp8: operands must be 16-byte aligned");
    MI8_REQUIRE(N * ldb < ((int64_t)1 << 32) && T < (1 << 30) && N < (1 << 30) && K < (1 << 30), MI8_ERR_UNSUPPORTED,
                "mi8_grouped_gemm_fp8: operand too large");
    const int tiles_n = (int)ceil_div(N, GBN);
    const int64_t m_tiles = ceil_div(T, GBM) + num_groups;  // every group adds at most one partial tile
    MI8_REQUIRE(m_tiles * tiles_n < ((int64_t)1 << 31), MI8_ERR_UNSUPPORTED, "mi8_grouped_gemm_fp8: grid too large");
    GroupedArgs g{(const uint8_t*)a, (const uint8_t*)b, out, out_dtype == MI8_F32 ? 1 : 0, lda, ldb, ldc,
                  b_group_stride, sb_group_stride, group_sizes, num_groups, T, (int)N, (int)K, sa, sb, tiles_n,
                  accumulate ? 1 : 0};
    const int blocks = (int)(m_tiles * tiles_n);
    hipStream_t st = (hipStream_t)stream;
    // full-tile shapes with bf16 output run on the persistent direct-to-LDS kernel (which rewrites the overlap of its
    // shifted last tile column when N is not a multiple of 256: not possible when accumulating)
    if (out_dtype == MI8_BF16 && T >= 256 && N >= 256 && K % 128 == 0 && N % 8 == 0 && ldc % 8 == 0 && aligned16(out) &&
        sb_group_stride % 4 == 0 && aligned16(sb) && lda < (1 << 23) && ldb < (1 << 23) && ldc < (1 << 22) &&
        (!accumulate || N % 256 == 0))
        return launch_m16_grouped((const uint8_t*)a, a_dtype, lda, (const uint8_t*)b, b_dtype, ldb, b_group_stride,
                                   group_sizes, num_groups, T, (int)N, (int)K, sa, sb, sb_group_stride, (uint16_t*)out,
                                   ldc, accumulate, st);
    if (a_dtype == MI8_E4M3)
        return b_dtype == MI8_E4M3 ? launch_grouped<0, 0>(g, blocks, st) : launch_grouped<0, 1>(g, blocks, st);
    return b_dtype == MI8_E4M3 ? launch_grouped<1, 0>(g, blocks, st) : launch_grouped<1, 1>(g, blocks, st);
}
}  // namespace

extern "C" int mi8_grouped_gemm_fp8(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                                    int64_t b_group_stride, const int64_t* group_sizes, int32_t num_groups, int64_t T,
                                    int64_t N, int64_t K, const float* sa, const float* sb, int64_t sb_group_stride,
                                    void* out, int out_dtype, int64_t ldc, void* stream)
{
    return grouped_gemm_entry(a, a_dtype, lda, b, b_dtype, ldb, b_group_stride, group_sizes, num_groups, T, N, K, sa, sb,
                              sb_group_stride, out, out_dtype, ldc, false, stream);
}

extern "C" int mi8_grouped_gemm_fp8_accumulate(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype,
                                               int64_t ldb, int64_t b_group_stride, const int64_t* group_sizes,
                                               int32_t num_groups, int64_t T, int64_t N, int64_t K, const float* sa,
                                               const float* sb, int64_t sb_group_stride, void* out, int out_dtype,
                                               int64_t ldc, void* stream)
{
    return grouped_gemm_entry(a, a_dtype, lda, b, b_dtype, ldb, b_group_stride, group_sizes, num_groups, T, N, K, sa, sb,
                              sb_group_stride, out, out_dtype, ldc, true, stream);
}

extern "C" int mi8_grouped_gemm_fp8_dual_supported(int64_t T, int64_t N, int64_t K1, int64_t K2)
{
    return (T >= 256 && T < (1 << 30) && N >= 256 && N % 8 == 0 && N < (1 << 30) && K1 >= 256 && K2 >= 256 && K1 % 256 == 0 &&
            K2 % 256 == 0 && K1 < (1 << 30) && K2 < (1 << 30))
               ? 1
               : 0;
}

extern "C" int mi8_grouped_gemm_fp8_dual(const void* a1, const void* a2, int a_dtype, int64_t lda, const void* b1,
                                         const void* b2, int b_dtype, int64_t ldb, int64_t b_group_stride,
                                         const int64_t* group_sizes, int32_t num_groups, int64_t T, int64_t N, int64_t K1,
                                         int64_t K2, const float* sa1, const float* sa2, const float* sb1, const float* sb2,
                                         int64_t sb_group_stride, void* out, int64_t ldc, void* stream)
{
    MI8_REQUIRE(a1 && a2 && b1 && b2 && group_sizes && sa1 && sa2 && sb1 && sb2 && out, MI8_ERR_ARG,
                "mi8_grouped_gemm_fp8_dual: null pointer");
    MI8_REQUIRE(fp8_code(a_dtype) && fp8_code(b_dtype), MI8_ERR_ARG, "mi8_grouped_gemm_fp8_dual: unknown fp8 dtype");
    MI8_REQUIRE(num_groups > 0, MI8_ERR_ARG, "mi8_grouped_gemm_fp8_dual: no groups");
    MI8_REQUIRE(mi8_grouped_gemm_fp8_dual_supported(T, N, K1, K2), MI8_ERR_UNSUPPORTED,
                "mi8_grouped_gemm_fp8_dual: needs T, N >= 256, N %% 8 == 0 and K1, K2 multiples of 256 (got T=%lld N=%lld K1=%lld "
                "K2=%lld); use mi8_grouped_gemm_fp8 and mi8_grouped_gemm_fp8_accumulate",
                (long long)T, (long long)N, (long long)K1, (long long)K2);
    const int64_t kmax = K1 > K2 ? K1 : K2;
    MI8_REQUIRE(lda % 16 == 0 && ldb % 16 == 0 && lda >= kmax && ldb >= kmax && b_group_stride % 16 == 0 && lda < (1 << 23) &&
                    ldb < (1 << 23),
                MI8_ERR_UNSUPPORTED, "mi8_grouped_gemm_fp8_dual: lda, ldb and the group stride must be multiples of 16, lda, ldb >= K1, K2 and below 2^23");
    MI8_REQUIRE(ldc >= N && ldc % 8 == 0 && ldc < (1 << 22) && aligned16(out), MI8_ERR_UNSUPPORTED,
                "mi8_grouped_gemm_fp8_dual: the output needs ldc >= N, ldc %% 8 == 0 and 16-byte alignment");
    MI8_REQUIRE(aligned16(a1) && aligned16(a2) && aligned16(b1) && aligned16(b2) && aligned16(sb1) && aligned16(sb2) &&
                    sb_group_stride % 4 == 0,
                MI8_ERR_UNSUPPORTED, "mi8_grouped_gemm_fp8_dual: operands and column scales must be 16-byte aligned");
    MI8_REQUIRE(N * ldb < ((int64_t)1 << 32), MI8_ERR_UNSUPPORTED, "mi8_grouped_gemm_fp8_dual: operand too large");
    const int64_t m_tiles = ceil_div(T, 256) + num_groups;
    MI8_REQUIRE(m_tiles * ceil_div(N, 256) < ((int64_t)1 << 30), MI8_ERR_UNSUPPORTED, "mi8_grouped_gemm_fp8_dual: grid too large");
    return launch_m16_grouped_dual((const uint8_t*)a1, (const uint8_t*)a2, a_dtype, lda, (const uint8_t*)b1, (const uint8_t*)b2,
                                   b_dtype, ldb, b_group_stride, group_sizes, num_groups, T, (int)N, (int)K1, (int)K2, sa1, sa2,
                                   sb1, sb2, sb_group_stride, (uint16_t*)out, ldc, (hipStream_t)stream);
}

extern "C" int mi8_grouped_wgrad_fp8(const void* a_t, int a_dtype, const void* b_t, int b_dtype, int64_t ld_t,
                                     const int64_t* group_sizes, int32_t num_groups, int64_t T, int64_t N, int64_t Kl,
                                     const float* sa, const float* sb, void* out, int out_dtype, void* stream)
{
    MI8_REQUIRE(a_t && b_t && group_sizes && sa && sb && out, MI8_ERR_ARG, "mi8_grouped_wgrad_fp8: null pointer");
    MI8_REQUIRE(fp8_code(a_dtype) && fp8_code(b_dtype), MI8_ERR_ARG, "mi8_grouped_wgrad_fp8: unknown fp8 dtype");
    MI8_REQUIRE(out_dtype == MI8_BF16 || out_dtype == MI8_F32, MI8_ERR_ARG, "mi8_grouped_wgrad_fp8: unknown output dtype");
    MI8_REQUIRE(T > 0 && N > 0 && Kl > 0 && num_groups > 0, MI8_ERR_ARG, "mi8_grouped_wgrad_fp8: empty problem");
    MI8_REQUIRE(ld_t % 16 == 0 && ld_t >= mi8_grouped_padded_rows(T, num_groups), MI8_ERR_UNSUPPORTED,
                "mi8_grouped_wgrad_fp8: ld_t (%lld) must be a multiple of 16 and at least mi8_grouped_padded_rows()",
                (long long)ld_t);
    MI8_REQUIRE(aligned16(a_t) && aligned16(b_t), MI8_ERR_UNSUPPORTED, "mi8_grouped_wgrad_fp8: operands must be 16-byte aligned");
    MI8_REQUIRE(N * ld_t < ((int64_t)1 << 32) && Kl * ld_t < ((int64_t)1 << 32), MI8_ERR_UNSUPPORTED,
                "mi8_grouped_wgrad_fp8: operand larger than 4 GiB");
    const int tiles_n = (int)ceil_div(N, GBM), tiles_k = (int)ceil_div(Kl, GBN);
    GroupedWgradArgs g{(const uint8_t*)a_t, (const uint8_t*)b_t, ld_t, group_sizes, num_groups, T, (int)N, (int)Kl,
                       sa, sb, out, out_dtype == MI8_F32 ? 1 : 0, tiles_n, tiles_k};
    const int blocks = num_groups * tiles_n * tiles_k;
    hipStream_t st = (hipStream_t)stream;
    if (out_dtype == MI8_BF16 && N >= 256 && Kl >= 256 && Kl % 8 == 0 && aligned16(out) && aligned16(sb) &&
        ld_t % 128 == 0 && ld_t < (1 << 23))
        return launch_m16_grouped_wgrad((const uint8_t*)a_t, a_dtype, (const uint8_t*)b_t, b_dtype, ld_t, group_sizes,
                                         num_groups, T, (int)N, (int)Kl, sa, sb, (uint16_t*)out, st);
    if (a_dtype == MI8_E4M3)
        return b_dtype == MI8_E4M3 ? launch_wgrad<0, 0>(g, blocks, st) : launch_wgrad<0, 1>(g, blocks, st);
    return b_dtype == MI8_E4M3 ? launch_wgrad<1, 0>(g, blocks, st) : launch_wgrad<1, 1>(g, blocks, st);
}
