// Token permutation for mixture-of-experts layers: the row copies that bracket the expert GEMMs.
//
//   gather          out[i]       = x[indices[i] / top_k] * w[indices[i]]            (rows sorted by expert)
//   scatter         out[t]       = sum_j round(x[inv[t*top_k + j]] * w[t*top_k + j]) (back to token order)
//   scatter_wgrad   out[indices[i]] = dot(x[i], grad[indices[i] / top_k])            (gradient of the weights)
//
// and their capacity-limited ("binned") forms, where expert e owns `capacity` rows and keeps at most that many
// of its tokens.  All of it is HBM-bound row traffic: one wave per row, 16-byte accesses, products in fp32 with
// one rounding to the element type.  The scatter never materialises the [tokens, top_k, hidden] intermediate of
// a copy-then-sum formulation: a small kernel inverts the permutation (inv[indices[i]] = i) and every output row
// is then reduced in registers, term by term in slot order.
//
// An index outside [0, tokens * top_k) is skipped (treated as a dropped token) rather than followed.
#include "mi8_common.h"

namespace mi8 {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / 64;
constexpr int64_t kMaxBlocks = 256 * 8;

// ---- element types --------------------------------------------------------------------------------------
template <int DT>
struct El;
template <>
struct El<MI8_BF16> {
    using T = uint16_t;
    __device__ static __forceinline__ float to_f32(T v) { return bits_to_f32((uint32_t)v << 16); }
    __device__ static __forceinline__ T from_f32(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
};
template <>
struct El<MI8_F16> {
    using T = uint16_t;
    __device__ static __forceinline__ float to_f32(T v) { return (float)__builtin_bit_cast(_Float16, v); }
    __device__ static __forceinline__ T from_f32(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
};
template <>
struct El<MI8_F32> {
    using T = uint32_t;
    __device__ static __forceinline__ float to_f32(T v) { return bits_to_f32(v); }
    __device__ static __forceinline__ T from_f32(float f) { return f32_to_bits(f); }
};
template <>
struct El<MI8_RAW8> {  // opaque bytes (fp8 rows): copied, never scaled
    using T = uint8_t;
    __device__ static __forceinline__ float to_f32(T v) { return (float)v; }
    __device__ static __forceinline__ T from_f32(float f) { return (T)f; }
};

__device__ __forceinline__ float load_weight(const void* w, int w_dtype, int64_t i)
{
    if (w_dtype == MI8_F32) return reinterpret_cast<const float*>(w)[i];
    const uint16_t v = reinterpret_cast<const uint16_t*>(w)[i];
    return w_dtype == MI8_BF16 ? El<MI8_BF16>::to_f32(v) : El<MI8_F16>::to_f32(v);
}

// A 16-byte chunk as N elements of type T
template <typename T>
union Chunk {
    uint4 raw;
    T e[16 / sizeof(T)];
};

// ---- one row: dst = round(src * w) (src == nullptr: zeros).  `vec`: rows are 16-byte aligned multiples of 16.
template <int DT, bool SCALE>
__device__ __forceinline__ void copy_row(const void* src, void* dst, int64_t hidden, float w, bool vec, int lane)
{
    using T = typename El<DT>::T;
    constexpr int N = 16 / sizeof(T);
    if (vec) {
        const int64_t chunks = hidden / N;
        const uint4* s = reinterpret_cast<const uint4*>(src);
        uint4* d = reinterpret_cast<uint4*>(dst);
        for (int64_t c = lane; c < chunks; c += 64 * 4) {
            Chunk<T> v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                v[u].raw = (src && c + 64 * u < chunks) ? s[c + 64 * u] : make_uint4(0, 0, 0, 0);
            if (SCALE && src) {
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int k = 0; k < N; ++k) v[u].e[k] = El<DT>::from_f32(El<DT>::to_f32(v[u].e[k]) * w);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (c + 64 * u < chunks) d[c + 64 * u] = v[u].raw;
        }
    } else {
        const T* s = reinterpret_cast<const T*>(src);
        T* d = reinterpret_cast<T*>(dst);
        for (int64_t c = lane; c < hidden; c += 64) {
            T v = src ? s[c] : (T)0;
            if (SCALE && src) v = El<DT>::from_f32(El<DT>::to_f32(v) * w);
            d[c] = v;
        }
    }
}

struct PermuteArgs {
    const void* x;
    void* out;
    const int32_t* indices;  // [n]
    const void* weights;     // [n] or null
    int w_dtype;
    const int32_t* bins;     // binned forms: inclusive prefix sums of the tokens per expert, [experts]
    int32_t* inverse;        // scatter: [n]
    const void* grad;        // scatter_wgrad: [tokens, hidden]
    int64_t n;               // tokens * top_k
    int64_t hidden;
    int32_t top_k, experts, capacity;
    bool vec;
};

// Source slot of row r of the expert-sorted side: dropless r -> r; binned (e, j) -> bins[e-1] + j, or -1 when
// expert e has fewer than j + 1 tokens.  Returns the token-slot index (indices[...]) or -1.
template <bool BINNED>
__device__ __forceinline__ int64_t slot_of_row(const PermuteArgs& a, int64_t r)
{
    int64_t pos = r;
    if (BINNED) {
        const int e = (int)(r / a.capacity), j = (int)(r % a.capacity);
        const int start = e ? a.bins[e - 1] : 0;
        if (j >= a.bins[e] - start) return -1;
        pos = start + j;
    }
    if (pos >= a.n) return -1;
    const int64_t idx = a.indices[pos];
    return (idx < 0 || idx >= a.n) ? -1 : idx;
}

template <int DT, bool SCALE, bool BINNED>
__global__ __launch_bounds__(kThreads) void gather_kernel(PermuteArgs a, int64_t rows)
{
    const int lane = threadIdx.x & 63;
    using T = typename El<DT>::T;
    for (int64_t r = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6); r < rows;
         r += (int64_t)gridDim.x * kWavesPerBlock) {
        const int64_t idx = slot_of_row<BINNED>(a, r);
        const T* src = idx < 0 ? nullptr : reinterpret_cast<const T*>(a.x) + (idx / a.top_k) * a.hidden;
        const float w = (SCALE && idx >= 0) ? load_weight(a.weights, a.w_dtype, idx) : 1.0f;
        copy_row<DT, SCALE>(src, reinterpret_cast<T*>(a.out) + r * a.hidden, a.hidden, w, a.vec, lane);
    }
}

template <typename T>
__global__ void fill_kernel(T* p, int64_t n, T v)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

template <bool BINNED>
__global__ void inverse_kernel(PermuteArgs a, int64_t rows)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const int64_t idx = slot_of_row<BINNED>(a, r);
    if (idx >= 0) a.inverse[idx] = (int32_t)r;
}

// out[t] = sum over the token's top_k slots of round(x[inverse[slot]] * w[slot]); slots nobody filled add zero
template <int DT, bool SCALE>
__global__ __launch_bounds__(kThreads) void scatter_reduce_kernel(PermuteArgs a, int64_t tokens)
{
    using T = typename El<DT>::T;
    constexpr int N = 16 / sizeof(T);
    const int lane = threadIdx.x & 63;
    const T* x = reinterpret_cast<const T*>(a.x);
    const int k = a.top_k;
    for (int64_t t = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6); t < tokens;
         t += (int64_t)gridDim.x * kWavesPerBlock) {
    T* out = reinterpret_cast<T*>(a.out) + t * a.hidden;
    if (a.vec) {
        const int64_t chunks = a.hidden / N;
        // The token's rows and weights are fetched once, slot j by lane j, and handed round as wave-uniform values (top_k
        // up to 64; beyond, every term reads its own).  A lane then has four chunks of two rows in flight at a time: a
        // chain of one index load and one row load per term left the memory system idle most of the time.
        const bool held = k <= 64;
        int32_t my_r = -1;
        float my_w = 1.0f;
        if (held && lane < k) {
            my_r = a.inverse[t * k + lane];
            if (SCALE && my_r >= 0) my_w = load_weight(a.weights, a.w_dtype, t * k + lane);
        }
        auto term = [&](int j, int32_t& r, float& w) __attribute__((always_inline)) {
            if (held) {
                r = __builtin_amdgcn_readlane(my_r, j);
                w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_w), j));
            } else {
                r = a.inverse[t * k + j];
                w = (SCALE && r >= 0) ? load_weight(a.weights, a.w_dtype, t * k + j) : 1.0f;
            }
        };
        constexpr int U = 4;
        for (int64_t c0 = lane; c0 < chunks; c0 += 64 * U) {
            float acc[U][N];
            Chunk<T> first[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                first[u].raw = make_uint4(0, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < N; ++e) acc[u][e] = 0.0f;
            }
            auto fetch = [&](int32_t r, Chunk<T> (&v)[U]) __attribute__((always_inline)) {
                const uint4* row = reinterpret_cast<const uint4*>(x + (int64_t)(r < 0 ? 0 : r) * a.hidden);
#pragma unroll
                for (int u = 0; u < U; ++u)
                    v[u].raw = (r >= 0 && c0 + 64 * u < chunks) ? load_stream16(row + c0 + 64 * u) : make_uint4(0, 0, 0, 0);
            };
            auto add = [&](int32_t r, float w, Chunk<T> (&v)[U]) __attribute__((always_inline)) {
                if (r < 0) return;  // (uniform) an unfilled slot adds nothing, not even +0 to a -0
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (SCALE) {
#pragma unroll
                        for (int e = 0; e < N; ++e) v[u].e[e] = El<DT>::from_f32(El<DT>::to_f32(v[u].e[e]) * w);
                    }
                    if (k == 1) first[u] = v[u];
#pragma unroll
                    for (int e = 0; e < N; ++e) acc[u][e] += El<DT>::to_f32(v[u].e[e]);
                }
            };
            int j = 0;
            for (; j + 1 < k; j += 2) {  // two terms' rows in flight; added in slot order
                int32_t r0, r1;
                float w0, w1;
                term(j, r0, w0);
                term(j + 1, r1, w1);
                Chunk<T> v0[U], v1[U];
                fetch(r0, v0);
                fetch(r1, v1);
                add(r0, w0, v0);
                add(r1, w1, v1);
            }
            if (j < k) {
                int32_t r0;
                float w0;
                term(j, r0, w0);
                Chunk<T> v0[U];
                fetch(r0, v0);
                add(r0, w0, v0);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (c0 + 64 * u >= chunks) continue;
                Chunk<T> o;
#pragma unroll
                for (int e = 0; e < N; ++e) o.e[e] = El<DT>::from_f32(acc[u][e]);
                reinterpret_cast<uint4*>(out)[c0 + 64 * u] = (k == 1) ? first[u].raw : o.raw;  // top_k 1 is a pure move (keeps -0)
            }
        }
    } else {
        for (int64_t c = lane; c < a.hidden; c += 64) {
            float acc = 0.0f;
            T first = 0;
            for (int j = 0; j < k; ++j) {
                const int64_t slot = t * k + j;
                const int32_t r = a.inverse[slot];
                if (r < 0) continue;
                T v = x[(int64_t)r * a.hidden + c];
                if (SCALE) v = El<DT>::from_f32(El<DT>::to_f32(v) * load_weight(a.weights, a.w_dtype, slot));
                if (k == 1) first = v;
                acc += El<DT>::to_f32(v);
            }
            out[c] = (k == 1) ? first : El<DT>::from_f32(acc);
        }
    }
    }
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// out[slot] = dot(x[r], grad[slot / top_k]) for every filled row r of the expert-sorted side
template <int DT, bool BINNED>
__global__ __launch_bounds__(kThreads) void scatter_wgrad_kernel(PermuteArgs a, int64_t rows)
{
    using T = typename El<DT>::T;
    constexpr int N = 16 / sizeof(T);
    const int lane = threadIdx.x & 63;
    for (int64_t r = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6); r < rows;
         r += (int64_t)gridDim.x * kWavesPerBlock) {
    const int64_t idx = slot_of_row<BINNED>(a, r);
    if (idx < 0) continue;
    const T* x = reinterpret_cast<const T*>(a.x) + r * a.hidden;
    const T* g = reinterpret_cast<const T*>(a.grad) + (idx / a.top_k) * a.hidden;
    float acc = 0.0f;
    if (a.vec) {
        const int64_t chunks = a.hidden / N;
        constexpr int U = 4;  // chunks in flight per lane; summed in the order of a chunk-by-chunk loop
        for (int64_t c0 = lane; c0 < chunks; c0 += 64 * U) {
            Chunk<T> xv[U], gv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool ok = c0 + 64 * u < chunks;
                xv[u].raw = ok ? load_stream16(reinterpret_cast<const uint4*>(x) + c0 + 64 * u) : make_uint4(0, 0, 0, 0);
                gv[u].raw = ok ? reinterpret_cast<const uint4*>(g)[c0 + 64 * u] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (c0 + 64 * u >= chunks) continue;
#pragma unroll
                for (int e = 0; e < N; ++e) acc += El<DT>::to_f32(xv[u].e[e]) * El<DT>::to_f32(gv[u].e[e]);
            }
        }
    } else {
        for (int64_t c = lane; c < a.hidden; c += 64) acc += El<DT>::to_f32(x[c]) * El<DT>::to_f32(g[c]);
    }
    acc = wave_sum(acc);
    if (lane == 0) reinterpret_cast<T*>(a.out)[idx] = El<DT>::from_f32(acc);
    }
}

// ---- host side --------------------------------------------------------------------------------------------
int elem_size(int dt) { return dt == MI8_F32 ? 4 : (dt == MI8_RAW8 ? 1 : 2); }
bool valid_dt(int dt, bool allow_raw) { return dt == MI8_BF16 || dt == MI8_F32 || dt == MI8_F16 || (allow_raw && dt == MI8_RAW8); }
bool valid_w(int dt) { return dt == MI8_BF16 || dt == MI8_F32 || dt == MI8_F16; }
// one wave per row; long inputs are walked by a fixed-size grid (8 blocks per CU's worth) so that waves stay
// resident and keep several rows in flight
unsigned wave_blocks(int64_t rows)
{
    const int64_t need = ceil_div(rows, kWavesPerBlock);
    return (unsigned)(need < kMaxBlocks ? need : kMaxBlocks);
}

bool rows_vectorisable(int64_t hidden, int dt, const void* p0, const void* p1, const void* p2 = nullptr)
{
    return (hidden * elem_size(dt)) % 16 == 0 && aligned16(p0) && aligned16(p1) && aligned16(p2);
}

int check_common(const char* what, const void* x, const void* out, const int32_t* indices, int dtype, bool allow_raw,
                 const void* weights, int w_dtype, int64_t tokens, int64_t hidden, int32_t top_k)
{
    MI8_REQUIRE(x && out && indices, MI8_ERR_ARG, "%s: null pointer", what);
    MI8_REQUIRE(valid_dt(dtype, allow_raw), MI8_ERR_ARG, "%s: unknown element type %d", what, dtype);
    MI8_REQUIRE(!weights || (valid_w(w_dtype) && dtype != MI8_RAW8), MI8_ERR_ARG,
                "%s: weights need a floating-point element type and weight type", what);
    MI8_REQUIRE(tokens > 0 && hidden > 0 && top_k > 0, MI8_ERR_ARG, "%s: empty problem (tokens %lld, hidden %lld, top_k %d)",
                what, (long long)tokens, (long long)hidden, top_k);
    MI8_REQUIRE(tokens * top_k < ((int64_t)1 << 31), MI8_ERR_UNSUPPORTED, "%s: more than 2^31 token slots", what);
    return MI8_OK;
}

int check_bins(const char* what, const int32_t* bins, int32_t experts, int64_t capacity)
{
    MI8_REQUIRE(bins && experts > 0 && capacity > 0, MI8_ERR_ARG, "%s: bins, experts and capacity are required", what);
    MI8_REQUIRE((int64_t)experts * capacity < ((int64_t)1 << 31), MI8_ERR_UNSUPPORTED, "%s: more than 2^31 binned rows", what);
    return MI8_OK;
}

template <bool BINNED>
int launch_gather(PermuteArgs& a, int dtype, int64_t rows, hipStream_t st)
{
    const bool scale = a.weights != nullptr;
#define MI8_G(DT_)                                                                                              \
    if (scale)                                                                                                  \
        hipLaunchKernelGGL((gather_kernel<DT_, true, BINNED>), dim3(wave_blocks(rows)), dim3(kThreads), 0, st, a, rows); \
    else                                                                                                        \
        hipLaunchKernelGGL((gather_kernel<DT_, false, BINNED>), dim3(wave_blocks(rows)), dim3(kThreads), 0, st, a, rows)
    switch (dtype) {
        case MI8_BF16: MI8_G(MI8_BF16); break;
        case MI8_F16: MI8_G(MI8_F16); break;
        case MI8_F32: MI8_G(MI8_F32); break;
        default: hipLaunchKernelGGL((gather_kernel<MI8_RAW8, false, BINNED>), dim3(wave_blocks(rows)), dim3(kThreads), 0, st, a, rows);
    }
#undef MI8_G
    return launch_status(BINNED ? "mi8_moe_binned_gather" : "mi8_moe_gather");
}

template <bool BINNED>
int launch_scatter(PermuteArgs& a, int dtype, int64_t rows, int64_t tokens, hipStream_t st)
{
    const unsigned tb = 256;
    // tokens beyond an expert's capacity fill no slot; neither does a slot that `indices` fails to name
    hipLaunchKernelGGL(fill_kernel<int32_t>, dim3((unsigned)ceil_div(a.n, tb)), dim3(tb), 0, st, a.inverse, a.n, (int32_t)-1);
    hipLaunchKernelGGL((inverse_kernel<BINNED>), dim3((unsigned)ceil_div(rows, tb)), dim3(tb), 0, st, a, rows);
    const bool scale = a.weights != nullptr;
#define MI8_S(DT_)                                                                                               \
    if (scale)                                                                                                   \
        hipLaunchKernelGGL((scatter_reduce_kernel<DT_, true>), dim3(wave_blocks(tokens)), dim3(kThreads), 0, st, a, tokens); \
    else                                                                                                         \
        hipLaunchKernelGGL((scatter_reduce_kernel<DT_, false>), dim3(wave_blocks(tokens)), dim3(kThreads), 0, st, a, tokens)
    switch (dtype) {
        case MI8_BF16: MI8_S(MI8_BF16); break;
        case MI8_F16: MI8_S(MI8_F16); break;
        default: MI8_S(MI8_F32);
    }
#undef MI8_S
    return launch_status(BINNED ? "mi8_moe_binned_scatter" : "mi8_moe_scatter");
}

template <bool BINNED>
int launch_wgrad(PermuteArgs& a, int dtype, int64_t rows, hipStream_t st)
{
    switch (dtype) {
        case MI8_BF16:
            hipLaunchKernelGGL((scatter_wgrad_kernel<MI8_BF16, BINNED>), dim3(wave_blocks(rows)), dim3(kThreads), 0, st, a, rows);
            break;
        case MI8_F16:
            hipLaunchKernelGGL((scatter_wgrad_kernel<MI8_F16, BINNED>), dim3(wave_blocks(rows)), dim3(kThreads), 0, st, a, rows);
            break;
        default:
            hipLaunchKernelGGL((scatter_wgrad_kernel<MI8_F32, BINNED>), dim3(wave_blocks(rows)), dim3(kThreads), 0, st, a, rows);
    }
    return launch_status(BINNED ? "mi8_moe_binned_scatter_wgrad" : "mi8_moe_scatter_wgrad");
}

}  // namespace
}  // namespace mi8

using namespace mi8;

extern "C" int mi8_moe_gather(const void* x, int dtype, int64_t tokens, int64_t hidden, const int32_t* indices,
                              const void* weights, int w_dtype, int32_t top_k, void* out, void* stream)
{
    int rc = check_common("mi8_moe_gather", x, out, indices, dtype, true, weights, w_dtype, tokens, hidden, top_k);
    if (rc != MI8_OK) return rc;
    PermuteArgs a{x, out, indices, weights, w_dtype, nullptr, nullptr, nullptr, tokens * top_k, hidden, top_k, 0, 0,
                  rows_vectorisable(hidden, dtype, x, out)};
    return launch_gather<false>(a, dtype, a.n, (hipStream_t)stream);
}

extern "C" int mi8_moe_binned_gather(const void* x, int dtype, int64_t tokens, int64_t hidden, const int32_t* indices,
                                     const void* weights, int w_dtype, const int32_t* bins, int32_t experts,
                                     int64_t capacity, int32_t top_k, void* out, void* stream)
{
    int rc = check_common("mi8_moe_binned_gather", x, out, indices, dtype, true, weights, w_dtype, tokens, hidden, top_k);
    if (rc == MI8_OK) rc = check_bins("mi8_moe_binned_gather", bins, experts, capacity);
    if (rc != MI8_OK) return rc;
    PermuteArgs a{x, out, indices, weights, w_dtype, bins, nullptr, nullptr, tokens * top_k, hidden, top_k, experts,
                  (int32_t)capacity, rows_vectorisable(hidden, dtype, x, out)};
    return launch_gather<true>(a, dtype, (int64_t)experts * capacity, (hipStream_t)stream);
}

extern "C" int mi8_moe_scatter(const void* x, int dtype, int64_t tokens, int64_t hidden, const int32_t* indices,
                               const void* weights, int w_dtype, int32_t top_k, int32_t* inverse_workspace, void* out,
                               void* stream)
{
    int rc = check_common("mi8_moe_scatter", x, out, indices, dtype, false, weights, w_dtype, tokens, hidden, top_k);
    if (rc != MI8_OK) return rc;
    MI8_REQUIRE(inverse_workspace, MI8_ERR_ARG, "mi8_moe_scatter: the inverse workspace (tokens * top_k int32) is required");
    PermuteArgs a{x, out, indices, weights, w_dtype, nullptr, inverse_workspace, nullptr, tokens * top_k, hidden, top_k, 0,
                  0, rows_vectorisable(hidden, dtype, x, out)};
    return launch_scatter<false>(a, dtype, a.n, tokens, (hipStream_t)stream);
}

extern "C" int mi8_moe_binned_scatter(const void* x, int dtype, int64_t tokens, int64_t hidden, const int32_t* indices,
                                      const void* weights, int w_dtype, const int32_t* bins, int32_t experts,
                                      int64_t capacity, int32_t top_k, int32_t* inverse_workspace, void* out,
                                      void* stream)
{
    int rc = check_common("mi8_moe_binned_scatter", x, out, indices, dtype, false, weights, w_dtype, tokens, hidden, top_k);
    if (rc == MI8_OK) rc = check_bins("mi8_moe_binned_scatter", bins, experts, capacity);
    if (rc != MI8_OK) return rc;
    MI8_REQUIRE(inverse_workspace, MI8_ERR_ARG, "mi8_moe_binned_scatter: the inverse workspace (tokens * top_k int32) is required");
    PermuteArgs a{x, out, indices, weights, w_dtype, bins, inverse_workspace, nullptr, tokens * top_k, hidden, top_k,
                  experts, (int32_t)capacity, rows_vectorisable(hidden, dtype, x, out)};
    return launch_scatter<true>(a, dtype, (int64_t)experts * capacity, tokens, (hipStream_t)stream);
}

extern "C" int mi8_moe_scatter_wgrad(const void* x, const void* grad, int dtype, int64_t tokens, int64_t hidden,
                                     const int32_t* indices, int32_t top_k, void* out, void* stream)
{
    int rc = check_common("mi8_moe_scatter_wgrad", x, out, indices, dtype, false, nullptr, 0, tokens, hidden, top_k);
    if (rc != MI8_OK) return rc;
    MI8_REQUIRE(grad, MI8_ERR_ARG, "mi8_moe_scatter_wgrad: grad is null");
    PermuteArgs a{x, out, indices, nullptr, 0, nullptr, nullptr, grad, tokens * top_k, hidden, top_k, 0, 0,
                  rows_vectorisable(hidden, dtype, x, grad)};
    return launch_wgrad<false>(a, dtype, a.n, (hipStream_t)stream);
}

extern "C" int mi8_moe_binned_scatter_wgrad(const void* x, const void* grad, int dtype, int64_t tokens, int64_t hidden,
                                            const int32_t* indices, const int32_t* bins, int32_t experts,
                                            int64_t capacity, int32_t top_k, void* out, void* stream)
{
    int rc = check_common("mi8_moe_binned_scatter_wgrad", x, out, indices, dtype, false, nullptr, 0, tokens, hidden, top_k);
    if (rc == MI8_OK) rc = check_bins("mi8_moe_binned_scatter_wgrad", bins, experts, capacity);
    if (rc != MI8_OK) return rc;
    MI8_REQUIRE(grad, MI8_ERR_ARG, "mi8_moe_binned_scatter_wgrad: grad is null");
    hipStream_t st = (hipStream_t)stream;
    // slots of dropped tokens get no contribution: the output starts from zero
    const int64_t n = tokens * top_k;
    if (elem_size(dtype) == 4)
        hipLaunchKernelGGL(fill_kernel<uint32_t>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, st, (uint32_t*)out, n, 0u);
    else
        hipLaunchKernelGGL(fill_kernel<uint16_t>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, st, (uint16_t*)out, n,
                           (uint16_t)0);
    PermuteArgs a{x, out, indices, nullptr, 0, bins, nullptr, grad, tokens * top_k, hidden, top_k, experts,
                  (int32_t)capacity, rows_vectorisable(hidden, dtype, x, grad)};
    return launch_wgrad<true>(a, dtype, (int64_t)experts * capacity, st);
}
