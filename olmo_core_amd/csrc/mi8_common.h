// Shared host/device helpers for libmi8 (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/mi8.h"

namespace mi8 {

// ---- host side: error reporting --------------------------------------------------------------
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
int launch_status(const char* what);  // MI8_OK or MI8_ERR_LAUNCH after a kernel launch

// One-time set-up per kernel and device, safe under concurrent first calls: `done` holds one bit per device
// ordinal; setting the attribute twice is harmless, so two racing threads only repeat the call.
int reserve_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done, const char* what);
int num_compute_units();  // of the current device (cached per device)

#define MI8_REQUIRE(cond, code, ...)     \
    do {                                 \
        if (!(cond)) {                   \
            ::mi8::set_error(__VA_ARGS__); \
            return (code);               \
        }                                \
    } while (0)

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// ---- device side ---------------------------------------------------------------------------------

template <int FP8>
struct Fp8Traits;
template <>
struct Fp8Traits<MI8_E4M3> {
    static constexpr float kMax = 448.0f;
    static constexpr double kMaxD = 448.0;
    static constexpr int kMant = 3;
    static constexpr int kBias = 7;
};
template <>
struct Fp8Traits<MI8_E5M2> {
    static constexpr float kMax = 57344.0f;
    static constexpr double kMaxD = 57344.0;
    static constexpr int kMant = 2;
    static constexpr int kBias = 15;
};

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __float_as_uint(f); }

// Maximum that orders NaN patterns above everything: on |x| bit patterns an unsigned integer max is
// the IEEE maximum for non-NaN values and keeps a NaN (pattern > 0x7F800000) once one was seen.
__device__ __forceinline__ uint32_t umax32(uint32_t a, uint32_t b) { return a > b ? a : b; }

__device__ __forceinline__ uint32_t wave_umax(uint32_t v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = umax32(v, (uint32_t)__shfl_xor((int)v, off, 64));
    return v;
}

// The contiguous range [lo, hi) of n items that workgroup blockIdx.x of a 256-thread, one-dimensional-in-x grid
// streams: ranges are multiples of 256 items (4 KB of 16-byte vectors), the last ones may be short or empty.
// A workgroup that walks its own contiguous range keeps DRAM pages open; the same loads issued grid-stride
// (every workgroup touching 4 KB every gridDim.x * 4 KB) reach 10-15 % less of the HBM bandwidth.
struct BlockRange {
    int64_t lo, hi;
};
__device__ __forceinline__ BlockRange block_range(int64_t n, int64_t block, int64_t blocks)
{
    const int64_t per = (((n + blocks - 1) / blocks) + 255) & ~(int64_t)255;
    int64_t lo = block * per;
    lo = lo < n ? lo : n;
    int64_t hi = lo + per;
    hi = hi < n ? hi : n;
    return BlockRange{lo, hi};
}
__device__ __forceinline__ BlockRange block_range(int64_t n) { return block_range(n, blockIdx.x, gridDim.x); }

// scale = float32(FP8_MAX * (1 / max(float64(amax), 1e-12))); NaN amax gives a NaN scale, +inf gives 0.
// Optional round-down to a power of two clears the mantissa (scale is always a normal float or 0 here).
template <int FP8>
__device__ __forceinline__ float scale_from_amax_bits(uint32_t amax_bits, bool pow2)
{
    double a = (double)bits_to_f32(amax_bits);
    a = (a < 1e-12) ? 1e-12 : a;  // false for NaN: NaN is kept
    const double r = 1.0 / a;     // IEEE double division
    float s = (float)(r * Fp8Traits<FP8>::kMaxD);
    if (pow2 && s == s) s = bits_to_f32(f32_to_bits(s) & 0x7F800000u);
    return s;
}

// clamp to [-m, m]; a NaN passes through (both comparisons are false)
__device__ __forceinline__ float clamp_keep_nan(float y, float m)
{
    y = (y > m) ? m : y;
    y = (y < -m) ? -m : y;
    return y;
}

// Integer round-to-nearest-even conversion of an already clamped float (|y| <= FP8_MAX or NaN) to one fp8
// byte.  Normal range: add the rounding bias to the float's bit pattern and shift; subnormal range: add
// 2^(23 + e_min - mant) so that the float adder performs the round-to-nearest-even at the right bit.
template <int FP8>
__device__ __forceinline__ uint32_t sw_cvt_byte(float y)
{
    constexpr int MB = Fp8Traits<FP8>::kMant;
    constexpr int BIAS = Fp8Traits<FP8>::kBias;
    const uint32_t u = f32_to_bits(y);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7FFFFFFFu;
    uint32_t code;
    if (a > 0x7F800000u) {
        code = 0x7Fu;
    } else if (a >= ((uint32_t)(127 + 1 - BIAS) << 23)) {
        constexpr int SH = 23 - MB;
        uint32_t r = a + ((1u << (SH - 1)) - 1u) + ((a >> SH) & 1u);
        code = (r >> SH) - ((uint32_t)(127 - BIAS) << MB);
    } else {
        constexpr uint32_t MAGIC = (uint32_t)(127 + 23 + 1 - BIAS - MB) << 23;
        const float t = bits_to_f32(a) + bits_to_f32(MAGIC);
        code = f32_to_bits(t) - MAGIC;
    }
    return sign | code;
}

// Four clamped floats -> four packed fp8 bytes (a in the lowest byte).
template <int FP8, bool SW>
__device__ __forceinline__ uint32_t cvt4(float a, float b, float c, float d)
{
    if constexpr (SW) {
        return sw_cvt_byte<FP8>(a) | (sw_cvt_byte<FP8>(b) << 8) | (sw_cvt_byte<FP8>(c) << 16) |
               (sw_cvt_byte<FP8>(d) << 24);
    } else if constexpr (FP8 == MI8_E4M3) {
        int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
        r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
        return (uint32_t)r;
    } else {
        int r = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
        r = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, r, true);
        return (uint32_t)r;
    }
}

// scale, clamp, convert four values
template <int FP8, bool SW>
__device__ __forceinline__ uint32_t quant4(float a, float b, float c, float d, float s0, float s1, float s2,
                                           float s3)
{
    constexpr float M = Fp8Traits<FP8>::kMax;
    return cvt4<FP8, SW>(clamp_keep_nan(a * s0, M), clamp_keep_nan(b * s1, M), clamp_keep_nan(c * s2, M),
                         clamp_keep_nan(d * s3, M));
}

// 4x4 byte transpose: r[j] holds bytes (row j, cols 0..3); afterwards c[i] holds bytes (col i, rows 0..3).
__device__ __forceinline__ void transpose4x4_bytes(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3,
                                                   uint32_t& c0, uint32_t& c1, uint32_t& c2, uint32_t& c3)
{
    const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
    const uint32_t t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
    const uint32_t t2 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    c0 = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    c1 = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    c2 = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    c3 = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

// Eight consecutive high-precision elements starting at a 16-byte aligned address -> float[8]
// Streaming accesses (the nt bit): for data a kernel reads for the last time, or writes for a later kernel to read.
// Such lines take no space from data that is about to be read again - in a two-pass cast the second pass's
// outputs otherwise evict what the first pass left of the input in the memory-side cache (16384 x 11008: amax + cast
// 232 -> 181 us); rows gathered several times and tables read again keep the default.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 load_stream16(const void* p)
{
    const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(t[0], t[1], t[2], t[3]);
}
__device__ __forceinline__ void store_stream16(void* p, uint4 v)
{
    __builtin_nontemporal_store((u32x4_t){v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4_t*>(p));
}
__device__ __forceinline__ void store_stream8(void* p, uint32_t lo, uint32_t hi)
{
    __builtin_nontemporal_store((u32x2_t){lo, hi}, reinterpret_cast<u32x2_t*>(p));
}

template <int HP>
struct HpVec;
template <>
struct HpVec<MI8_BF16> {
    static constexpr int kBytes = 2;
    template <bool STREAM = false>
    __device__ static __forceinline__ void load8(const void* p, bool ok, float (&f)[8])
    {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (ok) v = STREAM ? load_stream16(p) : *reinterpret_cast<const uint4*>(p);
        f[0] = bits_to_f32(v.x << 16);
        f[1] = bits_to_f32(v.x & 0xFFFF0000u);
        f[2] = bits_to_f32(v.y << 16);
        f[3] = bits_to_f32(v.y & 0xFFFF0000u);
        f[4] = bits_to_f32(v.z << 16);
        f[5] = bits_to_f32(v.z & 0xFFFF0000u);
        f[6] = bits_to_f32(v.w << 16);
        f[7] = bits_to_f32(v.w & 0xFFFF0000u);
    }
};
template <>
struct HpVec<MI8_F32> {
    static constexpr int kBytes = 4;
    template <bool STREAM = false>
    __device__ static __forceinline__ void load8(const void* p, bool ok, float (&f)[8])
    {
        const uint4* q = reinterpret_cast<const uint4*>(p);
        uint4 v0 = make_uint4(0, 0, 0, 0), v1 = v0;
        if (ok) {
            v0 = STREAM ? load_stream16(q) : q[0];
            v1 = STREAM ? load_stream16(q + 1) : q[1];
        }
        f[0] = bits_to_f32(v0.x);
        f[1] = bits_to_f32(v0.y);
        f[2] = bits_to_f32(v0.z);
        f[3] = bits_to_f32(v0.w);
        f[4] = bits_to_f32(v1.x);
        f[5] = bits_to_f32(v1.y);
        f[6] = bits_to_f32(v1.z);
        f[7] = bits_to_f32(v1.w);
    }
};

// |x| bit pattern (as float32 bits) maximum over 8 floats
__device__ __forceinline__ uint32_t absmax8_bits(const float (&f)[8])
{
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) m = umax32(m, f32_to_bits(f[i]) & 0x7FFFFFFFu);
    return m;
}

}  // namespace mi8
