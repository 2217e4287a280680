// Diagnostics (libmi8_diag.so, declared in include/mi8_diag.h; not part of libmi8.so): back-to-back fp8 MFMAs with nothing else running, on all-zero or on random operand registers; and the
// same stream with the operand feed of a GEMM K step beside it (mi8_probe_mfma_feed).
// The rate on random operands is what the chip sustains under its power limit (the clock drops under matrix load),
// the rate on zeros what the matrix pipes do at full clock: the two numbers bracket what a GEMM can reach.
#include "mi8_common.h"

namespace mi8 {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t mix(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

// one wave: a 128 x 128 x 128 product per iteration from resident fragments (64 MFMAs of 16x16x128 or 32 of 32x32x64)
template <int MODE>
__global__ __launch_bounds__(256, 1) void mfma_loop_kernel(int iters, int random, float* __restrict__ sink)
{
    v8i a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t ra = mix(threadIdx.x * 131 + i * 17 + e + blockIdx.x * 7919);
            const uint32_t rb = mix(threadIdx.x * 257 + i * 29 + e * 3 + 1 + blockIdx.x * 104729);
            // random fp8 bytes of moderate magnitude, never NaN: the top exponent bit of every byte is cleared
            a[i][e] = random ? (int)(ra & 0xBFBFBFBFu) : 0;
            b[i][e] = random ? (int)(rb & 0xBFBFBFBFu) : 0;
        }
    float s = 0;
    if constexpr (MODE == 0) {
        v16f acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int x = 0; x < 16; ++x)
                    acc[x] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[(x & 3) + 4 * h], a[(x >> 2) + 4 * h], acc[x], 0, 0,
                                                                             0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += acc[i][e];
    } else {
        v4f acc[64];
#pragma unroll
        for (int i = 0; i < 64; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int x = 0; x < 64; ++x)
                acc[x] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[x & 7], a[x >> 3], acc[x], 0, 0, 0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 64; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) s += acc[i][e];
    }
    sink[blockIdx.x * 256 + threadIdx.x] = s;
}

// What feeding the operands costs a stream of MFMAs: one wave per SIMD runs 64 16x16x128 MFMAs per iteration (one
// 128-byte K step of the GEMM's 128 x 128 wave tile) from resident registers, and beside them, as the feed of that
// K step would, `loads` loads of 1 KB per wave (the GEMM issues 16) and `reads` ds_read_b128 (the GEMM issues 32,
// with the GEMM's bank-conflict-free fragment addresses), with `barriers` workgroup barriers per iteration (the GEMM
// has two: they bring the four waves' loads to the same instant).  Loads take their rows from a 2 MB window that every XCD's
// workgroups share (L2 hits), so the figure is the cost of issuing and landing the loads, not of memory.
//   kind 0: global_load_lds_dwordx4 (direct to LDS, what the GEMM uses)    kind 1: global_load_dwordx4 to registers
//   kind 2: ds_write_b128 of resident registers (no global access)          kind 3: kind 1 and kind 2 interleaved
// Asynchronous results land in registers that stay dedicated to them for the whole loop (read-write asm operands):
// a register the compiler believed free after the instruction could otherwise be reused for an address.
typedef int v4i __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

template <int KIND, int LOADS, int READS>
__global__ __launch_bounds__(256, 1) void mfma_feed_kernel(const uint8_t* __restrict__ src, int iters, int random, int barriers,
                                                           float* __restrict__ sink, unsigned long long* __restrict__ clocks)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    v8i a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t ra = mix(threadIdx.x * 131 + i * 17 + e + blockIdx.x * 7919);
            const uint32_t rb = mix(threadIdx.x * 257 + i * 29 + e * 3 + 1 + blockIdx.x * 104729);
            a[i][e] = random ? (int)(ra & 0xBFBFBFBFu) : 0;
            b[i][e] = random ? (int)(rb & 0xBFBFBFBFu) : 0;
        }
    for (int i = threadIdx.x; i < 32768; i += 256) reinterpret_cast<uint32_t*>(lds)[i] = random ? (mix(i) & 0xBFBFBFBFu) : 0;
    __syncthreads();
    constexpr uint32_t kSpan = 2u << 20, kPitch = 8192 + 128;
    const uint32_t lane_off = (uint32_t)(lane / 8) * kPitch + (lane % 8) * 16;
    const uint32_t base = (uint32_t)(((size_t)(blockIdx.x >> 3) * 7919 * 4096) % kSpan);
    // fragment read addresses of the GEMM (row lane % 16, 16-byte chunk XOR-swizzled by the row)
    const int r16 = lane & 15, kb = lane >> 4;
    const int swz = ((r16 >> 2) & 1) | (((r16 >> 1) & 1) << 2);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)lds;
    const uint32_t rd0 = lds0 + (uint32_t)(r16 * 128 + (((2 * kb) ^ swz) << 4)) + wave * 16384;
    const uint32_t rd1 = lds0 + (uint32_t)(r16 * 128 + (((2 * kb + 1) ^ swz) << 4)) + wave * 16384;
    const uint32_t wr = lds0 + 65536 + wave * 16384 + lane * 16;
    v4i got[4], staged[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) got[i] = (v4i){0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 16; ++i) staged[i] = (v4i){0, 0, 0, 0};
    v4f acc[64];
#pragma unroll
    for (int i = 0; i < 64; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][e] = 0.f;
    const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
        int issued = 0, reads = 0;
#pragma unroll
        for (int x = 0; x < 64; ++x) {
            // (uniform) the GEMM's waves meet at a barrier at the start and in the middle of a K step
            if ((x == 0 && barriers >= 1) || (x == 32 && barriers >= 2)) asm volatile("s_barrier" ::: "memory");
            acc[x] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[x & 7], a[x >> 3], acc[x], 0, 0, 0, 0, 0, 0);
            if (READS > 0 && x % (64 / (READS > 0 ? READS : 1)) == 0) {
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "+v"(got[reads & 3]) : "v"((reads & 1) ? rd1 : rd0), "n"(((x / 2) % 8) * 2048) : "memory");
                ++reads;
            }
            if (LOADS > 0 && x % (64 / (LOADS > 0 ? LOADS : 1)) == (64 / (LOADS > 0 ? LOADS : 1)) - 1) {
                const int slot = issued & 15;
                uint32_t uni = (base + (uint32_t)((wave * 16 + slot) * 8) * kPitch + (uint32_t)it * 128) % kSpan;
                uni = __builtin_amdgcn_readfirstlane(uni);
                if (KIND == 0) {
                    __builtin_amdgcn_global_load_lds((gptr_t)(src + uni + lane_off), (lptr_t)(lds + 65536 + (wave * 16 + slot) * 1024), 16, 0, 0);
                } else {
                    if (KIND == 2 || KIND == 3)
                        asm volatile("ds_write_b128 %1, %0 offset:%2" : "+v"(staged[slot]) : "v"(wr), "n"(slot * 1024) : "memory");
                    if (KIND == 1 || KIND == 3)
                        asm volatile("global_load_dwordx4 %0, %1, %2" : "+v"(staged[(slot + 15) & 15]) : "v"(lane_off), "s"(src + uni) : "memory");
                }
                ++issued;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (READS > 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (LOADS > 0 && KIND != 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");  // at most one iteration of loads in flight
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0 && blockIdx.x == 17) {
        clocks[0] = c1 - c0;  // shader clock cycles
        clocks[1] = r1 - r0;  // ticks of the constant 100 MHz clock
    }
    __syncthreads();
    float s = 0;
#pragma unroll
    for (int i = 0; i < 64; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) s += acc[i][e];
#pragma unroll
    for (int i = 0; i < 4; ++i) s += (float)got[i][0];
#pragma unroll
    for (int i = 0; i < 16; ++i) s += (float)staged[i][0];
    sink[blockIdx.x * 256 + threadIdx.x] = s + lds[65536 + threadIdx.x];
}

template <int KIND, int LOADS, int READS>
int launch_feed(const uint8_t* src, int iters, int random, int barriers, float* sink, unsigned long long* clocks, hipStream_t st)
{
    auto kern = mfma_feed_kernel<KIND, LOADS, READS>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), 131072, configured, "mi8_probe_mfma_feed")) return rc;
    hipLaunchKernelGGL(kern, dim3(256), dim3(256), 131072, st, src, iters, random, barriers, sink, clocks);
    return launch_status("mi8_probe_mfma_feed");
}

}  // namespace
}  // namespace mi8

using namespace mi8;

extern "C" int mi8_probe_mfma_feed(int kind, int loads, int reads, int barriers, int random_operands, int iterations, const void* window,
                                   float* sink, unsigned long long* clocks, void* stream)
{
    MI8_REQUIRE(window && sink && clocks, MI8_ERR_ARG, "mi8_probe_mfma_feed: null pointer");
    MI8_REQUIRE(iterations > 0 && iterations <= (1 << 20), MI8_ERR_ARG, "mi8_probe_mfma_feed: 1..2^20 iterations");
    MI8_REQUIRE(kind >= 0 && kind <= 3 && (loads == 0 || loads == 8 || loads == 16) && (reads == 0 || reads == 32) &&
                    barriers >= 0 && barriers <= 2,
                MI8_ERR_ARG, "mi8_probe_mfma_feed: kind 0..3, loads 0, 8 or 16, reads 0 or 32, barriers 0..2");
    const uint8_t* src = (const uint8_t*)window;
    hipStream_t st = (hipStream_t)stream;
#define MI8_FEED(K_, L_, R_) \
    if (kind == K_ && loads == L_ && reads == R_) return launch_feed<K_, L_, R_>(src, iterations, random_operands, barriers, sink, clocks, st)
    MI8_FEED(0, 0, 0);
    MI8_FEED(0, 0, 32);
    MI8_FEED(0, 8, 0);
    MI8_FEED(0, 16, 0);
    MI8_FEED(0, 8, 32);
    MI8_FEED(0, 16, 32);
    MI8_FEED(1, 16, 0);
    MI8_FEED(1, 16, 32);
    MI8_FEED(2, 16, 0);
    MI8_FEED(2, 16, 32);
    MI8_FEED(3, 16, 0);
    MI8_FEED(3, 16, 32);
#undef MI8_FEED
    set_error("mi8_probe_mfma_feed: combination kind %d, loads %d, reads %d is not built", kind, loads, reads);
    return MI8_ERR_UNSUPPORTED;
}

extern "C" int mi8_probe_mfma_loop(int mfma_shape, int random_operands, int iterations, int workgroups, float* sink,
                                   void* stream)
{
    MI8_REQUIRE(sink, MI8_ERR_ARG, "mi8_probe_mfma_loop: sink is null");
    MI8_REQUIRE((mfma_shape == 0 || mfma_shape == 1) && iterations > 0 && iterations <= (1 << 22) && workgroups > 0 &&
                    workgroups <= 4096,
                MI8_ERR_ARG, "mi8_probe_mfma_loop: shape 0 (32x32x64) or 1 (16x16x128), 1..2^22 iterations, 1..4096 workgroups");
    hipStream_t st = (hipStream_t)stream;
    if (mfma_shape == 0)
        hipLaunchKernelGGL((mfma_loop_kernel<0>), dim3(workgroups), dim3(256), 0, st, iterations, random_operands, sink);
    else
        hipLaunchKernelGGL((mfma_loop_kernel<1>), dim3(workgroups), dim3(256), 0, st, iterations, random_operands, sink);
    return launch_status("mi8_probe_mfma_loop");
}

// ---- store path -----------------------------------------------------------------------------------
// Every active wave streams 16-byte-per-lane stores into its 128-row x 256-byte quadrant of the workgroup's 256 x 512-byte
// window (the layout of a GEMM output tile with a row pitch of `pitch` bytes): one instruction covers `rows` rows with
// 64 / rows lanes each.  Lane 0 of every wave reports the shader-clock cycles of its loop.
__global__ __launch_bounds__(256, 1) void store_rate_kernel(uint8_t* out, int64_t pitch, int rows, int waves, int iterations,
                                                            uint32_t* cycles)
{
    typedef int v4i __attribute__((ext_vector_type(4)));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (wave >= waves) return;
    const int lanes_per_row = 64 / rows, row = lane / lanes_per_row, chunk = lane % lanes_per_row;
    const int row_bytes = lanes_per_row * 16;                    // bytes of one row written by one instruction
    const int col_blocks = row_bytes >= 256 ? 1 : 256 / row_bytes;
    const int per_sweep = 128 / rows >= 8 ? 8 : 128 / rows;      // instructions per unrolled group
    uint8_t* p0 = out + (int64_t)((int)blockIdx.x % 64) * 256 * pitch + ((int)blockIdx.x / 64) * 512 + (int64_t)(wave >> 1) * 128 * pitch +
                  (wave & 1) * 256 + (int64_t)row * pitch + chunk * 16;
    const int64_t step = (int64_t)rows * pitch;
    const v4i v = {lane, tid, iterations, 7};
    const uint64_t t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iterations; ++it) {
        const int first = it * per_sweep * rows;
        uint8_t* p = p0 + (int64_t)(first & 127) * pitch + ((first >> 7) & (col_blocks - 1)) * row_bytes;
#pragma unroll
        for (int u = 0; u < 8; ++u) *reinterpret_cast<v4i*>(p + (u % per_sweep) * step) = v;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    const uint64_t t1 = __builtin_readcyclecounter();
    if (lane == 0) cycles[blockIdx.x * 4 + wave] = (uint32_t)(t1 - t0);
}

extern "C" int mi8_probe_store_rate(int rows, int waves, int workgroups, int iterations, void* window, int64_t pitch,
                                    uint32_t* cycles, void* stream)
{
    MI8_REQUIRE(window && cycles, MI8_ERR_ARG, "mi8_probe_store_rate: null pointer");
    MI8_REQUIRE((rows == 2 || rows == 4 || rows == 8 || rows == 16) && waves >= 1 && waves <= 4 && workgroups >= 1 &&
                    workgroups <= 256 && iterations > 0 && iterations <= (1 << 16) && pitch >= 2048 && pitch % 16 == 0,
                MI8_ERR_ARG, "mi8_probe_store_rate: rows 2, 4, 8 or 16, 1..4 waves, 1..256 workgroups, pitch >= 2048 and a multiple of 16");
    hipLaunchKernelGGL(store_rate_kernel, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, (uint8_t*)window, pitch, rows, waves,
                       iterations, cycles);
    return launch_status("mi8_probe_store_rate");
}

extern "C" const char* mi8_last_error(void);
extern "C" const char* mi8_diag_last_error(void) { return mi8_last_error(); }
