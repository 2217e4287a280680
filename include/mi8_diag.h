/*
 * mi8 diagnostics: C ABI of libmi8_diag.so, a separate library with measurement kernels that are no part of the
 * float8 linear path and of its drop-in boundary (include/mi8.h, libmi8.so).  Built by the same recipe
 * (python -m olmo_core_amd.build); loaded only by bench.py (--power-probe, --feed-probe, --store-probe, --tile-timeline).  No counterpart in the
 * reference.  Conventions as in mi8.h: int status (0 = ok), mi8_diag_last_error() for the text, work is only
 * enqueued on `stream`.
 */
#ifndef MI8_DIAG_H
#define MI8_DIAG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* mi8_diag_last_error(void);

/* `workgroups` x 4 waves issue back-to-back fp8 MFMAs on resident
 * registers, 2 * 128^3 flop per wave and iteration, shape 0 = 32x32x64, 1 = 16x16x128, on all-zero or on random
 * operand bytes.  Timed by the caller; on random operands this is the matrix throughput the chip sustains under
 * its power limit.  sink: float32 [workgroups * 256], overwritten.
 */
int mi8_probe_mfma_loop(int mfma_shape, int random_operands, int iterations, int workgroups, float* sink, void* stream);
/* What the operand feed of a GEMM K step costs a stream of MFMAs (diagnostic, no counterpart in the reference):
 * 256 workgroups of four waves run 64 16x16x128 MFMAs per iteration from resident registers and, beside them,
 * `loads` (0, 8, 16) loads of 1 KB per wave - kind 0: direct to LDS, 1: to registers, 2: LDS stores of resident
 * registers instead, 3: loads to registers and LDS stores interleaved - and `reads` (0, 32) 16-byte LDS fragment
 * reads per wave, with `barriers` (0..2) workgroup barriers per iteration.  window: at least 2 MiB + 128 KiB of
 * readable device memory; sink: 65536 floats;
 * clocks[0] = shader-clock cycles of the loop on one workgroup, clocks[1] = the same span in ticks of the constant
 * 100 MHz clock (host-visible or device memory). */
int mi8_probe_mfma_feed(int kind, int loads, int reads, int barriers, int random_operands, int iterations, const void* window,
                        float* sink, unsigned long long* clocks, void* stream);

/* The store path of a compute unit: `workgroups` x `waves` (1..4, one per SIMD) waves each issue 8 * iterations stores of 16
 * bytes per lane, one instruction covering `rows` (2, 4, 8, 16) rows of 1024 / rows contiguous bytes, into the layout of a
 * GEMM output tile (256 rows x 512 bytes per workgroup at row pitch `pitch`; window: 16384 * pitch + 4096 bytes of device
 * memory, overwritten).  cycles: uint32 [workgroups * 4], shader-clock cycles of every wave's loop including the wait for
 * its last store. */
int mi8_probe_store_rate(int rows, int waves, int workgroups, int iterations, void* window, int64_t pitch, uint32_t* cycles,
                         void* stream);
/* One launch of the library's persistent fp8 GEMM (the kernel of mi8_gemm_fp8 for M, N >= 256, K % 128 == 0, N % 8 == 0,
 * single scales, bf16 output, contiguous operands) built with time stamps: wave 0 of workgroup w writes into
 * stamps[256 * w ..], for each of its first 16 tiles t, the low 32 bits of the shader clock at 13 points -
 * [13 t + 0] K loop start, [+1] after three K steps, [+2] epilogue start, [+3 .. +10] the eight epilogue passes (each
 * after its staging writes have landed), [+11] last store issued, [+12] tile end (unused entries stay 0) - and in
 * [254], [255] the constant 100 MHz clock at kernel start and end.  stamps: uint32 [256 * 256] of device memory.
 * Synchronises `stream` before and after the launch (the stamp pointer is a device global of the library). */
int mi8_diag_gemm_tile_timeline(const void* a, const float* sa, const void* b, const float* sb, void* out, int64_t M, int64_t N,
                                int64_t K, int a_dtype, int b_dtype, uint32_t* stamps, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI8_DIAG_H */
