/*
 * mi8 diagnostics: C ABI of libmi8_diag.so, a separate library with measurement kernels that are no part of the
 * float8 linear path and of its drop-in boundary (include/mi8.h, libmi8.so).  Built by the same recipe
 * (python -m olmo_core_amd.build); loaded only by bench.py (--power-probe, --feed-probe).  No counterpart in the
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

#ifdef __cplusplus
}
#endif
#endif /* MI8_DIAG_H */
