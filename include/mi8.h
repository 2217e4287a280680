/*
 * mi8 - float8 linear path for gfx950 (MI355X): C ABI of libmi8.so.
 *
 * Every entry point is a plain C function over raw device pointers, sizes and a HIP stream handle.
 * Unless a function says otherwise it
 *   - returns MI8_OK (0) or a negative mi8_status; mi8_last_error() gives the text for the calling
 *     thread's most recent failure;
 *   - only enqueues work on `stream` (a hipStream_t passed as void*; NULL = the default stream): it never
 *     synchronises, never allocates or frees device memory, and keeps no state between calls that a caller could
 *     observe (the only memory of the library is per-device one-time set-up: a kernel's dynamic-LDS attribute and
 *     the compute-unit count, both latched with atomics, so first calls from several threads or on several
 *     devices are safe).  The one exception is mi8_cast_tensorwise_static, which works in a scratch array the
 *     library owns per GPU (see there);
 *   - requires every pointer to be 16-byte aligned device memory of at least the stated size.
 * All matrices are dense row-major with the row pitch given (or implied) in elements.
 *
 * The arithmetic these functions implement is the dynamic-scaling float8 training path the reference
 * reaches through torchao (reference: src/olmo_core/float8/__init__.py:133-150 converts every eligible
 * nn.Linear; src/olmo_core/float8/ao.py:152-186 carries the options).  The per-function comments cite
 * the reference interface each one stands in for.
 */
#ifndef MI8_H
#define MI8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI8_VERSION 100 /* major*10000 + minor*100 + patch */

typedef enum mi8_status {
    MI8_OK = 0,
    MI8_ERR_ARG = -1,         /* NULL pointer, negative size, unknown enum value */
    MI8_ERR_UNSUPPORTED = -2, /* shape or alignment outside what the kernels handle */
    MI8_ERR_LAUNCH = -3       /* HIP reported an error at launch */
} mi8_status;

/* float8 encodings (OCP): reference dtype names src/olmo_core/config.py:373-374 */
typedef enum mi8_fp8 { MI8_E4M3 = 0 /* float8_e4m3fn, max 448 */, MI8_E5M2 = 1 /* float8_e5m2, max 57344 */ } mi8_fp8;

/* high-precision element types accepted by the casts (src/olmo_core/config.py:370-372) */
typedef enum mi8_hp {
    MI8_BF16 = 0,
    MI8_F32 = 1,
    MI8_F16 = 2,  /* token-permutation entry points only */
    MI8_RAW8 = 3  /* opaque 1-byte elements (fp8 rows): unweighted permutation only */
} mi8_hp;

/* flags shared by the cast entry points */
#define MI8_FLAG_POW2_SCALE 1u /* round every scale down to a power of two (ao.py:167 round_scales_to_power_of_2) */
#define MI8_FLAG_SW_CVT 2u     /* convert with integer arithmetic instead of v_cvt_pk_{fp8,bf8}_f32 (same bytes) */
#define MI8_FLAG_AMAX_READY 4u /* grouped casts: the amax workspaces already hold the amax of x (see mi8_grouped_swiglu_*) */

/* Number of uint32 slots a tensorwise amax workspace must have. */
#define MI8_AMAX_SLOTS 2048

int mi8_version(void);
const char* mi8_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * Tensorwise dynamic cast.   Stands in for torchao tensor_to_amax / amax_to_scale /
 * hp_tensor_and_scale_to_float8 as invoked by Float8Linear for TENSORWISE cast configs
 * (reference: the default AOCastConfig, src/olmo_core/float8/ao.py:76-86).
 * ------------------------------------------------------------------------------------------- */

/* Partial maxima of |x| over n contiguous elements.  Writes *n_slots_used (host int, may be NULL) and
 * fills slots[0 .. used) with the bit patterns of per-workgroup maxima (float32 bit pattern of |x|; a NaN
 * input yields a NaN pattern, which compares greatest).  slots must hold MI8_AMAX_SLOTS uint32.
 * The number of slots used depends only on n. */
int mi8_amax_partials(const void* x, int hp_dtype, int64_t n, uint32_t* slots, int32_t* n_slots_used, void* stream);

/* mi8_amax_partials for up to MI8_AMAX_BATCH tensors of one dtype in ONE launch (the input and the three weights of a
 * feed-forward block, whose tensorwise scales the reference reduces one after the other: torchao tensor_to_scale per
 * Float8Linear, reference src/olmo_core/float8/ao.py:76-86).  xs, ns, n_slots_used are HOST arrays of `count` entries;
 * tensor t's partials go to slots[t * MI8_AMAX_SLOTS ...], n_slots_used[t] (may be NULL) = mi8_amax_slots_for(ns[t]);
 * the values equal those of `count` separate mi8_amax_partials calls.  slots must hold count * MI8_AMAX_SLOTS uint32. */
#define MI8_AMAX_BATCH 8
int mi8_amax_partials_batch(const void* const* xs, const int64_t* ns, int32_t count, int hp_dtype, uint32_t* slots,
                            int32_t* n_slots_used, void* stream);

/* Number of slots mi8_amax_partials uses for n elements (host-side, no GPU work). */
int32_t mi8_amax_slots_for(int64_t n);

/* amax = max(slots[0..n_slots)), scale = float32(FP8_MAX * (1 / max(float64(amax), 1e-12))), optionally rounded
 * down to a power of two.  out[0] = scale, out[1] = amax (both float32, device). */
int mi8_scale_from_partials(const uint32_t* slots, int32_t n_slots, int fp8_dtype, uint32_t flags, float* out,
                            void* stream);

/* Tensorwise dynamic scales of many tensors in three launches: the once-per-optimizer-step refresh of all
 * float8 weight scales (reference: torchao precompute_float8_dynamic_scale_for_fsdp, called from
 * src/olmo_core/nn/transformer/model.py:1001-1008 when Float8Config.should_precompute_float8_dynamic_scale_for_fsdp,
 * src/olmo_core/float8/__init__.py:54-62).
 *   ptrs / numels: DEVICE arrays [n_tensors] of tensor base pointers (16-byte aligned) and element counts
 *   (multiples of 8 for bf16, 4 for float32); amax_workspace: uint32 [n_tensors] (overwritten);
 *   scales_out: float32 [n_tensors], the same values mi8_scale_from_partials gives tensor by tensor. */
int mi8_multi_tensor_scales(const void* const* ptrs, const int64_t* numels, int32_t n_tensors, int hp_dtype,
                            int fp8_dtype, uint32_t flags, uint32_t* amax_workspace, float* scales_out, void* stream);

/* Saturating cast of x[rows, cols] with one scale for the whole tensor.
 *   scale source: if slots != NULL the scale is reduced from slots[0..n_slots) exactly as
 *   mi8_scale_from_partials does (and written to scale_out[0] if scale_out != NULL);
 *   otherwise, if scale_in != NULL, it is read from scale_in[0] (device float32);
 *   with neither (tensors of at most 65536 elements, row-major output only: the activations of a generation
 *   step) one workgroup takes the amax, derives the scale and converts in a single launch.
 *   out   (may be NULL): fp8 [rows, ld_out], row-major with row pitch ld_out >= cols, ld_out % 16 == 0;
 *                        bytes cols..ld_out-1 of a row are not touched.
 *   out_t (may be NULL): fp8 [cols, ld_t], the transposed copy; ld_t >= rows, ld_t % 16 == 0; columns
 *                        rows..round_up(rows,16)-1 of out_t are written as zero (so that a GEMM may contract
 *                        over round_up(rows,16)), columns beyond are not touched.
 * cols % 16 == 0 is required.  The GEMMs accept any operand pitch that is a multiple of 16. */
int mi8_cast_tensorwise(const void* x, int hp_dtype, int64_t rows, int64_t cols, const uint32_t* slots,
                        int32_t n_slots, const float* scale_in, int fp8_dtype, uint32_t flags, void* out,
                        int64_t ld_out, void* out_t, int64_t ld_t, float* scale_out, void* stream);

/* The dynamic tensorwise cast in one call for callers that cannot allocate device memory or hand over a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): amax pass +
 * cast pass as mi8_amax_partials followed by mi8_cast_tensorwise(slots), with the partial maxima kept in an 8 KiB
 * array that is part of the library's device image (one copy per GPU, held until the process ends) instead of a
 * caller-owned workspace.  No counterpart in the reference.  Same outputs, bytes and scale as the two-call
 * route.  Limits: rows, cols <= MI8_STATIC_CAST_MAX_DIM and rows * cols <= MI8_STATIC_CAST_MAX_ELEMS, larger
 * inputs are refused with MI8_ERR_UNSUPPORTED.  All calls on one GPU share that GPU's array: calls that may
 * overlap on one GPU (different streams, different threads, replays of two captured graphs side by side) race and
 * nothing in the library guards against it; calls ordered on one stream do not.  The first call on a device looks
 * up the array's address (hipGetSymbolAddress, a host-side query that is no stream operation): make one call per
 * device outside of any stream capture before capturing calls into a graph. */
#define MI8_STATIC_CAST_MAX_DIM ((int64_t)1 << 22)
#define MI8_STATIC_CAST_MAX_ELEMS ((int64_t)1 << 32)
int mi8_cast_tensorwise_static(const void* x, int hp_dtype, int64_t rows, int64_t cols, int fp8_dtype, uint32_t flags,
                               void* out, int64_t ld_out, void* out_t, int64_t ld_t, float* scale_out, void* stream);


/* ---------------------------------------------------------------------------------------------
 * Axiswise ("rowwise" recipe) dynamic casts: AXISWISE cast configs of the rowwise recipes
 * (reference: AOFloat8LinearRecipe.rowwise / rowwise_with_gw_hp, src/olmo_core/float8/ao.py:100-109).
 * ------------------------------------------------------------------------------------------- */

/* One scale per row (amax over the last axis): out fp8 [rows, ld_out] (ld_out >= cols, ld_out % 16 == 0),
 * scale_out float32 [rows].  cols % 16 == 0, cols <= 65536. Single pass over x. */
int mi8_cast_rowwise(const void* x, int hp_dtype, int64_t rows, int64_t cols, int fp8_dtype, uint32_t flags,
                     void* out, int64_t ld_out, float* scale_out, void* stream);

/* Number of uint32 a column-amax workspace needs for a [rows, cols] input. */
int64_t mi8_colamax_workspace_slots(int64_t rows, int64_t cols);

/* One scale per column (amax over axis 0), output written TRANSPOSED: out_t fp8 [cols, ld_t] (pad columns
 * rows..round_up(rows,16)-1 zero), scale_out float32 [cols].  This is the operand layout the grad_weight GEMM and the
 * axiswise grad_input GEMM consume.  workspace: mi8_colamax_workspace_slots(rows, cols) uint32.
 * Two kernels: column amax, then cast + transpose. */
int mi8_cast_colwise_t(const void* x, int hp_dtype, int64_t rows, int64_t cols, int fp8_dtype, uint32_t flags,
                       uint32_t* workspace, void* out_t, int64_t ld_t, float* scale_out, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Scaled float8 GEMM.  Stands in for torch._scaled_mm as driven by torchao's float8 mm dispatch
 * (the three GEMMs of one linear: output, grad_input, grad_weight).
 *   out[M, N] = bf16( (sum_k A[m,k] * B[n,k]) * (1/sa) * (1/sb) ), fp32 accumulation on fp8 MFMA.
 *   A: fp8 [M, lda] row-major, B: fp8 [N, ldb] row-major - both operands K-contiguous; K % 16 == 0,
 *   lda, ldb % 16 == 0.  a_dtype / b_dtype may differ (e5m2 x e4m3 for the gradient GEMMs).
 *   sa: quantisation scale(s) of A - one float32 if sa_rows == 0, else float32 [M]; sb likewise ([N]).
 *   out: [M, ldc] of out_dtype (MI8_BF16 or MI8_F32), ldc >= N.
 *   variant: -1 picks a tile configuration from the shape; 0..mi8_gemm_num_variants()-1 forces one.
 * ------------------------------------------------------------------------------------------- */
int mi8_gemm_fp8(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb, int64_t M,
                 int64_t N, int64_t K, const float* sa, int sa_is_vector, const float* sb, int sb_is_vector,
                 void* out, int out_dtype, int64_t ldc, int variant, void* stream);

/* out[M, N] += the product mi8_gemm_fp8 would write: the new term is rounded to out_dtype first and the sum of the
 * two is formed in float32 and rounded once, i.e. exactly what `out = out + gemm(...)` gives when both terms are
 * tensors of out_dtype.  This is how the grad_input of a block whose input feeds two linears (w1 and w3 of the
 * feed-forward block, src/olmo_core/nn/feed_forward.py:171) is summed by autograd; here the second GEMM adds into the
 * first one's output and the separate elementwise pass over [M, N] disappears.  Arguments as mi8_gemm_fp8 (the kernel
 * is chosen by shape). */
int mi8_gemm_fp8_accumulate(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb, int64_t M,
                            int64_t N, int64_t K, const float* sa, int sa_is_vector, const float* sb, int sb_is_vector,
                            void* out, int out_dtype, int64_t ldc, void* stream);

/* The two input projections of a SwiGLU feed-forward block and the activation between them and the output projection
 * in one launch (reference: src/olmo_core/nn/feed_forward.py:171, `self.w2(F.silu(self.w1(x)) * self.w3(x))`):
 *   x1[M, H] = bf16((A . B1^T) / sa / sb1),  x3[M, H] = bf16((A . B3^T) / sa / sb3)   (what mi8_gemm_fp8 writes, bit for bit)
 *   h[M, H]  = silu(x1) * x3                                                          (what mi8_swiglu_fwd writes, bit for bit)
 *   slots_h[0 .. *n_slots_used) = partial maxima of |h| as mi8_swiglu_fwd produces them for the cast of h that follows.
 * Every workgroup computes matching 128-column tiles of x1 and x3 and forms h in its epilogue, so x1 and x3 are written
 * once and never read back.  A fp8 [M, lda]; B1, B3 fp8 [H, ldb] of one type; single scales (float32 [1] each);
 * x1, x3, h bf16 [M, ldc]; slots_h must hold MI8_AMAX_SLOTS uint32.  Needs M >= 256, H >= 128, H % 8 == 0,
 * K % 128 == 0, ldc < 2^22 (MI8_ERR_UNSUPPORTED otherwise: run the three calls it stands for).
 * x_codes: NULL, or uint16[mi8_rowseg_code_count(M, H)] that receives the row-segment codes of the element-wise
 * larger of x1 and x3 (what mi8_rowseg_max_codes(x1, x3) computes; needs H % 64 == 0), for the backward pass's
 * mi8_swiglu_bwd_amax_from_codes. */
int mi8_gemm_fp8_swiglu_matches_separate(int64_t M, int64_t H, int64_t K); /* host only: 1 if the fused launch takes
    the shape and mi8_gemm_fp8 would run both projections on the same tile kernel, so that the bits agree as well */
int mi8_gemm_fp8_swiglu(const void* a, int a_dtype, int64_t lda, const void* b1, const void* b3, int b_dtype, int64_t ldb,
                        int64_t M, int64_t H, int64_t K, const float* sa, const float* sb1, const float* sb3, void* x1,
                        void* x3, void* h, int64_t ldc, uint32_t* slots_h, int32_t* n_slots_used, uint16_t* x_codes,
                        void* stream);

/* The same product with K cut into `splits` slices, for problems whose few output tiles would leave most of the
 * GPU idle (a few hundred rows of A against a weight matrix): every slice is summed by its own workgroups into
 * an fp32 plane of `workspace`, a second kernel adds the planes in slice order (results do not depend on
 * scheduling), applies the scales and rounds.  Arguments as mi8_gemm_fp8; splits in 1..min(64, ceil(K/128));
 * workspace: 16-byte aligned device memory of mi8_gemm_splitk_workspace_bytes(M, N, splits) bytes, owned by the
 * caller, free for reuse once the call's work on `stream` is done.  mi8_gemm_splitk_suggest returns the number
 * of slices the library would use for a shape (1: call mi8_gemm_fp8 instead).  No counterpart upstream: the
 * reference leaves the choice of GEMM algorithm to torch._scaled_mm's backend. */
int mi8_gemm_fp8_splitk(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                        int64_t M, int64_t N, int64_t K, const float* sa, int sa_is_vector, const float* sb,
                        int sb_is_vector, void* out, int out_dtype, int64_t ldc, int splits, void* workspace,
                        int64_t workspace_bytes, void* stream);
int mi8_gemm_splitk_suggest(int64_t M, int64_t N, int64_t K);
int64_t mi8_gemm_splitk_workspace_bytes(int64_t M, int64_t N, int splits);

/* Number of GEMM kernel variants compiled in (variant ids 0..n-1; -1 lets the library choose by shape). */
int mi8_gemm_num_variants(void);
const char* mi8_gemm_variant_name(int variant);

/* ---------------------------------------------------------------------------------------------
 * Ragged grouped operations for the dropless-MoE expert layer.  The reference runs this layer in bf16 through
 * grouped_gemm.ops.gmm(x, w, batch_sizes, trans_b) or a per-expert loop (src/olmo_core/nn/moe/mlp.py:256-270);
 * these entry points are its float8 counterpart with the axiswise recipe applied to every expert's slice
 * independently.  Rows of the activation matrix form consecutive groups; group_sizes is an int64 device array
 * (as DroplessMoEMLP.forward receives it, mlp.py:272-280) that is never copied to the host.
 * ------------------------------------------------------------------------------------------- */

/* Upper bound of the padded token axis used by the grouped transposed layouts: every group's segment starts at a
 * multiple of 128 (T rounded up to 128, plus 128 per group after the first). */
int64_t mi8_grouped_padded_rows(int64_t T, int32_t num_groups);

/* Per-group, per-column dynamic cast with transposed output: for group e (rows R_e of x[T, cols]) the scale of
 * column c is taken over R_e only; out_t[c, 128 * tiles_before(e) + (r - first row of e)] holds the bytes, the
 * rest of each 128-aligned segment is zero.  amax_ws: uint32 [num_groups * cols], ZERO on entry.
 * scale_out: float32 [num_groups, cols] (rows of empty groups are not written).
 * ld_t >= mi8_grouped_padded_rows(T, num_groups), ld_t % 16 == 0.  With equal group sizes that are multiples of
 * 128 this is a batched transpose-cast (used for the expert weights). */
int mi8_grouped_cast_colwise_t(const void* x, int hp_dtype, int64_t T, int64_t cols, const int64_t* group_sizes,
                               int32_t num_groups, int fp8_dtype, uint32_t flags, uint32_t* amax_ws, void* out_t,
                               int64_t ld_t, float* scale_out, void* stream);

/* The same two passes (amax, cast) also produce the per-row cast of x that the forward / grad_input GEMMs take:
 * out_rows fp8 [T, ld_rows] row-major with one scale per row (row_scale_out float32 [T], the values
 * mi8_cast_rowwise gives), saving the separate pass over x.  row_amax_ws: uint32 [T], ZERO on entry.  Both
 * products use fp8_dtype and flags.  Rows beyond the last group (if the sizes sum to less than T) are not
 * written. */
int mi8_grouped_cast_rows_and_colwise_t(const void* x, int hp_dtype, int64_t T, int64_t cols,
                                        const int64_t* group_sizes, int32_t num_groups, int fp8_dtype, uint32_t flags,
                                        uint32_t* amax_ws, void* out_t, int64_t ld_t, float* scale_out,
                                        uint32_t* row_amax_ws, void* out_rows, int64_t ld_rows, float* row_scale_out,
                                        void* stream);

/* h = silu(x1) * x2 of the expert layer (src/olmo_core/nn/moe/mlp.py:286-291; bf16 [T, cols], the rounding points
 * of mi8_swiglu_fwd) together with the amax pass of the cast that follows: amax_ws (uint32 [num_groups * cols]) and
 * row_amax_ws (uint32 [T]), both ZERO on entry, receive the per-(group, column) and per-row amax of h, so that
 * mi8_grouped_cast_rows_and_colwise_t(h, ..., flags | MI8_FLAG_AMAX_READY, ...) skips its own first pass.  Rows
 * beyond the last group are not written.  The backward form writes the gradients g1 (of x1) and g2 (of x2) of that
 * product for the incoming gradient gh, each with its own pair of amax workspaces. */
int mi8_grouped_swiglu_fwd(const void* x1, const void* x2, int64_t T, int64_t cols, const int64_t* group_sizes,
                           int32_t num_groups, void* h, uint32_t* amax_ws, uint32_t* row_amax_ws, void* stream);
int mi8_grouped_swiglu_bwd(const void* x1, const void* x2, const void* gh, int64_t T, int64_t cols,
                           const int64_t* group_sizes, int32_t num_groups, void* g1, void* g2, uint32_t* amax_ws1,
                           uint32_t* row_amax_ws1, uint32_t* amax_ws2, uint32_t* row_amax_ws2, void* stream);

/* out[R_e, :N] = (A[R_e, :K] . B_e[:N, :K]^T) / sa[r] / sb_e[n]   for every group e.
 *   A fp8 [T, lda]; B_e = b + e * b_group_stride (bytes), N rows of pitch ldb; sa float32 [T];
 *   sb_e = sb + e * sb_group_stride (floats), N values; out [T, ldc] of out_dtype. */
int mi8_grouped_gemm_fp8(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                         int64_t b_group_stride, const int64_t* group_sizes, int32_t num_groups, int64_t T, int64_t N,
                         int64_t K, const float* sa, const float* sb, int64_t sb_group_stride, void* out,
                         int out_dtype, int64_t ldc, void* stream);

/* out[R_e, :N] += that product, summed as mi8_gemm_fp8_accumulate does (the two grad_input terms of the expert
 * layer, src/olmo_core/nn/moe/mlp.py:286-291). */
int mi8_grouped_gemm_fp8_accumulate(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb,
                                    int64_t b_group_stride, const int64_t* group_sizes, int32_t num_groups, int64_t T,
                                    int64_t N, int64_t K, const float* sa, const float* sb, int64_t sb_group_stride,
                                    void* out, int out_dtype, int64_t ldc, void* stream);

/* out[rows of group e, :N] = (a1 . B1_e^T) / sa1 / sb1_e + (a2 . B2_e^T) / sa2 / sb2_e, both products summed in one
 * float32 accumulation and rounded once to bf16: the grad_input of an expert layer whose input feeds two projections
 * (gx = g1 . W1 + g2 . W3, src/olmo_core/nn/moe/mlp.py:272-292 in backward) as one launch instead of
 * mi8_grouped_gemm_fp8 + mi8_grouped_gemm_fp8_accumulate, without the read-modify-write of the output.  a1 [T, K1] and
 * a2 [T, K2] share the row pitch lda; B1_e [N, K1] and B2_e [N, K2] the row pitch ldb and the group stride; sa1, sa2:
 * float32 [T]; sb1, sb2: float32, group e at + e * sb_group_stride, N values.  EVERY SCALE MUST BE AN EXACT POWER OF TWO
 * (what the casts write under MI8_FLAG_POW2_SCALE): the scales are applied inside the matrix instructions as exponents,
 * a mantissa is ignored.  The sum differs from the two-call route by one rounding (that route rounds each product to bf16
 * before adding).  Shapes: mi8_grouped_gemm_fp8_dual_supported (T, N >= 256, N % 8 == 0, K1 and K2 multiples of 256);
 * out: bf16 [T, ldc], ldc % 8 == 0. */
int mi8_grouped_gemm_fp8_dual_supported(int64_t T, int64_t N, int64_t K1, int64_t K2);
int mi8_grouped_gemm_fp8_dual(const void* a1, const void* a2, int a_dtype, int64_t lda, const void* b1, const void* b2,
                              int b_dtype, int64_t ldb, int64_t b_group_stride, const int64_t* group_sizes,
                              int32_t num_groups, int64_t T, int64_t N, int64_t K1, int64_t K2, const float* sa1,
                              const float* sa2, const float* sb1, const float* sb2, int64_t sb_group_stride, void* out,
                              int64_t ldc, void* stream);

/* out[e, :N, :Kl] = (A_t[:N, S_e] . B_t[:Kl, S_e]^T) / sa[e, n] / sb[e, k]: the contraction runs over group e's
 * 128-aligned segment S_e of the padded token axis (layout written by mi8_grouped_cast_colwise_t; both operands
 * have pitch ld_t).  Empty groups produce zeros.  out is [num_groups, N, Kl] contiguous. */
int mi8_grouped_wgrad_fp8(const void* a_t, int a_dtype, const void* b_t, int b_dtype, int64_t ld_t,
                          const int64_t* group_sizes, int32_t num_groups, int64_t T, int64_t N, int64_t Kl,
                          const float* sa, const float* sb, void* out, int out_dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * SwiGLU pointwise kernels between the projections of the feed-forward block
 * (reference: src/olmo_core/nn/feed_forward.py:171  w2(silu(w1 x) * w3 x)).
 *   forward : h = bf16(bf16(silu(x1)) * x3), optionally also the amax partials of h.
 *   backward: given gh, g1 = gh * x3 * silu'(x1), g3 = gh * silu(x1), evaluated with bf16 roundings of
 *             torch's elementwise autograd formulas; optionally amax partials of g1 and g3.
 * All tensors bf16, n elements, n % 8 == 0.
 * ------------------------------------------------------------------------------------------- */
int mi8_swiglu_fwd(const void* x1, const void* x3, void* h, int64_t n, uint32_t* slots_h, void* stream);
int mi8_swiglu_bwd(const void* x1, const void* x3, const void* gh, void* g1, void* g3, int64_t n,
                   uint32_t* slots_g1, uint32_t* slots_g3, void* stream);

/* The feed-forward block's backward needs g1 and g3 only as fp8 operands.  Two passes that never write them in bf16:
 * mi8_swiglu_bwd with g1 = g3 = NULL leaves just the amax partials of what it would have written; this entry point
 * then recomputes the gradients tile by tile and writes the tensorwise casts of both (row-major [rows, ld_out]
 * and/or transposed [cols, ld_t] copies, the layouts of mi8_cast_tensorwise; the same layouts for both outputs) with
 * the scales taken from those partials.  Bytes and scales equal mi8_swiglu_bwd + mi8_cast_tensorwise on each output. */
int mi8_swiglu_bwd_cast(const void* x1, const void* x3, const void* gh, int64_t rows, int64_t cols,
                        const uint32_t* slots_g1, const uint32_t* slots_g3, int32_t n_slots, int fp8_dtype, uint32_t flags,
                        void* out1, void* out3, int64_t ld_out, void* out1_t, void* out3_t, int64_t ld_t,
                        float* scale_out1, float* scale_out3, void* stream);

/* The amax of g1 and g3 without computing every element (the tensorwise scale of the gradient operands,
 * torchao tensor_to_amax over what src/olmo_core/nn/feed_forward.py:171 back-propagates).
 *
 * A row segment is 64 consecutive columns of a row (the last one of a row may be shorter).  Its code is the largest
 * magnitude in it as a 16-bit integer: the exponent and mantissa bits of the bf16 value, which grow with the
 * magnitude and add like logarithms.  codes = uint16[mi8_rowseg_code_count(rows, cols)], segment (r, c / 64) at
 * index (c / 64) * rows + r.  mi8_rowseg_max_codes computes them for one tensor, or for the element-wise larger of
 * two (b may be NULL); mi8_gemm_fp8_codes and mi8_gemm_fp8_swiglu write them for the tensors they produce.
 *
 * The sum of a segment's codes in gh and in (x1, x3) bounds log2 of both gradients on all its elements.
 * mi8_swiglu_bwd_amax_from_codes computes exactly only the segments whose bound could still raise the maxima (all
 * segments that may hold a non-finite input among them) and leaves state[0] = amax bits of g1, state[1] = of g3
 * (float32 bit patterns, the values mi8_swiglu_bwd's partials reduce to; pass them to mi8_swiglu_bwd_cast with
 * n_slots = 1); state is uint32[mi8_swiglu_amax_state_words(rows, cols)], overwritten (nothing to clear beforehand).
 * Tensors are bf16 [rows, cols] contiguous, cols % 8 == 0; the code arrays 16-byte aligned. */
int64_t mi8_rowseg_code_count(int64_t rows, int64_t cols);
int64_t mi8_swiglu_amax_state_words(int64_t rows, int64_t cols);
int mi8_rowseg_max_codes(const void* a, const void* b, int64_t rows, int64_t cols, uint16_t* codes, void* stream);
int mi8_swiglu_bwd_amax_from_codes(const void* x1, const void* x3, const void* gh, int64_t rows, int64_t cols,
                                   const uint16_t* gh_codes, const uint16_t* x_codes, uint32_t* state, void* stream);
/* out = mi8_gemm_fp8(a, b) for single scales and a bf16 output, with the row-segment codes of out written by the
 * epilogue (the gradient reaching h = silu(x1) * x3, grad_h = grad_y W2 of src/olmo_core/nn/feed_forward.py:171, is
 * produced this way).  mi8_gemm_fp8_codes_supported: shapes it takes (those mi8_gemm_fp8 runs on the same kernel, so
 * out has the same bits; N % 64 == 0; ldc < 2^22). */
int mi8_gemm_fp8_codes_supported(int64_t M, int64_t N, int64_t K);
int mi8_gemm_fp8_codes(const void* a, int a_dtype, int64_t lda, const void* b, int b_dtype, int64_t ldb, int64_t M, int64_t N,
                       int64_t K, const float* sa, const float* sb, void* out, int64_t ldc, uint16_t* codes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Token permutation around the expert GEMMs of a mixture-of-experts layer.  These replace the copy kernels of
 * src/olmo_core/kernels/moe.py (gather :101-139, padded_scatter / scatter :142-192, scatter_wgrad :251-298,
 * binned_gather :377-406, binned_scatter :409-441, binned_scatter_wgrad :512-537), which the autograd functions
 * of src/olmo_core/ops/moe.py:26-205 call.
 *
 *   tokens, hidden : x is [tokens, hidden]; every token has top_k slots, slot s belongs to token s / top_k.
 *   indices        : int32 [tokens * top_k], the slot held by each row of the expert-sorted side
 *                    (argsort of the flattened expert assignment, ops/moe.py / parallel_mlp.py:102-125).
 *   weights        : [tokens * top_k] of w_dtype (MI8_BF16 / MI8_F16 / MI8_F32) indexed by slot, or NULL.
 *   bins           : int32 [experts], inclusive prefix sums of the tokens per expert (binned forms).
 * Products are formed in float32 and rounded once to the element type, as the reference kernels do.  Rows are
 * moved with 16-byte accesses when hidden * element size is a multiple of 16 and the buffers are 16-byte
 * aligned, element by element otherwise.  An index outside [0, tokens * top_k) is treated as a dropped token.
 * ------------------------------------------------------------------------------------------- */

/* out[i, :] = x[indices[i] / top_k, :] * weights[indices[i]]           out: [tokens * top_k, hidden] */
int mi8_moe_gather(const void* x, int dtype, int64_t tokens, int64_t hidden, const int32_t* indices,
                   const void* weights, int w_dtype, int32_t top_k, void* out, void* stream);

/* mi8_moe_gather (weights NULL: unweighted) followed by mi8_grouped_cast_rows_and_colwise_t, without the gathered high-precision
 * tensor in between: the token rows are read through `indices` in both passes (x stays cache resident: every token
 * row is read top_k times), and only the float8 products are written - the per-row cast [tokens * top_k, ld_rows]
 * with its scales and the per-(group, column) transposed cast with its scales, i.e. the operands of the expert
 * GEMMs of a dropless mixture-of-experts layer (the copy kernel of src/olmo_core/kernels/moe.py:42-139 fused with the
 * quantisation that follows it in a float8 expert layer; its backward stays mi8_moe_scatter).  With weights (the
 * backward of the weighted scatter: grad_output rows times the router weight of the slot) every product is rounded to
 * the element type before it is quantised, as mi8_moe_gather writes it.  A slot index outside
 * [0, tokens * top_k) reads as a row of zeros.  Workspaces, outputs and group semantics as
 * mi8_grouped_cast_rows_and_colwise_t with T = tokens * top_k; bytes and scales equal the two-call route. */
int mi8_moe_gather_cast_rows_and_colwise_t(const void* x, int hp_dtype, int64_t tokens, int64_t cols,
                                           const int32_t* indices, int32_t top_k, const void* weights, int w_dtype,
                                           const int64_t* group_sizes,
                                           int32_t num_groups, int fp8_dtype, uint32_t flags, uint32_t* amax_ws,
                                           void* out_t, int64_t ld_t, float* scale_out, uint32_t* row_amax_ws,
                                           void* out_rows, int64_t ld_rows, float* row_scale_out, void* stream);

/* out[e, j, :] = the j-th token row of expert e (scaled), zero rows beyond the expert's token count; tokens
 * beyond `capacity` are dropped.                                          out: [experts, capacity, hidden] */
int mi8_moe_binned_gather(const void* x, int dtype, int64_t tokens, int64_t hidden, const int32_t* indices,
                          const void* weights, int w_dtype, const int32_t* bins, int32_t experts, int64_t capacity,
                          int32_t top_k, void* out, void* stream);

/* out[t, :] = sum over the top_k slots s of token t of round(x[row holding s, :] * weights[s]), summed in float32
 * in slot order and rounded once (top_k == 1: a pure move).  x: [tokens * top_k, hidden], out: [tokens, hidden].
 * inverse_workspace: int32 [tokens * top_k], overwritten. */
int mi8_moe_scatter(const void* x, int dtype, int64_t tokens, int64_t hidden, const int32_t* indices,
                    const void* weights, int w_dtype, int32_t top_k, int32_t* inverse_workspace, void* out,
                    void* stream);

/* The same from the binned layout x: [experts, capacity, hidden]; dropped tokens contribute zero. */
int mi8_moe_binned_scatter(const void* x, int dtype, int64_t tokens, int64_t hidden, const int32_t* indices,
                           const void* weights, int w_dtype, const int32_t* bins, int32_t experts, int64_t capacity,
                           int32_t top_k, int32_t* inverse_workspace, void* out, void* stream);

/* Gradient of the scatter weights: out[indices[i]] = dot(x[i, :], grad[indices[i] / top_k, :]) accumulated in
 * float32.  x: [tokens * top_k, hidden], grad: [tokens, hidden], out: [tokens * top_k] of dtype. */
int mi8_moe_scatter_wgrad(const void* x, const void* grad, int dtype, int64_t tokens, int64_t hidden,
                          const int32_t* indices, int32_t top_k, void* out, void* stream);

/* The same from the binned layout; slots of dropped tokens get zero. */
int mi8_moe_binned_scatter_wgrad(const void* x, const void* grad, int dtype, int64_t tokens, int64_t hidden,
                                 const int32_t* indices, const int32_t* bins, int32_t experts, int64_t capacity,
                                 int32_t top_k, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI8_H */
