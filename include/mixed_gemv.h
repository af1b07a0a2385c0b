/*
 * mixed_gemv.h — C-ABI of the MI355X (gfx950) weight-only-quantised GEMV library.
 *
 *     y[b][n] = fp16( sum_k dequant(W)[n][k] * x[b][k]  (+ bias[n]) )
 *
 * int4 or int8 weights, fp16 (or, in the _bf16 entry points, bfloat16) activations, fp32
 * accumulation, output in the activation type.  The entry
 * points below are what a binding of JJXiangJiaoJun/mixed_gemv's C++ call sites needs; each
 * one names the reference interface it stands in for.  Dimension names follow the model
 * view: n_out = output features (the reference's M), k = reduction length, m_batch =
 * activation rows (the reference's N, fixed to 1 there).
 *
 * Conventions
 *   - fp16 values cross the ABI as uint16_t bit patterns (IEEE-754 binary16).
 *   - Functions taking a `stream` work on DEVICE pointers, enqueue asynchronously on that
 *     HIP stream (NULL = the null stream), never allocate and never synchronise.
 *   - Functions without a `stream` are host utilities working on HOST pointers.
 *   - Every function returns an mgemv_status; none prints or calls exit().  The conditions
 *     on which the reference prints a message and exits are reported as error codes.
 *   - The library keeps no per-call state: calls from several host threads on different
 *     streams are safe.
 */
#ifndef MIXED_GEMV_H_
#define MIXED_GEMV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(MGEMV_BUILDING_LIBRARY)
#define MGEMV_API __attribute__((visibility("default")))
#else
#define MGEMV_API
#endif

/* Status codes. */
typedef enum mgemv_status {
  MGEMV_OK = 0,
  MGEMV_ERR_NULL_POINTER = 1,   /* a required pointer is NULL */
  MGEMV_ERR_RANK = 2,           /* shape rank not 2 or 3 (utils/preprocess.h:486-489) */
  MGEMV_ERR_ROWS = 3,           /* n_out not a multiple of 4 (utils/preprocess.h:319-322) */
  MGEMV_ERR_COLS = 4,           /* k not a multiple of 8 (utils/preprocess.h:324-327) */
  MGEMV_ERR_GROUP_SIZE = 5,     /* group_size < 64 (gemv/device/gemv_adaptor.h:199-203), not a multiple of 32, or not dividing k */
  MGEMV_ERR_QUANT_OP = 6,       /* quant_op not 1, 2 or 3 (gemv/weight_only_quant_op.h:12-18) */
  MGEMV_ERR_QUANT_TYPE = 7,     /* weight type not W8_A16 / W4_A16 (utils/preprocess.h:110, 287-288) */
  MGEMV_ERR_BATCH = 8,          /* batch_count < 1 or m_batch outside [1, MGEMV_MAX_M_BATCH] */
  MGEMV_ERR_LAYOUT = 9,         /* layout flag not row/column major (utils/preprocess.h:486-489; the reference's further
                                   demand that a row-major matrix have dimensions of whole 64-element tiles,
                                   utils/preprocess.h:157-162, does not apply: any legal n_out, k is transposed) */
  MGEMV_ERR_SIZE = 10,          /* a dimension is <= 0 or overflows the 32-bit index space of the kernels */
  MGEMV_ERR_LAUNCH = 11,        /* the HIP runtime refused the launch (gemv/device/gemv_adaptor.h:249-254) */
  MGEMV_ERR_NO_DEVICE = 12,     /* the stream's device (the current device for the null stream) is not a gfx950 */
  MGEMV_ERR_ALIGNMENT = 13,     /* a device pointer is not aligned as required: weights and activations 16 bytes (and
                                   the batch strides to match); scales, zeros, bias, outputs 2 bytes; the output of
                                   mgemv_dequantize 4 bytes */
  MGEMV_ERR_LEADING_DIMENSION = 14, /* mgemv_gemv_arguments: a leading dimension other than the dense one */
  MGEMV_ERR_ALLOCATION = 15,    /* mgemv_host_gemv: device memory could not be allocated */
  MGEMV_ERR_SCRATCH_SIZE = 16   /* mgemv_host_gemv_static: the problem needs more than MGEMV_STATIC_SCRATCH_BYTES */
} mgemv_status;

/* gemv/weight_only_quant_op.h:12-18 — same numeric values. */
enum {
  MGEMV_PER_COLUMN_SCALE_ONLY = 1,
  MGEMV_FINEGRAINED_SCALE_ONLY = 2,
  MGEMV_FINEGRAINED_SCALE_AND_ZEROS = 3
};

/* utils/type_base.h:7-11 — same numeric values (W4_AFP8 = 2 has no kernel in the reference and none here). */
enum { MGEMV_W8_A16 = 0, MGEMV_W4_A16 = 1 };

/* utils/type_base.h:13-16 — same numeric values. */
enum { MGEMV_ROW_MAJOR = 0, MGEMV_COLUMN_MAJOR = 1 };

#define MGEMV_MAX_M_BATCH 16

/* Human-readable text for a status code (never NULL). */
MGEMV_API const char *mgemv_status_string(int status);

/* Library version, major*10000 + minor*100 + patch. */
MGEMV_API int mgemv_version(void);

/* ------------------------------------------------------------------------------------------
 * Host utilities
 * ---------------------------------------------------------------------------------------- */

/* Replaces SubBytePacker<int4b_t,int8_t>::pack (utils/preprocess.h:55-84).
 * Packs n_unpacked signed 4-bit values held one per int8 into n_unpacked/2 bytes (an odd
 * n_unpacked is MGEMV_ERR_SIZE):
 * element 2i in bits 0..3 of byte i, element 2i+1 in bits 4..7.  Values are truncated to
 * their low 4 bits, as in the reference. */
MGEMV_API int mgemv_pack_int4(uint8_t *packed, const int8_t *unpacked, size_t n_unpacked);

/* Replaces SubBytePacker<int4b_t,int8_t>::unpack (utils/preprocess.h:41-53): sign-extending inverse. */
MGEMV_API int mgemv_unpack_int4(int8_t *unpacked, const uint8_t *packed, size_t n_packed);

/* Replaces ZeroPointPreprocessor<half_t,int8_t>::neg_zero_point_multiplies_scale
 * (utils/preprocess.h:94-101): out[i] = fp16(-zeros[i]) * scales[i], one fp16 multiply.
 * The result is the additive term the GEMV takes as `zero_add` (mixed_gemv_test.cu:237-239, 275). */
MGEMV_API int mgemv_fold_zero_points(uint16_t *out, const uint16_t *scales, const int8_t *zeros, size_t n);

/* Bytes that mgemv_preprocess_weights writes for this shape (>= the input size: rows are
 * padded to 16 and k to one wave step).  shape as in mgemv_preprocess_weights.  Returns 0
 * for an invalid rank / quant_type. */
MGEMV_API size_t mgemv_preprocessed_size(const size_t *shape, int rank, int quant_type);

/* Replaces MixedGemvWeightPreprocessor::run (utils/preprocess.h:482-522).
 *   src     quantised weights: int4 packed two per byte (low nibble = even element) or int8.
 *   shape   {k, n_out} or {experts, k, n_out}, exactly the reference's `shape` argument.
 *   layout  MGEMV_COLUMN_MAJOR: memory is n_out rows of k elements (the reference's shipped
 *           call, mixed_gemv_test.cu:247-254); MGEMV_ROW_MAJOR: memory is k rows of n_out
 *           elements and is transposed first (utils/preprocess.h:507-511).
 *   quant_type MGEMV_W4_A16 or MGEMV_W8_A16 (the reference's interleave rejects W8_A16,
 *           utils/preprocess.h:350-362; here both are laid out).
 * Same input meaning as the reference, different OUTPUT layout: the gfx950 tile layout
 * consumed by mgemv_gemv (16-row tiles, 1 KiB wave-contiguous blocks, biased 4-bit fields at
 * the bit positions the dequantiser masks out directly).  The layout belongs to this library
 * version (mgemv_version).  dst must hold mgemv_preprocessed_size() bytes and may not alias src. */
MGEMV_API int mgemv_preprocess_weights(uint8_t *dst, const uint8_t *src, const size_t *shape, int rank,
                                       int layout, int quant_type);

/* Inverse of mgemv_preprocess_weights for MGEMV_COLUMN_MAJOR input: recovers the n_out x k
 * row-major quantised weights from a preprocessed buffer.  No counterpart in the reference;
 * it exists so that layouts can be audited and round-trip tested. */
MGEMV_API int mgemv_unpreprocess_weights(uint8_t *dst, const uint8_t *src_preprocessed, const size_t *shape,
                                         int rank, int quant_type);

/* ------------------------------------------------------------------------------------------
 * Device entry points
 * ---------------------------------------------------------------------------------------- */

/* Replaces device_gemv (mixed_gemv_test.cu:124-165) and GemvAdaptor::initialize + run
 * (gemv/device/gemv_adaptor.h:198-255) for batch_count == 1.
 *   weights   preprocessed weights (device), output of mgemv_preprocess_weights
 *   x         activations, m_batch rows of k fp16, row stride k   (reference ref_B, ldb = 0 for its single row)
 *   scale     fp16 [k/group_size][n_out], n_out contiguous (reference ref_scale, ld = n_out);
 *             per-column mode: [n_out]
 *   zero_add  fp16 additive term -z*s, same shape as scale; read only in mode 3
 *             (mixed_gemv_test.cu:145-147), may be NULL otherwise
 *   bias      fp16 [n_out] added in fp32 before the final rounding, or NULL
 *             (reference ref_C with a source-enabled epilogue, epilogue/threadblock/epilogue.h:50-75)
 *   y         fp16 output, m_batch rows of n_out, row stride n_out (reference ref_D, ldd = n_out)
 *   group_size ignored (taken as k) in per-column mode (mixed_gemv_test.cu:142-143)
 *   quant_op  MGEMV_PER_COLUMN_SCALE_ONLY / _FINEGRAINED_SCALE_ONLY / _FINEGRAINED_SCALE_AND_ZEROS,
 *             a run-time argument here, a template parameter in the reference
 *   weight_bits 4 or 8
 * Dequantisation is fp16 multiply then fp16 add, separately rounded
 * (gemv/warp/warp_dequantizer.h:52-59), accumulation is fp32. */
MGEMV_API int mgemv_gemv(const void *weights, const uint16_t *x, const uint16_t *scale, const uint16_t *zero_add,
                         const uint16_t *bias, uint16_t *y, int n_out, int m_batch, int k, int group_size,
                         int quant_op, int weight_bits, void *stream);

/* As mgemv_gemv, with the reference's batch arguments (gemv/device/gemv_adaptor.h:129-135;
 * gemv/kernel/mixed_gemv.h:140-149, 222-223): batch_count independent problems, operand
 * pointers advanced per problem by the given strides.  stride_weights is in BYTES of the
 * preprocessed buffer (mgemv_preprocessed_size of one matrix for expert-stacked weights);
 * the other strides are in fp16 elements; stride_scale applies to scale and zero_add,
 * stride_bias to bias.  A stride of 0 shares the operand between problems. */
MGEMV_API int mgemv_gemv_batched(const void *weights, const uint16_t *x, const uint16_t *scale,
                                 const uint16_t *zero_add, const uint16_t *bias, uint16_t *y, int batch_count,
                                 int n_out, int m_batch, int k, int group_size, int quant_op, int weight_bits,
                                 int64_t stride_weights, int64_t stride_x, int64_t stride_scale,
                                 int64_t stride_bias, int64_t stride_y, void *stream);

/* Routed launch over a stack of matrices -- the use that the 3-D, expert-stacked shapes of the
 * reference's preprocessor are for (utils/preprocess.h:134-136, 315-317).  The reference has no
 * such launch: its batch arguments step through a stack at a fixed stride
 * (gemv/kernel/mixed_gemv.h:140-149), so a decode step that wants the top-k experts of a token
 * would need one launch per expert.  As mgemv_gemv_batched, except that problem b takes the
 * weights, scales, zeros and bias of entry route[b] of the stack (their strides are multiplied by
 * route[b]), while x and y are still stepped by b (stride_x = 0: one token and its chosen
 * experts).  route is a DEVICE array of batch_count 32-bit indices, read by the kernel, so a
 * router's output is used where it lies, with no copy to the host; route_extent is the number of
 * entries in the stack.  A problem whose index lies outside [0, route_extent) is skipped, its
 * outputs are left as they were (the host cannot check device data without a synchronisation, and
 * an unchecked index would be a read outside the stack).  Results are those of
 * mgemv_gemv_batched on the same matrices, bit for bit. */
MGEMV_API int mgemv_gemv_routed(const void *weights, const uint16_t *x, const uint16_t *scale,
                                const uint16_t *zero_add, const uint16_t *bias, uint16_t *y, const int32_t *route,
                                int route_extent, int batch_count, int n_out, int m_batch, int k, int group_size,
                                int quant_op, int weight_bits, int64_t stride_weights, int64_t stride_x,
                                int64_t stride_scale, int64_t stride_bias, int64_t stride_y, void *stream);

/* GemvAdaptor::Arguments (gemv/device/gemv_adaptor.h:114-178) as a plain struct, and
 * GemvAdaptor::operator()(args, stream) (:258-261) as one call: everything mgemv_gemv_batched
 * takes, plus the epilogue's alpha and beta and the leading dimensions of the reference's
 * TensorRefs.  y = element( alpha * acc + beta * bias ), computed in fp32 with the outer
 * multiply-add fused (the reference's LinearCombination, mixed_gemv_test.cu:72-81;
 * epilogue/threadblock/epilogue.h:64, 93); bias == NULL drops the term.  alpha = beta = 1 is
 * mgemv_gemv_batched bit for bit.  The operands are dense: a leading dimension must be 0
 * ("dense") or the value the reference's caller passes for that operand -- lda 4*k (or k), ldb k
 * (0 is also accepted for m_batch == 1, mixed_gemv_test.cu:137), ld_scale / ld_zero / ldc / ldd
 * n_out (mixed_gemv_test.cu:136-140, 153-154) -- anything else is MGEMV_ERR_LEADING_DIMENSION,
 * never a silently different result.  Batch strides as in mgemv_gemv_batched. */
enum { MGEMV_ELEMENT_F16 = 0, MGEMV_ELEMENT_BF16 = 1 };
typedef struct mgemv_arguments {
  int n_out, m_batch, k;                    /* problem_size: the reference's (M, N, K) */
  const void *weights; int64_t lda;         /* ref_A: preprocessed weights */
  const uint16_t *x; int64_t ldb;           /* ref_B */
  const uint16_t *scale; int64_t ld_scale;  /* ref_scale */
  const uint16_t *zero_add; int64_t ld_zero;/* ref_zero_point: the folded additive term */
  const uint16_t *bias; int64_t ldc;        /* ref_C */
  uint16_t *y; int64_t ldd;                 /* ref_D */
  float alpha, beta;                        /* epilogue */
  int group_size, batch_count;
  int64_t batch_stride_weights, batch_stride_x, batch_stride_scale, batch_stride_bias, batch_stride_y;
  int quant_op, weight_bits;                /* template parameters in the reference */
  int element;                              /* MGEMV_ELEMENT_F16 / _BF16: ElementB = ElementScale = ElementOutput */
} mgemv_arguments;
MGEMV_API int mgemv_gemv_arguments(const mgemv_arguments *args, void *stream);

/* host::reference::MixedGemv::operator() (host/mixed_gemv.h:60-70) with the GPU behind it: the
 * same argument list and meaning -- HOST pointers, `weights` the UN-preprocessed quantised
 * matrix ([n_out][k] row-major; int4 packed two per byte as utils/vector_subbyte.h:150-156 lays
 * them out, or int8), `zero_point` the int8 zero points [k/group_size][n_out] (not folded; read
 * only in mode 3), `bias` may be NULL -- so a caller of the reference's HOST_CHECK path can be
 * pointed at the device without touching its data.  Preprocesses, folds the zero points
 * (utils/preprocess.h:94-101), uploads, runs mgemv_gemv on the null stream of the current
 * device and downloads; synchronous.  Unlike every other device entry point it ALLOCATES (one
 * hipMalloc / hipFree per call): a convenience and parity entry, not a hot path.  Beyond the
 * reference (which exits unless N == 1, :72-75) m_batch up to 16 rows is accepted; batch must be
 * 1 (:77-80).  quant_op and weight_bits are template parameters in the reference, which only
 * instantiates int4 with zero points (:23-42). */
MGEMV_API int mgemv_host_gemv(int batch, int n_out, int m_batch, int k, int group_size, const uint8_t *weights,
                              const uint16_t *x, const uint16_t *scale, const int8_t *zero_point,
                              const uint16_t *bias, uint16_t *y, int quant_op, int weight_bits);

/* mgemv_host_gemv without any allocation.  It has no counterpart in the reference; it is for
 * callers that cannot allocate device memory where they call from -- harnesses that forbid
 * hipMalloc, tight serving loops -- and still want the HOST_CHECK-shaped call.  Same arguments,
 * same results bit for bit.  The device staging that mgemv_host_gemv allocates per call
 * (preprocessed weights, folded zeros, activations, tables, bias, outputs; 256-byte aligned
 * pieces) lives in a static device array of MGEMV_STATIC_SCRATCH_BYTES that every GPU the library
 * runs on holds until the process ends, and the host-side temporaries in a static host array of
 * the same size: no hipMalloc, hipFree or heap allocation on this path.  A problem whose pieces do
 * not fit returns MGEMV_ERR_SCRATCH_SIZE (mgemv_static_scratch_bytes_needed tells beforehand).
 * All calls in a process share the arrays (each GPU its own device copy, all of them the one
 * host array) and are serialised by a lock inside the library; the arrays keep the previous
 * call's contents, which the next call overwrites as far as it reads them.  Synchronous, null
 * stream of the current device. */
#define MGEMV_STATIC_SCRATCH_BYTES (16u << 20)
MGEMV_API int mgemv_host_gemv_static(int batch, int n_out, int m_batch, int k, int group_size, const uint8_t *weights,
                                     const uint16_t *x, const uint16_t *scale, const int8_t *zero_point,
                                     const uint16_t *bias, uint16_t *y, int quant_op, int weight_bits);
/* Bytes of the static arrays such a call would use (0 if the arguments are not a legal problem). */
MGEMV_API size_t mgemv_static_scratch_bytes_needed(int n_out, int m_batch, int k, int group_size, int quant_op,
                                                   int weight_bits, int has_bias);

/* Parity/debug entry: writes the dequantised weights, fp16 [n_out][k] row-major, produced by
 * the SAME device conversion and dequantisation code the GEMV kernels use
 * (gemv/interleaved_numeric_conversion.h:62-81, 232-291 then gemv/warp/warp_dequantizer.h:52-59, 86-92).
 * No direct counterpart in the reference, where this value only exists in registers. */
MGEMV_API int mgemv_dequantize(const void *weights, const uint16_t *scale, const uint16_t *zero_add,
                               uint16_t *out, int n_out, int k, int group_size, int quant_op, int weight_bits,
                               void *stream);

/* Launch geometry override for tuning and tests: k-split waves per tile, tile sequences per
 * workgroup, tiles handled by one wave of the matrix-core kernel (1, 2 or 4), and the largest
 * number of workgroups of the VALU kernel (with fewer workgroups than tiles every wave walks
 * several consecutive tiles, one after the other); 0 restores the built-in heuristic for that
 * knob.  Process-wide.  These are the counterparts of the reference's compile-time
 * ThreadBlockShape / WarpShape choices (mixed_gemv_test.cu:67-70). */
MGEMV_API int mgemv_set_launch_override(int split_k_waves, int tiles_per_workgroup, int tiles_per_wave,
                                        int max_workgroups);

/* Smallest m_batch served by the matrix-core kernels instead of the VALU kernel.  0 restores the
 * built-in rules: the k-stationary kernel (MGEMV_MATRIX_CORE_K_STATIONARY below) at 2-16 rows on fp16 problems of 4-16 k
 * steps of 512 (int4; int8: 8-16 k steps of 256, which then count as "up to 8" here) whose 16-row tiles outnumber the
 * compute units -- always with up to 8 k steps (2 rows: 8 k steps
 * and 2.5 tiles per compute unit; 4-5 k steps: 1.5), with 9-16 where its walks of ceil(tiles / compute units) tiles fill
 * the device better than the LDS-staged kernel's workgroups, or as well at 3-4 rows on walks of 2-3 or evenly divided
 * tiles, at 5-8 rows up to 12 k steps on walks of 2, at 2 rows from walks of 3; at 9-16 rows (int4) only where it fills
 * the device better, the partial sums of a walk fit 128 KiB of LDS, and walks of 8-wave workgroups stay within 6 tiles
 * --; else the LDS-staged (a single tile:
 * the register-operand) kernel from 5 rows; from 3 rows on matrices of more than 256 tiles (n_out > 4096); from 4 rows
 * on more than 128 tiles with 16 or more k steps; from 2 rows on 1536 or more tiles with 8 or more k steps or more than
 * 16384 units; int8 weights: from 5 rows, from 3 rows on 1536 or more tiles; never for a single row.  17 keeps every
 * batch size on the VALU kernel, 1 sends every batch size to the matrix cores.  For tuning and tests.  Process-wide. */
MGEMV_API int mgemv_set_matrix_core_threshold(int min_m_batch);

/* Which of the matrix-core kernels serves the small batches:
 *   MGEMV_MATRIX_CORE_AUTO (default)          the k-stationary kernel where the built-in rule finds it ahead
 *                                             (mgemv_set_matrix_core_threshold), else the LDS-staged kernel wherever
 *                                             the matrix has at least two 16-row tiles, else the register-operand
 *                                             kernel;
 *   MGEMV_MATRIX_CORE_REGISTER_OPERAND        always the kernel that reads its activation operand from
 *                                             L2 into registers;
 *   MGEMV_MATRIX_CORE_LDS_STAGED              the LDS-staged kernel wherever the matrix has at least two
 *                                             tiles;
 *   MGEMV_MATRIX_CORE_K_STATIONARY            the kernel whose waves each keep one k step of 512 (int4) or 256
 *                                             (int8) reduction elements and its activation operand in registers
 *                                             while the workgroup walks its tiles, wherever k has at most 16 such
 *                                             steps (fp16 only; else as AUTO).
 * Same results to tolerance either way (the k split, hence the order of the fp32 sums, differs).
 * For tests and measurements; no counterpart in the reference.  Process-wide. */
enum {
  MGEMV_MATRIX_CORE_AUTO = 0,
  MGEMV_MATRIX_CORE_REGISTER_OPERAND = 1,
  MGEMV_MATRIX_CORE_LDS_STAGED = 2,
  MGEMV_MATRIX_CORE_K_STATIONARY = 3
};
MGEMV_API int mgemv_set_matrix_core_variant(int variant);

/* The reference's kStages (mixed_gemv_test.cu:40; gemv/threadblock/default_dq_mma_simt.h:224-234 for
 * the single-stage main loop, :394-404 for the two-stage one) for the VALU kernel: 2 keeps the
 * loads of the next 16-row x 512-k unit in flight while a unit is computed, 1 waits for every load
 * before it computes (loads and arithmetic strictly one after the other), 0 restores the built-in
 * choice (2).  Same results either way.  The matrix-core kernels always run two stages.  For
 * tuning and tests.  Process-wide. */
MGEMV_API int mgemv_set_prefetch_stages(int stages);

/* Which int4 dequantiser the kernels may use.  Both produce the same bits, rn16(rn16(q*s) + z)
 * as gemv/warp/warp_dequantizer.h:52-59:
 *   MGEMV_DEQUANT_AUTO (default)    per wave and k step, the one-FMA form wherever every scale
 *                                   involved is a positive fp16 below 2^-5, else the exact-integer
 *                                   form (the route of gemv/interleaved_numeric_conversion.h:232-291
 *                                   followed by a multiply);
 *   MGEMV_DEQUANT_EXACT_INTEGER     always the exact-integer form.
 * For tests and measurements.  Process-wide. */
enum { MGEMV_DEQUANT_AUTO = 0, MGEMV_DEQUANT_EXACT_INTEGER = 1 };
MGEMV_API int mgemv_set_dequant_form(int form);

/* bfloat16 variants: activations, scales, additive zeros, bias and outputs are bfloat16 bit
 * patterns (the upper 16 bits of a binary32); everything else -- weights, layouts, argument
 * meaning, status codes -- is as in the entry point of the same name without the suffix.
 * They instantiate the reference's templates with ElementB = ElementScale = ElementOutput =
 * cutlass::bfloat16_t: the converters of gemv/interleaved_numeric_conversion.h:130-183 (int8)
 * and :340-401 (int4) followed by the dequantiser of gemv/warp/warp_dequantizer.h:52-59, 86-92 --
 * an instantiation the reference itself still rejects at compile time
 * (gemv/threadblock/default_dq_mma_simt.h:133-134).  Dequantisation is a bf16 multiply and a bf16
 * add, each rounded to nearest even; accumulation is fp32; the output is rounded once to bf16.
 * Kernel choice follows the fp16 rules (mgemv_set_matrix_core_threshold), except that of the two
 * matrix-core kernels only the LDS-staged one exists for bf16 (mgemv_query_launch_bf16 tells). */
MGEMV_API int mgemv_gemv_bf16(const void *weights, const uint16_t *x, const uint16_t *scale,
                              const uint16_t *zero_add, const uint16_t *bias, uint16_t *y, int n_out, int m_batch,
                              int k, int group_size, int quant_op, int weight_bits, void *stream);
MGEMV_API int mgemv_gemv_batched_bf16(const void *weights, const uint16_t *x, const uint16_t *scale,
                                      const uint16_t *zero_add, const uint16_t *bias, uint16_t *y, int batch_count,
                                      int n_out, int m_batch, int k, int group_size, int quant_op, int weight_bits,
                                      int64_t stride_weights, int64_t stride_x, int64_t stride_scale,
                                      int64_t stride_bias, int64_t stride_y, void *stream);
MGEMV_API int mgemv_gemv_routed_bf16(const void *weights, const uint16_t *x, const uint16_t *scale,
                                     const uint16_t *zero_add, const uint16_t *bias, uint16_t *y,
                                     const int32_t *route, int route_extent, int batch_count, int n_out, int m_batch,
                                     int k, int group_size, int quant_op, int weight_bits, int64_t stride_weights,
                                     int64_t stride_x, int64_t stride_scale, int64_t stride_bias, int64_t stride_y,
                                     void *stream);
MGEMV_API int mgemv_dequantize_bf16(const void *weights, const uint16_t *scale, const uint16_t *zero_add,
                                    uint16_t *out, int n_out, int k, int group_size, int quant_op, int weight_bits,
                                    void *stream);
/* ZeroPointPreprocessor<bfloat16_t,int8_t>::neg_zero_point_multiplies_scale (utils/preprocess.h:94-101):
 * out[i] = bf16(-zeros[i]) * scales[i], one bf16 multiply. */
MGEMV_API int mgemv_fold_zero_points_bf16(uint16_t *out, const uint16_t *scales, const int8_t *zeros, size_t n);

/* Tuned plans: a table keyed on the problem (n_out, k, weight_bits, group_size, m_batch) that
 * replaces the built-in launch rules for exactly that problem -- the run-time counterpart of
 * choosing the reference's compile-time ThreadBlockShape / WarpShape / kStages per problem
 * (mixed_gemv_test.cu:40, 67-70; the 1- vs 2-stage main loops of
 * gemv/threadblock/default_dq_mma_simt.h:224-234 and 394-404).  group_size = 0 in an entry
 * matches every group size (an entry for the exact group size wins); per-column problems are
 * looked up with group_size = k.  The knobs have the meaning of mgemv_set_launch_override
 * (0 = built-in rule for that knob); `kernel` picks the kernel.  A process-wide override that is
 * set (mgemv_set_launch_override, _matrix_core_threshold, _matrix_core_variant, _prefetch_stages) takes precedence
 * over the table.  Setting an existing key replaces it.  Results never depend on the plan beyond
 * the order of the fp32 partial sums.  An entry serves launches of its own element type only (a
 * bf16 launch clamps an entry to what its kernels allow).  Thread-safe. */
enum {
  MGEMV_KERNEL_AUTO = 0,
  MGEMV_KERNEL_VALU = 1,
  MGEMV_KERNEL_MATRIX_CORE_REGISTER_OPERAND = 2,
  MGEMV_KERNEL_MATRIX_CORE_LDS_STAGED = 3,
  MGEMV_KERNEL_MATRIX_CORE_K_STATIONARY = 4
};
typedef struct mgemv_tuned_plan {
  int n_out, k, weight_bits, group_size, m_batch; /* key */
  int kernel;                                     /* MGEMV_KERNEL_* */
  int split_k_waves, tiles_per_workgroup, tiles_per_wave, max_workgroups;
  int stages;                                     /* 0 built-in, 1 or 2: see mgemv_set_prefetch_stages */
  int element;                                    /* key: MGEMV_ELEMENT_F16 / MGEMV_ELEMENT_BF16 launches only */
} mgemv_tuned_plan;
MGEMV_API int mgemv_tuned_plan_set(const mgemv_tuned_plan *plan);
/* Removes the entry with exactly plan's key fields, if there is one (the other fields are not read). */
MGEMV_API int mgemv_tuned_plan_erase(const mgemv_tuned_plan *plan);
MGEMV_API int mgemv_tuned_plan_clear(void);
/* The library also carries a built-in table of the same kind (mixed_gemv_amd/default_plans.json,
 * compiled in): plans measured on an unpartitioned MI355X that the built-in rules do not produce.
 * It is consulted after the caller's table, for launches on a device of 256 compute units only, and
 * bypassed like the caller's table while a process-wide override is set.
 * mgemv_set_default_plans(0) switches it off (1 on again); mgemv_default_plan_count tells how many
 * entries it has. */
MGEMV_API int mgemv_set_default_plans(int enable);
MGEMV_API int mgemv_default_plan_count(void);
MGEMV_API int mgemv_tuned_plan_count(void);

/* Reports the geometry mgemv_gemv would use for this problem (group_size as passed to mgemv_gemv,
 * k for per-column problems, 0 to consult only table entries for any group size):
 * out[0] = workgroups, out[1] = threads per
 * workgroup, out[2] = k-split waves per tile, out[3] = tile sequences per workgroup,
 * out[4] = k steps per wave and tile, out[5] = 0 VALU kernel / 1 matrix-core kernel with the
 * activation operand in registers / 2 LDS-staged matrix-core kernel,
 * out[6] = tiles per wave (matrix-core path), out[7] = most tiles a wave walks one after the
 * other (VALU path). */
MGEMV_API int mgemv_query_launch(int n_out, int m_batch, int k, int weight_bits, int group_size, int out[8]);
/* mgemv_query_launch assumes an unpartitioned MI355X (256 compute units); a launch plans for the
 * compute units of the device its stream belongs to.
 * The same for the _bf16 entry points (their kernels are compiled for at most 8 waves per workgroup, and of
 * the matrix-core kernels only the LDS-staged one exists for bf16). */
MGEMV_API int mgemv_query_launch_bf16(int n_out, int m_batch, int k, int weight_bits, int group_size, int out[8]);
/* The same for either element type (MGEMV_ELEMENT_*) and a device of num_compute_units compute
 * units (a partition of an MI355X has 32 per XCD), plus what the plan asks of the hardware:
 * out[8] = bytes of dynamic LDS per workgroup, out[9] = the workgroup size limit the chosen
 * kernel is compiled for, out[10] = prefetch stages (1 or 2), out[11] = launches that serve all
 * activation rows (the VALU kernel takes four rows per launch). */
MGEMV_API int mgemv_query_launch_for(int n_out, int m_batch, int k, int weight_bits, int group_size, int element,
                                     int num_compute_units, int out[12]);

/* Replays, on the host, the index arithmetic every wave of that launch would do -- the same
 * functions the kernels are compiled from -- and reports whether the plan covers the problem:
 * the counterpart of checking the reference's grid (gemv/device/gemv_adaptor.h:190-197) against
 * its threadblock tile offsets (gemv/kernel/mixed_gemv.h:134-139).  Needs no GPU.
 * out[0] = tiles (16 output rows) whose k steps are not covered exactly once (must be 0),
 * out[1] = waves whose range leaves the problem or that have no k step, duplicate workgroups (0),
 * out[2] = most bytes behind one wave's weight descriptor (< 2^31),
 * out[3] = VALU kernel: bytes of LDS up to the last partial sum any wave parks (<= out[4]),
 * out[4] = bytes of dynamic LDS the launch asks for, out[5] = waves with work,
 * out[6] = launched waves without a tile, out[7] = most 16-row x k-step units one wave computes. */
MGEMV_API int mgemv_plan_coverage(int n_out, int m_batch, int k, int weight_bits, int group_size, int element,
                                  int num_compute_units, int64_t out[8]);

#ifdef __cplusplus
}
#endif
#endif /* MIXED_GEMV_H_ */
