/* Measurement probes of libmixed_gemv_amd.so: kernels that the benchmark's "ceilings" are
 * measured with.  They are exported by the same library as the entry points of mixed_gemv.h but
 * are no part of the boundary that stands in for the reference: nothing here has a counterpart
 * in JJXiangJiaoJun/mixed_gemv and nothing here is on a product path.  A binding of the
 * reference's interface needs mixed_gemv.h only. */
#ifndef MIXED_GEMV_PROBES_H_
#define MIXED_GEMV_PROBES_H_

#include "mixed_gemv.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Measurement probes.  No counterpart in the reference and not on any product path: they are
 * what the benchmark's "ceilings" are measured with, so that a figure such as "this launch
 * shape cannot read faster than X" is a kernel anybody can run, not a remark.
 * ---------------------------------------------------------------------------------------- */

/* One empty kernel launch (one wave, no instruction but the end of the program). */
MGEMV_API int mgemv_probe_empty_launch(void *stream);
/* The same with a grid of `workgroups` workgroups of `waves_per_workgroup` waves (1-16), e.g. the
 * GEMV's own launch shape: what dispatching that many waves costs before any of them does anything. */
MGEMV_API int mgemv_probe_empty_grid(int workgroups, int waves_per_workgroup, void *stream);

/* Streams `bytes` of device memory at src (rounded down to whole 4-KiB units per wave) through
 * workgroups x waves_per_workgroup waves, each reading its own contiguous range with the weight
 * loads of the GEMV kernel (1 KiB per wave-wide 128-bit load, streaming cache hint) and
 * units_in_flight (2, 4 or 8) 4-KiB units requested ahead; the data is folded into an
 * exclusive-or and dropped.  sink: 4 writable bytes or NULL. */
MGEMV_API int mgemv_probe_stream_read(const void *src, size_t bytes, int workgroups, int waves_per_workgroup,
                                      int units_in_flight, uint32_t *sink, void *stream);

/* Measurement builds of the single-row int4 scale-and-zero fp16 GEMV kernel (one group per lane
 * run: group sizes that are multiples of 128), launched with the geometry mgemv_gemv would use:
 *   MGEMV_PROBE_LOADS_ONLY  every load of the kernel, the arithmetic of a unit replaced by an
 *                           exclusive-or over its registers; y receives meaningless values;
 *   MGEMV_PROBE_TIMELINE    the kernel as it is, plus MGEMV_PROBE_TIMELINE_WORDS 64-bit words per
 *                           wave, written to trace[wave * MGEMV_PROBE_TIMELINE_WORDS + i] (wave =
 *                           workgroup * waves per workgroup + wave in workgroup; workgroups and
 *                           threads as mgemv_query_launch_for reports for the device).  Words 0-4
 *                           are readings of the 100 MHz constant clock (s_memrealtime): 0 the wave
 *                           starts, 1 its first unit is requested, 2 that unit's first block has
 *                           arrived, 3 its last unit is computed, 4 its outputs are stored;
 *                           word 11 is the number of units the wave computed, words 5-10 are 0;
 *                           words 12 and 13 are the shader clock counter (s_memtime) at the wave's
 *                           start and after its stores, so that (13 - 12) / (4 - 0) * 100 MHz is the
 *                           clock the compute unit ran at.
 *                           trace_capacity_waves: waves the buffer has room for; a launch with
 *                           more returns MGEMV_ERR_SIZE and writes nothing.  y is the GEMV's result;
 *   MGEMV_PROBE_TIMELINE_WAITS  the same, and in front of each unit's arithmetic the wave waits
 *                           explicitly for that unit's operands and first weight block (two more
 *                           clock readings per unit, which slow the kernel by a few per cent):
 *                           words 5-7 are the ticks spent in those waits during the first, second
 *                           and last third of the wave's units, word 8 the longest single wait,
 *                           words 9-10 the clock when the second and the last third began (0 if never);
 *   MGEMV_PROBE_COMPUTE_ONLY every wave loads the first unit of its range and then runs the
 *                           arithmetic of that unit once per unit of the range, loading nothing
 *                           more: what the kernel's instructions alone take; y is meaningless. */
enum { MGEMV_PROBE_LOADS_ONLY = 1, MGEMV_PROBE_TIMELINE = 2, MGEMV_PROBE_COMPUTE_ONLY = 3, MGEMV_PROBE_TIMELINE_WAITS = 4 };
#define MGEMV_PROBE_TIMELINE_WORDS 14
MGEMV_API int mgemv_probe_gemv(int kind, unsigned long long *trace, size_t trace_capacity_waves, const void *weights,
                               const uint16_t *x,
                               const uint16_t *scale, const uint16_t *zero_add, uint16_t *y, int n_out, int k,
                               int group_size, void *stream);

/* The same two builds -- MGEMV_PROBE_LOADS_ONLY, MGEMV_PROBE_COMPUTE_ONLY -- for a launch of m_batch
 * activation rows, where they exist: one row as above; on the matrix cores the LDS-staged kernel whose
 * workgroups share their activation stage between two or more tiles (int4, scale and zero, fp16,
 * group sizes 64-512; e.g. 8192 x 8192 at 8-16 rows), and the k-stationary kernel (same operand types;
 * e.g. 28672 x 8192 at 2-16 rows).  On the LDS-staged kernel "loads only" keeps the staging of the
 * activation rows and the barriers, and "compute only" requests a wave's first k step only and
 * repeats that step's staging and arithmetic; on the k-stationary kernel "loads only" keeps the
 * operand's way through LDS, the parking of the partial sums, the barrier and the combine, and
 * "compute only" requests the first tile's unit only and repeats its arithmetic for every tile of
 * the walk.  Other launches return MGEMV_ERR_QUANT_OP. */
MGEMV_API int mgemv_probe_gemv_rows(int kind, int m_batch, const void *weights, const uint16_t *x,
                                    const uint16_t *scale, const uint16_t *zero_add, uint16_t *y, int n_out, int k,
                                    int group_size, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MIXED_GEMV_PROBES_H_ */
