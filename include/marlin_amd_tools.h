/*
 * Tools of libmarlin_amd.so beside its drop-in boundary (marlin_amd.h): what
 * the library would do with a problem, and per-thread overrides of its
 * planner.  None has a counterpart in the reference; tests and benchmarks use
 * them, a binding of the W4A16 path does not need them.  (The measurement
 * probes are a library of their own: marlin_amd_probe.h.)
 */
#ifndef MARLIN_AMD_TOOLS_H
#define MARLIN_AMD_TOOLS_H

#include "marlin_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Argument validation of marlin_gemm alone (no GPU touched): the code
 * marlin_gemm would return for these sizes and hints. */
int marlin_amd_check(int prob_m, int prob_n, int prob_k, int groupsize, int thread_k,
                     int thread_n);

/*
 * How marlin_gemm would run a problem on a device with `cus` compute units:
 * out[0] = kernel (0 = none, 1 = streaming, 2 = prefill, 3 = column strips),
 * out[1] = workgroups,
 * out[2] = granules per workgroup (streaming), out[3] = column tiles,
 * out[4] = granules per column tile, out[5] = number of launches,
 * out[6] = slices of the k range per tile (prefill), out[7] = rows of C per
 * workgroup (prefill; 0 for the streaming kernel), out[8] = workgroups per
 * column tile when the streaming kernel cuts every tile into that many runs
 * (then out[2] is the longest run), 0 when it cuts the tile-major sequence of
 * granules into equal runs of out[2]; out[9] = KiB of partial sums the launch
 * exchanges through the library's scratch (0 = none); out[10] = parts the
 * streaming kernel cuts the rows into (1 = uncut; every part is a problem of
 * its own for out[8] workgroups per column tile), out[11] = rows of a part;
 * out[12] = 16-column strips per workgroup of the column-strip kernel (else 0),
 * which cuts more than 16 rows into out[10] parts of 16, a workgroup per strip
 * set and part (out[1] = strip sets x parts).
 * `out` holds 13 ints.  Returns the marlin_gemm error code for the shape.
 */
int marlin_amd_plan(int prob_m, int prob_n, int prob_k, int groupsize, int thread_k,
                    int thread_n, int sms, int cus, int *out);

/*
 * The streaming kernel's assignment of work to workgroups: out[b] is the work
 * index of workgroup b of a launch of `grid` workgroups (work index w owns
 * granules [w * granules_per_wg, (w + 1) * granules_per_wg) of the plan).  A
 * permutation of 0..grid-1 in which the workgroups that the hardware deals to
 * one XCD (b mod 8) hold consecutive indices.  No reference counterpart; for
 * tests and tools.
 */
void marlin_amd_work_order(int grid, int *out);

/*
 * The fitted costs (microseconds on an MI355X) that the choice of kernel
 * compares, for a device with `cus` compute units: out[0] = the streaming
 * kernel as it would be launched (rows cut where that is cheaper), out[1] =
 * the prefill kernel with its cheapest tile height and slice count (-1 where
 * prob_n is no multiple of 256), out[2] = the column strips with their
 * cheapest width and out[3] that width (-1 beyond 1024 rows; cost -1 and width 0
 * where the planner's rules allow no width).  `out` holds 4
 * doubles.  Returns the marlin_gemm error code for the shape.  No reference
 * counterpart; for tests and tools that check the fit against measurements.
 */
int marlin_amd_plan_costs(int prob_m, int prob_n, int prob_k, int groupsize, int cus,
                          double *out);

/*
 * Which kernel marlin_gemm uses for calls made by the calling thread: 0 =
 * choose by cost (default), 1 = the streaming kernel, 64 rows per launch, 2 =
 * the prefill kernel (needs prob_n % 256 == 0, else the streaming kernel is
 * used), 3 = the column-strip kernel (at most 1024 rows and no `sms` hint,
 * else as with 0), 4 = by cost between the streaming and the prefill kernel
 * only (few rows then always meet the exchange between workgroups).  Like the
 * overrides below it is kept per host thread, so it never changes what other
 * threads' calls do.  No reference counterpart; for tests
 * and tools.
 */
void marlin_amd_force_kernel(int which);

/*
 * 16-column strips per workgroup of the column-strip kernel, for the calling
 * thread: 0 = choose by cost (default), or 1 to 4 (2 and 4 only where prob_n
 * is a multiple of 16 x strips, else 1; with 3 the last workgroup holds what
 * is left).  No reference counterpart; for tests and tools.
 */
void marlin_amd_force_strips(int strips);

/*
 * Slices of the k range per tile of the prefill kernel, for the calling
 * thread: 0 = choose by cost (default), n = n slices where the problem allows (each slice
 * at least 256 deep).  No reference counterpart; for tests and tools.
 */
void marlin_amd_force_k_slices(int slices);

/*
 * Whether the streaming kernel cuts the rows into parts that separate
 * workgroups compute (17..64 rows into two halves instead of cutting the k
 * range of a tile once more; more than 64 rows into parts of 32 in one launch
 * instead of a launch per 64 rows), for the calling thread: 0 = choose by cost
 * (default), 1 = never, 2 = wherever possible.  No reference counterpart; for
 * tests and tools.
 */
void marlin_amd_force_row_halves(int mode);

/*
 * Rows of C per workgroup of the prefill kernel, for the calling thread: 0 =
 * choose by cost (default), 64 or 128.  No reference counterpart; for tests and tools.
 */
void marlin_amd_force_tile_rows(int rows);

/*
 * out[0..4] = compute units, shader clock (kHz), memory clock (kHz), memory
 * bus width (bits), L2 size (bytes) of device dev, as the HIP runtime reports
 * them.  Returns MARLIN_OK or MARLIN_ERR_RUNTIME.
 */
int marlin_amd_device_info(int dev, int *out);

#ifdef __cplusplus
}
#endif
#endif
