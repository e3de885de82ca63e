/*
 * C ABI of the MI355X (gfx950) W4A16 Marlin GEMM library, libmarlin_amd.so.
 *
 * Plain pointers and sizes only.  Every buffer is a caller-owned DEVICE
 * pointer; calls are asynchronous on the given HIP stream and return after
 * enqueueing.  Return codes follow the reference launcher
 * (marlin_cute_kernel.cu:4-5): 0 = ok (also for an empty problem),
 * 1 = problem shape not compatible with the tile, 2 = no kernel for this
 * tile / group size, and in addition 3 = the HIP runtime reported an error
 * (the reference never checks).
 */
#ifndef MARLIN_AMD_H
#define MARLIN_AMD_H

#ifdef __cplusplus
extern "C" {
#endif

#define MARLIN_OK 0
#define MARLIN_ERR_PROB_SHAPE 1 /* marlin_cute_kernel.cu:4 */
#define MARLIN_ERR_KERN_SHAPE 2 /* marlin_cute_kernel.cu:5 */
#define MARLIN_ERR_RUNTIME 3
#define MARLIN_ERR_GROUPS 4    /* marlin_gemm.cpp:27-28 */
#define MARLIN_ERR_WORKSPACE 5 /* marlin_gemm.cpp:29-31 */

/*
 * FP16 x INT4 GEMM, C = A * dequant(B).  Replaces
 *   int marlin_cute(const void *A, const void *B, void *C, void *s,
 *                   int prob_m, int prob_n, int prob_k, void *workspace,
 *                   int groupsize, int dev, cudaStream_t stream,
 *                   int thread_k, int thread_n, int sms, int max_par)
 * (declared marlin_gemm.cpp:6-9, defined marlin_cute_kernel.cu:28-115), same
 * argument order and meaning:
 *   A   (prob_m, prob_k) fp16 row-major
 *   B   (prob_k/16, 2*prob_n) int32, Marlin-packed int4 (marlin.py:92-131)
 *   C   (prob_m, prob_n) fp16 row-major, fully overwritten
 *   s   (prob_k/groupsize, prob_n) fp16, or (1, prob_n) when groupsize == -1,
 *       permuted as Layer.pack leaves it
 *   workspace  at least prob_n/128*max_par int32, all zero on entry; all zero
 *       again when the call's kernels have finished
 *   groupsize  128 or -1 (per output column)
 *   stream     a hipStream_t (0 = the default stream)
 *   thread_k, thread_n   tile hints as in the reference: -1 = automatic
 *       ((128,128) up to 16 rows, else (64,256)).  They are validated exactly
 *       as the reference validates them but do not select the kernel.
 *   sms        number of workgroups of the streaming kernel, -1 = automatic
 *   max_par    at least 1 (else MARLIN_ERR_WORKSPACE); sizes the workspace
 *       contract, and the tile counters sit min(max_par, 16) ints apart in it
 * Not re-entrant over the same workspace or the same C concurrently.
 * Partial sums of output tiles that several workgroups share live in a
 * library-owned buffer per (device, stream), sized by the call's plan and
 * grown on demand (hipMalloc on the first call that needs more; 64 KiB of tile
 * counters + whole MiB of partial sums, 4 MiB for N = K = 4096 at one row).  A call that
 * would have to allocate while `stream` is being captured into a graph returns
 * MARLIN_ERR_RUNTIME: run the call once on that stream before the capture, or
 * use marlin_gemm_static.
 */
int marlin_gemm(const void *A, const void *B, void *C, const void *s, int prob_m, int prob_n,
                int prob_k, void *workspace, int groupsize, int dev, void *stream, int thread_k,
                int thread_n, int sms, int max_par);

/* Same entry under the two names the reference binding links against
 * (marlin_gemm.cpp:6-14); both run the same kernels here. */
int marlin_cute(const void *A, const void *B, void *C, void *s, int prob_m, int prob_n,
                int prob_k, void *workspace, int groupsize, int dev, void *stream, int thread_k,
                int thread_n, int sms, int max_par);
int marlin_official(const void *A, const void *B, void *C, void *s, int prob_m, int prob_n,
                    int prob_k, void *workspace, int groupsize, int dev, void *stream,
                    int thread_k, int thread_n, int sms, int max_par);

/*
 * marlin_gemm for callers that cannot allocate device memory (code under HIP
 * graph capture, serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same arguments, same kernels and same results
 * as marlin_gemm for the same plan, but partial sums and tile counters use a
 * fixed array inside the library's device image (32 MiB + 64 KiB, held by
 * every GPU the library runs on until the process ends) and the call never
 * calls hipMalloc, hipFree or any allocating routine.  The plan is made for
 * that size (fewer k slices where they would not fit); a call whose partial
 * sums still exceed marlin_gemm_static_capacity() bytes (only an explicit
 * `sms` above the device's compute units with more than 16 rows can) returns
 * MARLIN_ERR_RUNTIME with a message.  All calls on one GPU share the array:
 * calls that may overlap in time on one GPU (different streams, or graph
 * branches) race on it -- silently: wrong sums, or a tile that nobody writes --
 * and must use marlin_gemm instead.  The first call on a device looks the
 * array's address up (hipGetSymbolAddress; no kernel, no allocation); the
 * array's counters are zero when the library is loaded and every call hands
 * them back zeroed.
 */
int marlin_gemm_static(const void *A, const void *B, void *C, const void *s, int prob_m,
                       int prob_n, int prob_k, void *workspace, int groupsize, int dev,
                       void *stream, int thread_k, int thread_n, int sms, int max_par);
/* bytes of partial sums the fixed array of marlin_gemm_static holds */
long long marlin_gemm_static_capacity(void);

/*
 * The checks of the reference's tensor-level binding `mul`
 * (marlin_gemm.cpp:19-56) on plain sizes: derives groupsize from the number
 * of scale rows (1 row = per-channel), rejects k not divisible into the
 * groups (MARLIN_ERR_GROUPS) and a workspace shorter than
 * prob_n/128*max(max_par,1) entries (MARLIN_ERR_WORKSPACE), calls marlin_gemm and,
 * on any error, writes the reference's message text into err (if non-null).
 */
int marlin_mul(const void *A, const void *B, void *C, const void *s, int prob_m, int prob_n,
               int prob_k, int s_rows, void *workspace, long long workspace_numel, int dev,
               void *stream, int thread_k, int thread_n, int sms, int max_par, int cute_version,
               char *err, int err_len);

/*
 * Device memory the library holds for partial sums on device dev (all devices
 * if dev < 0): returns the bytes, *buffers (if non-null) the number of
 * (device, stream) buffers.  Touches no GPU.  No reference counterpart.
 */
long long marlin_amd_scratch_bytes(int dev, int *buffers);

/*
 * Frees the partial-sum buffers of device dev (all devices if dev < 0) after
 * waiting for the device's work; returns the bytes freed.  Graphs captured
 * earlier name the freed buffers and must not be replayed afterwards.  The
 * next call that needs scratch allocates again.  No reference counterpart (the
 * reference keeps its partial sums in C).
 */
long long marlin_amd_release(int dev);

/*
 * Introspection, planner overrides and measurement probes for tests and
 * benchmarks -- marlin_amd_check, marlin_amd_plan, marlin_amd_work_order,
 * marlin_amd_force_*, marlin_amd_device_info, marlin_amd_probe -- are declared
 * in marlin_amd_tools.h; a binding of the path does not need them.
 */

/* Text of the last HIP runtime error seen by this thread ("" if none). */
const char *marlin_amd_last_error(void);

/* Library version string. */
const char *marlin_amd_version(void);

#ifdef __cplusplus
}
#endif
#endif
