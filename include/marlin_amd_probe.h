/*
 * libmarlin_amd_probe.so: measurement probes beside libmarlin_amd.so (which it
 * links against for the plan of a shape).  They launch kernels that compute
 * nothing -- an empty one, a plain read of the packed weights, a loop of MFMAs
 * -- so that a benchmark can put the floor of the same box beside every GEMM
 * time.  No counterpart in the reference; the product library contains none of
 * this.
 */
#ifndef MARLIN_AMD_PROBE_H
#define MARLIN_AMD_PROBE_H

#include "marlin_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * A probe launch on `stream` of device `dev`.  Kinds 0 and 1 use the grid and
 * the workgroup size marlin_gemm uses for prob_m rows of this shape (where
 * that is the prefill kernel's, for 16 rows): kind 0 = an empty kernel (what a
 * launch costs), kind 1 = a kernel that reads the packed weights B
 * ((prob_k/16, 2*prob_n) int32) with the work split of the kernel planned for
 * the shape -- the streaming kernel's or the column-strip kernel's -- and
 * 128-bit loads and does nothing with them (what the weight stream alone
 * costs).  Kind 2 = a loop of nothing but v_mfma_f32_16x16x32_f16 on
 * pseudo-random operands, one workgroup of 8 waves per compute unit and
 * prob_n*prob_k/8192 MFMAs (16384 flop each) per wave, i.e. the multiply-adds
 * of 2048 rows of this shape: what the matrix pipes sustain when nothing
 * competes with them (B is not read).  Nothing is written.  Returns
 * MARLIN_OK, the marlin_gemm error code of the shape, or MARLIN_ERR_RUNTIME
 * (text in marlin_amd_probe_last_error).
 */
int marlin_amd_probe(int kind, const void *B, int prob_m, int prob_n, int prob_k, int dev,
                     void *stream);

/*
 * What a lone wave per SIMD can issue beside its MFMAs (synchronous, on the
 * current device's null stream): `workgroups` workgroups of four waves, one per
 * CU, run `iters` turns of 32 independent v_mfma_f32_16x16x32_f16, each MFMA
 * followed by n_valu independent packed-fp16 VALU operations (0..4), and the
 * first n_lds / n_global MFMAs of every eight also by a 16-byte LDS read / a
 * 16-byte global load (supported mixes: n_valu alone; n_lds 1, 2 or n_global
 * 1, 2 alone; n_valu = 2 with one of either).  cycles_out[w] = shader cycles
 * per turn of workgroup w (divide by 32 for cycles per MFMA).
 */
int marlin_amd_probe_issue(int n_valu, int n_lds, int n_global, int iters, int workgroups,
                           float *cycles_out);

/*
 * What compute units pull from memory (synchronous, null stream): workgroup w
 * of 256 threads reads bytes_per_workgroup (a multiple of 64 KiB) of `src`
 * (src_bytes long, at least workgroups * bytes_per_workgroup) starting at
 * w * bytes_per_workgroup with `depth` (1, 4 or 16) 16-byte loads in flight per
 * thread; ticks_out[w] = what it took in ticks of the 100 MHz constant clock.
 */
int marlin_amd_probe_pull(const void *src, long long src_bytes, long long bytes_per_workgroup,
                          int depth, int workgroups, float *ticks_out);

/* Text of the calling thread's last probe failure ("" if none). */
const char *marlin_amd_probe_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
