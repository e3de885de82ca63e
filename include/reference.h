/*
 * CPU reference of the W4A16 Marlin GEMM (dequantise, fp32-accumulate GEMM,
 * fp16 output; packing and comparison helpers).  TEST INFRASTRUCTURE: the
 * implementation lives in oracle/ and is the checker for the HIP kernels; the
 * shipped library (include/marlin_amd.h) neither includes nor links it.
 *
 * The file of this name in the reference tree holds only GPU timers and
 * compare helpers (include/reference.h:11-177) and no CPU GEMM; this header
 * supplies the CPU reference the parity tests need, plus host restatements of
 * those compare helpers (w4a16_compare: max-abs error, cosine >= 0.999 rule of
 * include/reference.h:145-165).
 */
#ifndef W4A16_REFERENCE_H
#define W4A16_REFERENCE_H
#include "../oracle/w4a16_ref.h"
#endif
