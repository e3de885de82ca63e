/*
 * CPU oracle for the W4A16 Marlin GEMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of what the reference computes on the path
 *   marlin.mul -> marlin_lib.mul -> marlin_cute / marlin_official
 * (gemm/marlin_gemm/ in the reference tree).  It is the checker for the HIP
 * kernels: only the tests, the smoke entry and the benchmark's CPU-baseline
 * leg may link or call it.  Nothing in the shipped library depends on it.
 *
 * Pinning status of each function (what fixes its behaviour independently
 * of this file's own formulae) is stated next to its declaration.  The
 * reference holds no golden vectors for this path, so every function is
 * pinned by mathematics (closed forms, exhaustive enumeration, two
 * independent derivations) and not by reference fixtures.
 */
#ifndef W4A16_REF_H
#define W4A16_REF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- IEEE binary16 soft-float ------------------------------------------
 * Pinned by: exhaustive comparison with numpy.float16 over all 65536 bit
 * patterns (to_f32) and over a dense sweep of float32 inputs (from_f32),
 * including ties, subnormals, overflow and NaN. */
float ref_f16_to_f32(uint16_t h);
uint16_t ref_f32_to_f16(float f);   /* round-to-nearest-even */
uint16_t ref_f64_to_f16(double d);  /* round-to-nearest-even, single rounding */
uint16_t ref_f16_mul(uint16_t a, uint16_t b);              /* RN(a*b)   */
uint16_t ref_f16_sub(uint16_t a, uint16_t b);              /* RN(a-b)   */
uint16_t ref_f16_fma(uint16_t a, uint16_t b, uint16_t c);  /* RN(a*b+c) */

/* ---- Marlin permutations ------------------------------------------------
 * Transcription of the integer algorithm in marlin.py:29-55 (_get_perms).
 * perm[1024], scale_perm[64], scale_perm_single[32].
 * Pinned by: equality with the closed forms below at all positions, the
 * bijection property, and the hand-derived value for lane 5
 * (perm[160..167] = 33,161,41,169,49,177,57,185). */
void marlin_get_perms(int *perm, int *scale_perm, int *scale_perm_single);

/* ---- Packing (restates Layer.pack, marlin.py:111-129) -------------------
 * q:  K x N row-major, one uint8 per weight, value in [0,15].
 * B:  (K/16) x (2N) int32, nibble i of each word at bits 4i..4i+3.
 * s:  G x N fp16 bits (G = K/groupsize, or 1 for per-channel).
 * sp: same shape, permuted within 64-column blocks (groupwise != 0) or
 *     32-column blocks (groupwise == 0).
 * Requires K % 16 == 0 and N % 64 == 0. */
void marlin_pack_weights(const uint8_t *q, int K, int N, int32_t *B);
void marlin_pack_scales(const uint16_t *s, int G, int N, int groupwise,
                        uint16_t *sp);

/* ---- Closed-form layout (independent derivation) ------------------------
 * Derived from what the kernels consume (m16n8k16 B-fragment ownership at
 * marlin_official_kernel.cu:292-299,438-452, dequant nibble order at
 * marlin_cute_trait.h:20-39), not from the packing code:
 *   word w of row kt:  n64 = w / 128, lane = (w % 128) / 4, j = w % 4,
 *   t = lane % 4, c = lane / 4;  nibble e holds
 *   W[16 kt + 2t + ((e>>2)&1) + 8(e&1)][64 n64 + 16 j + c + 8((e>>1)&1)].
 * Pinned by: agreement with marlin_pack_weights on all positions. */
void marlin_weight_coord(int kt, int word, int e, int *k, int *n);
void marlin_unpack_weights(const int32_t *B, int K, int N, uint8_t *q);
/* index into a packed scale row of the scale for logical column n */
int marlin_scale_index_group(int n);   /* 64b + 8(n%8) + (n%64)/8       */
int marlin_scale_index_single(int n);  /* see marlin.py:53-54            */
void marlin_unpack_scales(const uint16_t *sp, int G, int N, int groupwise,
                          uint16_t *s);

/* ---- Dequantisation -----------------------------------------------------
 * marlin_dequant_magic restates the bit trick of marlin_cute_trait.h:20-39
 * (== marlin_official_kernel.cu:131-152) in soft-float: out[0..1] is the
 * half2 from the low nibbles (nibbles 0 and 4 of q), out[2..3] the half2
 * from nibbles 1 and 5.  Pinned by: exhaustive equality with fp16(nibble-8).
 *
 * w4a16_dequant_ref: W[k][n] (fp16 bits, K x N row-major) from the packed
 * buffers.  groupsize > 0: W = RN_fp16((q-8) * s[k/groupsize][n]) (one
 * rounding, marlin_official_kernel.cu:155-159; equals the Python oracle's
 * (w-8).half()*s, marlin_test.py:31).  groupsize == -1: W = fp16(q-8), the
 * column scale is applied to the output instead (marlin_official_kernel.cu:
 * 622-626).  Pinned by: numpy.float16 arithmetic on independently unpacked
 * inputs. */
void marlin_dequant_magic(int32_t q, uint16_t out[4]);
void w4a16_dequant_ref(const int32_t *B, const uint16_t *sp, int K, int N,
                       int groupsize, uint16_t *W);

/* ---- GEMM -----------------------------------------------------------------
 * C[m][n] = fp16( sum_k fp32(A[m][k]) * fp32(W[k][n]) ), fp32 accumulation in
 * ascending k; per-channel mode multiplies the rounded fp16 result by the
 * column scale in fp16 (one more rounding).  threads <= 0 uses all cores.
 * Pinned by: the float64 brute force below on small shapes, closed forms
 * (all q == 8 gives 0; unit scales and small-integer A give exact integers;
 * one-hot rows of A return rows of W bit-exactly).
 * Returns 0, or -1 when the temporary buffer cannot be allocated. */
int w4a16_gemm_ref(const uint16_t *A, const int32_t *B, const uint16_t *sp,
                   uint16_t *C, int M, int N, int K, int groupsize,
                   int threads);
/* Dense fp16 GEMM of the sibling path gemm/streamk_gemm: C (M x N) =
 * A (M x K, row-major) * B^T with B as N rows of K; fp32 accumulation in
 * ascending k, one rounding to fp16.  Pinned against numpy's float64 matmul
 * (tests/test_streamk_host.py).  Returns 0, or -1 without memory. */
int f16_gemm_tn_ref(const uint16_t *A, const uint16_t *B, uint16_t *C, int M,
                    int N, int K, int threads);
/* Same result type, float64 accumulation straight from the packed nibbles
 * through marlin_weight_coord; O(MNK) scalar, for tiny shapes only. */
void w4a16_gemm_ref_f64(const uint16_t *A, const int32_t *B,
                        const uint16_t *sp, double *C, int M, int N, int K,
                        int groupsize);

/* ---- Quantiser (restates gen_quant4, marlin_test.py:18-55) ---------------
 * w: K x N fp16 bits.  Outputs q (K x N, [0,15]), s (G x N fp16 bits) and
 * ref (K x N fp16 bits, the fake-quantised weight).  s = max|w| * (2/15) per
 * group and column, q = clamp(round_half_even(w / s) + 8, 0, 15).
 * Pinned by tests/test_host.py (test_quantize_matches_oracle_quantiser): q, s and ref
 * equal, bit for bit, what the reference's own sequence of torch operations
 * (marlin_test.py:18-40: abs/amax, `s *= 2/15`, `w / s`, round, +8, clamp,
 * `(q - 8).half() * s`) gives when torch's CPU half kernels evaluate it -- an
 * independent library evaluation that a double rounding or a wrong tie rule
 * fails -- plus the invariants |ref - w| <= s/2 inside the clamp range and
 * q == 15 at the group maximum.  Residual: the reference runs those operations
 * with torch's CUDA half kernels, which cannot be run here; IEEE half
 * arithmetic leaves them no freedom in the results. */
void gen_quant4_ref(const uint16_t *w, int K, int N, int groupsize,
                    uint8_t *q, uint16_t *s, uint16_t *ref);

/* ---- Comparison helpers ----------------------------------------------------
 * max_abs_err / max_abs_ref implement the acceptance rule
 * max|C - C_ref| <= 1e-2 * max|C_ref|; rel_mean_abs_err is the figure the
 * reference test prints (marlin_test.py:74); cosine restates
 * include/reference.h:145-165. */
typedef struct {
  double max_abs_err;
  double max_abs_ref;
  double rel_mean_abs_err;
  double cosine;
  long long mismatched_bits; /* number of elements whose fp16 bits differ */
} w4a16_compare_t;
void w4a16_compare(const uint16_t *C, const uint16_t *Cref, size_t n,
                   w4a16_compare_t *out);

int w4a16_ref_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
