/*
 * CPU oracle for the W4A16 Marlin GEMM path.  TEST INFRASTRUCTURE ONLY:
 * the checker for the HIP kernels, never part of the shipped library.
 * See w4a16_ref.h for what each function restates and how it is pinned.
 */
#include "w4a16_ref.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 */

float ref_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int shift = 0;
      while (!(man & 0x400u)) {
        man <<= 1;
        shift++;
      }
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* Round a double to binary16, nearest-even, in one rounding step. */
uint16_t ref_f64_to_f16(double d) {
  uint64_t bits;
  memcpy(&bits, &d, 8);
  uint16_t sign = (uint16_t)((bits >> 48) & 0x8000u);
  int exp = (int)((bits >> 52) & 0x7ff);
  uint64_t man = bits & 0xfffffffffffffull;
  if (exp == 0x7ff) { /* inf / nan */
    if (man) return (uint16_t)(sign | 0x7e00u);
    return (uint16_t)(sign | 0x7c00u);
  }
  if (exp == 0) return sign; /* double subnormals are far below half range */
  int e = exp - 1023; /* unbiased */
  man |= 1ull << 52;  /* 53-bit significand, value = man * 2^(e-52) */
  /* target: normal halves keep 11 significant bits (shift 42); below 2^-14
   * the kept width shrinks by the distance to the subnormal range */
  int shift = 42;
  int he = e + 15; /* biased half exponent if normal */
  if (he <= 0) {
    shift += 1 - he;
    he = 0;
  }
  if (shift > 63) return sign; /* underflows to zero (below half the ulp) */
  uint64_t kept = man >> shift;
  uint64_t rem = man & ((1ull << shift) - 1);
  uint64_t half = 1ull << (shift - 1);
  if (rem > half || (rem == half && (kept & 1))) kept++;
  uint32_t out;
  if (he == 0) {
    out = (uint32_t)kept; /* may carry into the normal range: still right */
  } else {
    /* kept has the implicit bit at position 10 (or 11 after a carry) */
    out = ((uint32_t)he << 10) + (uint32_t)(kept - 0x400u);
  }
  if (out >= 0x7c00u) out = 0x7c00u; /* overflow to infinity */
  return (uint16_t)(sign | out);
}

uint16_t ref_f32_to_f16(float f) {
  /* float -> double is exact, so one rounding happens in ref_f64_to_f16 */
  return ref_f64_to_f16((double)f);
}

uint16_t ref_f16_mul(uint16_t a, uint16_t b) {
  /* the product of two 11-bit significands is exact in double */
  return ref_f64_to_f16((double)ref_f16_to_f32(a) * (double)ref_f16_to_f32(b));
}

uint16_t ref_f16_sub(uint16_t a, uint16_t b) {
  /* the exponent span of binary16 (40 binades + 11 bits) fits in a double */
  return ref_f64_to_f16((double)ref_f16_to_f32(a) - (double)ref_f16_to_f32(b));
}

uint16_t ref_f16_fma(uint16_t a, uint16_t b, uint16_t c) {
  /* exact while product and addend are within ~30 binades of each other,
   * which holds for the dequantisation constants this is used for */
  return ref_f64_to_f16((double)ref_f16_to_f32(a) * (double)ref_f16_to_f32(b) +
                        (double)ref_f16_to_f32(c));
}

/* ----------------------------------------------------------- permutations */

/* marlin.py:29-55 */
void marlin_get_perms(int *perm, int *scale_perm, int *scale_perm_single) {
  int raw[1024];
  int pos = 0;
  for (int i = 0; i < 32; i++) {
    int perm1[8];
    int cnt = 0;
    int col = i / 4;
    for (int block = 0; block < 2; block++) {
      int rows[4] = {2 * (i % 4), 2 * (i % 4) + 1, 2 * (i % 4 + 4),
                     2 * (i % 4 + 4) + 1};
      for (int r = 0; r < 4; r++) perm1[cnt++] = 16 * rows[r] + col + 8 * block;
    }
    for (int j = 0; j < 4; j++)
      for (int p = 0; p < 8; p++) raw[pos++] = perm1[p] + 256 * j;
  }
  static const int interleave[8] = {0, 2, 4, 6, 1, 3, 5, 7};
  for (int g = 0; g < 128; g++)
    for (int p = 0; p < 8; p++) perm[8 * g + p] = raw[8 * g + interleave[p]];
  pos = 0;
  for (int i = 0; i < 8; i++)
    for (int j = 0; j < 8; j++) scale_perm[pos++] = i + 8 * j;
  pos = 0;
  static const int offs[8] = {0, 1, 8, 9, 16, 17, 24, 25};
  for (int i = 0; i < 4; i++)
    for (int j = 0; j < 8; j++) scale_perm_single[pos++] = 2 * i + offs[j];
}

/* marlin.py:119-129: (K,N) -> 16x16 tiles laid out as rows of (K/16, 16N),
 * every 1024-element run gathered through perm, then 8 nibbles per word. */
void marlin_pack_weights(const uint8_t *q, int K, int N, int32_t *B) {
  int perm[1024], sp[64], sps[32];
  marlin_get_perms(perm, sp, sps);
  size_t rowlen = (size_t)N * 16;
  uint8_t *tiled = (uint8_t *)malloc(rowlen);
  uint8_t *gathered = (uint8_t *)malloc(rowlen);
  for (int kt = 0; kt < K / 16; kt++) {
    /* w.reshape(K/16,16,N/16,16).permute(0,2,1,3).reshape(K/16, 16N) */
    for (int nt = 0; nt < N / 16; nt++)
      for (int r = 0; r < 16; r++)
        for (int c = 0; c < 16; c++)
          tiled[(size_t)nt * 256 + r * 16 + c] =
              q[(size_t)(kt * 16 + r) * N + nt * 16 + c];
    /* res.reshape(-1, 1024)[:, perm] */
    for (size_t chunk = 0; chunk < rowlen / 1024; chunk++)
      for (int p = 0; p < 1024; p++)
        gathered[chunk * 1024 + p] = tiled[chunk * 1024 + perm[p]];
    /* q |= res[:, i::8] << 4i */
    for (size_t w = 0; w < rowlen / 8; w++) {
      uint32_t word = 0;
      for (int i = 0; i < 8; i++)
        word |= (uint32_t)(gathered[8 * w + i] & 0xf) << (4 * i);
      B[(size_t)kt * (rowlen / 8) + w] = (int32_t)word;
    }
  }
  free(tiled);
  free(gathered);
}

/* marlin.py:111-118 */
void marlin_pack_scales(const uint16_t *s, int G, int N, int groupwise,
                        uint16_t *sp) {
  int perm[1024], sperm[64], sperm1[32];
  marlin_get_perms(perm, sperm, sperm1);
  size_t total = (size_t)G * N;
  if (groupwise) {
    for (size_t blk = 0; blk < total / 64; blk++)
      for (int p = 0; p < 64; p++) sp[blk * 64 + p] = s[blk * 64 + sperm[p]];
  } else {
    for (size_t blk = 0; blk < total / 32; blk++)
      for (int p = 0; p < 32; p++) sp[blk * 32 + p] = s[blk * 32 + sperm1[p]];
  }
}

/* ------------------------------------------------- closed-form layout (ii) */

void marlin_weight_coord(int kt, int word, int e, int *k, int *n) {
  int n64 = word / 128;
  int lane = (word % 128) / 4;
  int j = word % 4;
  int t = lane % 4;
  int c = lane / 4;
  *k = 16 * kt + 2 * t + ((e >> 2) & 1) + 8 * (e & 1);
  *n = 64 * n64 + 16 * j + c + 8 * ((e >> 1) & 1);
}

void marlin_unpack_weights(const int32_t *B, int K, int N, uint8_t *q) {
  int words = 2 * N;
  /* rows kt write disjoint rows of q */
#pragma omp parallel for schedule(static)
  for (int kt = 0; kt < K / 16; kt++)
    for (int w = 0; w < words; w++) {
      uint32_t word = (uint32_t)B[(size_t)kt * words + w];
      for (int e = 0; e < 8; e++) {
        int k, n;
        marlin_weight_coord(kt, w, e, &k, &n);
        q[(size_t)k * N + n] = (uint8_t)((word >> (4 * e)) & 0xf);
      }
    }
}

/* A lane with column offset c inside a 64-column block reads eight
 * consecutive halves that must be columns c, c+8, ..., c+56
 * (marlin_official_kernel.cu:326-329,431): an 8x8 transpose. */
int marlin_scale_index_group(int n) {
  int b = n / 64, w = n % 64;
  return 64 * b + 8 * (w % 8) + w / 8;
}

/* Each accumulator lane owns column pairs (2t, 2t+1) + 8x, x = 0..3, of a
 * 32-column run and reads them as eight consecutive halves
 * (marlin_official_kernel.cu:634-637,720-723). */
int marlin_scale_index_single(int n) {
  int b = n / 32, u = n % 32;
  int t = (u % 8) / 2;
  int x = 2 * (u / 8) + (u % 2);
  return 32 * b + 8 * t + x;
}

void marlin_unpack_scales(const uint16_t *sp, int G, int N, int groupwise,
                          uint16_t *s) {
  for (int g = 0; g < G; g++)
    for (int n = 0; n < N; n++) {
      int idx = groupwise ? marlin_scale_index_group(n)
                          : marlin_scale_index_single(n);
      s[(size_t)g * N + n] = sp[(size_t)g * N + idx];
    }
}

/* ---------------------------------------------------------- dequantisation */

void marlin_dequant_magic(int32_t q, uint16_t out[4]) {
  const uint32_t LO = 0x000f000fu, HI = 0x00f000f0u, EX = 0x64006400u;
  uint32_t lo = ((uint32_t)q & LO) | EX;
  uint32_t hi = ((uint32_t)q & HI) | EX;
  const uint16_t SUB = 0x6408, MUL = 0x2c00, ADD = 0xd480;
  out[0] = ref_f16_sub((uint16_t)(lo & 0xffff), SUB);
  out[1] = ref_f16_sub((uint16_t)(lo >> 16), SUB);
  out[2] = ref_f16_fma((uint16_t)(hi & 0xffff), MUL, ADD);
  out[3] = ref_f16_fma((uint16_t)(hi >> 16), MUL, ADD);
}

void w4a16_dequant_ref(const int32_t *B, const uint16_t *sp, int K, int N,
                       int groupsize, uint16_t *W) {
  uint8_t *q = (uint8_t *)malloc((size_t)K * N);
  marlin_unpack_weights(B, K, N, q);
  uint16_t zp[16]; /* fp16(q - 8): small integers, exact */
  for (int i = 0; i < 16; i++) zp[i] = ref_f32_to_f16((float)(i - 8));
#pragma omp parallel for schedule(static)
  for (int k = 0; k < K; k++) {
    for (int n = 0; n < N; n++) {
      uint16_t v = zp[q[(size_t)k * N + n]];
      if (groupsize > 0) {
        int g = k / groupsize;
        uint16_t s = sp[(size_t)g * N + marlin_scale_index_group(n)];
        v = ref_f16_mul(v, s);
      }
      W[(size_t)k * N + n] = v;
    }
  }
  free(q);
}

/* -------------------------------------------------------------------- GEMM */

int w4a16_ref_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

int w4a16_gemm_ref(const uint16_t *A, const int32_t *B, const uint16_t *sp,
                   uint16_t *C, int M, int N, int K, int groupsize,
                   int threads) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  uint16_t *Wh = (uint16_t *)malloc((size_t)K * N * 2);
  float *W = (float *)malloc((size_t)K * N * 4);
  if (!Wh || !W) {
    free(Wh);
    free(W);
    return -1;
  }
#ifdef _OPENMP
  int nthreads = threads > 0 ? threads : omp_get_max_threads();
  omp_set_num_threads(nthreads);
#else
  (void)threads;
#endif
  w4a16_dequant_ref(B, sp, K, N, groupsize, Wh);
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)K * N; i++) W[i] = ref_f16_to_f32(Wh[i]);
  free(Wh);

  /* column blocks are independent; every (m,n) accumulates in ascending k */
  const int NB = 256;
  int nblocks = (N + NB - 1) / NB;
#pragma omp parallel for schedule(dynamic) collapse(2)
  for (int m = 0; m < M; m++) {
    for (int nb = 0; nb < nblocks; nb++) {
      float acc[256];
      int n0 = nb * NB;
      int w = N - n0 < NB ? N - n0 : NB;
      for (int j = 0; j < w; j++) acc[j] = 0.0f;
      for (int k = 0; k < K; k++) {
        float a = ref_f16_to_f32(A[(size_t)m * K + k]);
        const float *wrow = W + (size_t)k * N + n0;
        for (int j = 0; j < w; j++) acc[j] += a * wrow[j];
      }
      for (int j = 0; j < w; j++) {
        uint16_t c = ref_f32_to_f16(acc[j]);
        if (groupsize <= 0)
          c = ref_f16_mul(c, sp[marlin_scale_index_single(n0 + j)]);
        C[(size_t)m * N + n0 + j] = c;
      }
    }
  }
  free(W);
  return 0;
}

void w4a16_gemm_ref_f64(const uint16_t *A, const int32_t *B,
                        const uint16_t *sp, double *C, int M, int N, int K,
                        int groupsize) {
  int words = 2 * N;
  for (size_t i = 0; i < (size_t)M * N; i++) C[i] = 0.0;
  for (int kt = 0; kt < K / 16; kt++)
    for (int w = 0; w < words; w++) {
      uint32_t word = (uint32_t)B[(size_t)kt * words + w];
      for (int e = 0; e < 8; e++) {
        int k, n;
        marlin_weight_coord(kt, w, e, &k, &n);
        double wq = (double)((int)((word >> (4 * e)) & 0xf) - 8);
        double wv;
        if (groupsize > 0) {
          uint16_t s =
              sp[(size_t)(k / groupsize) * N + marlin_scale_index_group(n)];
          wv = (double)ref_f16_to_f32(ref_f64_to_f16(wq * ref_f16_to_f32(s)));
        } else {
          wv = wq;
        }
        for (int m = 0; m < M; m++)
          C[(size_t)m * N + n] +=
              (double)ref_f16_to_f32(A[(size_t)m * K + k]) * wv;
      }
    }
  if (groupsize <= 0)
    for (int m = 0; m < M; m++)
      for (int n = 0; n < N; n++)
        C[(size_t)m * N + n] *=
            (double)ref_f16_to_f32(sp[marlin_scale_index_single(n)]);
}

/* --------------------------------------------------------------- quantiser */

/* marlin_test.py:18-55 */
void gen_quant4_ref(const uint16_t *w, int K, int N, int groupsize,
                    uint8_t *q, uint16_t *s, uint16_t *ref) {
  int gs = groupsize > 0 ? groupsize : K;
  int G = K / gs;
  const float two_over_maxq = (float)(2.0 / 15.0);
  for (int g = 0; g < G; g++)
    for (int n = 0; n < N; n++) {
      float mx = 0.0f;
      for (int k = g * gs; k < (g + 1) * gs; k++) {
        float v = fabsf(ref_f16_to_f32(w[(size_t)k * N + n]));
        if (v > mx) mx = v;
      }
      uint16_t sh = ref_f32_to_f16(mx * two_over_maxq);
      s[(size_t)g * N + n] = sh;
      float sf = ref_f16_to_f32(sh);
      for (int k = g * gs; k < (g + 1) * gs; k++) {
        /* half / half evaluated in float, rounded to half, then
         * round-half-to-even to an integer */
        float ratio = ref_f16_to_f32(
            ref_f32_to_f16(ref_f16_to_f32(w[(size_t)k * N + n]) / sf));
        int qi = (int)nearbyintf(ratio) + 8;
        if (qi < 0) qi = 0;
        if (qi > 15) qi = 15;
        q[(size_t)k * N + n] = (uint8_t)qi;
        ref[(size_t)k * N + n] =
            ref_f16_mul(ref_f32_to_f16((float)(qi - 8)), sh);
      }
    }
}

/* ------------------------------------------------ dense fp16 GEMM ("TN") */

/* C[m][n] = fp16( sum_k A[m][k] * B[n][k] ), fp32 accumulation in ascending k:
 * the problem of the reference's gemm/streamk_gemm (gemm_streamk.cu:27-33,
 * A row-major, B column-major k x n = n rows of k, alpha 1, beta 0). */
int f16_gemm_tn_ref(const uint16_t *A, const uint16_t *B, uint16_t *C, int M,
                    int N, int K, int threads) {
  if (M <= 0 || N <= 0) return 0;
#ifdef _OPENMP
  omp_set_num_threads(threads > 0 ? threads : omp_get_max_threads());
#else
  (void)threads;
#endif
  float *Af = (float *)malloc((size_t)M * (K > 0 ? K : 1) * 4);
  float *Bf = (float *)malloc((size_t)N * (K > 0 ? K : 1) * 4);
  if (!Af || !Bf) {
    free(Af);
    free(Bf);
    return -1;
  }
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)M * K; i++) Af[i] = ref_f16_to_f32(A[i]);
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)N * K; i++) Bf[i] = ref_f16_to_f32(B[i]);
#pragma omp parallel for schedule(dynamic, 16) collapse(2)
  for (int m = 0; m < M; m++)
    for (int n = 0; n < N; n++) {
      const float *a = Af + (size_t)m * K, *b = Bf + (size_t)n * K;
      float acc = 0.0f;
      for (int k = 0; k < K; k++) acc += a[k] * b[k];
      C[(size_t)m * N + n] = ref_f32_to_f16(acc);
    }
  free(Af);
  free(Bf);
  return 0;
}

/* -------------------------------------------------------------- comparison */

void w4a16_compare(const uint16_t *C, const uint16_t *Cref, size_t n,
                   w4a16_compare_t *out) {
  double max_err = 0, max_ref = 0, sum_err = 0, sum_ref = 0;
  double xy = 0, xx = 0, yy = 0;
  long long mism = 0;
  int saw_nan = 0;
  for (size_t i = 0; i < n; i++) {
    double x = ref_f16_to_f32(C[i]);
    double y = ref_f16_to_f32(Cref[i]);
    double d = fabs(x - y);
    if (d != d) saw_nan = 1;
    if (d > max_err) max_err = d;
    if (fabs(y) > max_ref) max_ref = fabs(y);
    sum_err += d;
    sum_ref += fabs(y);
    xy += x * y;
    xx += x * x;
    yy += y * y;
    if (C[i] != Cref[i]) mism++;
  }
  out->max_abs_err = saw_nan ? NAN : max_err; /* a NaN anywhere fails */
  out->max_abs_ref = max_ref;
  out->rel_mean_abs_err = sum_ref > 0 ? sum_err / sum_ref : sum_err;
  out->cosine = xy / (sqrt(xx + 1e-5) * sqrt(yy + 1e-5));
  out->mismatched_bits = mism;
}
