// Shared device/host definitions for the gfx950 W4A16 kernels.
//
// Weight layout (Marlin format, reference marlin.py:119-129): row kt of B holds
// the 16 k-values [16kt, 16kt+16) of every column.  Each 64-column block is 32
// "Marlin lanes" x 16 bytes; lane (t = lane%4, c = lane/4) owns, in its four
// int32 words j = 0..3, the weights k in {2t, 2t+1, 2t+8, 2t+9} of columns
// 16j+c (nibbles 0,4,1,5) and 16j+c+8 (nibbles 2,6,3,7).
//
// Mapping onto one wave64 v_mfma_f32_16x16x32_f16 (weights are the first
// operand, activations the second, so the result is D[column][row]):
//   MFMA lane l = 16*kg + nu reads the 16-byte piece of Marlin lane
//   (t = kg, c = nu%8) of 64-column block nu/8 of a 128-column tile, once for
//   row kt = 2ks and once for row 2ks+1 (ks = index of the 32-deep k step).
//   MFMA (j,h) then has, in lane l, the 8 k-slots
//     32ks + {2kg, 2kg+1, 2kg+8, 2kg+9, 16+2kg, 17+2kg, 24+2kg, 25+2kg}
//   of column 64*(nu/8) + 16j + 8h + nu%8.  Activations are staged in LDS in
//   the same k-slot order, so no cross-lane shuffle of weights is needed.
//   The result lane l holds row m = l%16 and the four "columns" nu = 4*(l/16)+r.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace w4a16 {

typedef _Float16 half_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));
typedef int i2 __attribute__((ext_vector_type(2)));
typedef int i4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kTileN = 128;    // columns handled by one wave-level weight load
constexpr int kGranuleK = 64;  // k depth of one streaming granule (two MFMA k steps)

__device__ __forceinline__ h2 as_h2(int x) { return __builtin_bit_cast(h2, x); }
__device__ __forceinline__ int as_int(h2 x) { return __builtin_bit_cast(int, x); }

// Constants of the int4 -> fp16 conversion, kept in registers so that
// (q & mask) | exponent is one v_and_or_b32.
struct DequantConsts {
  int lo_mask, hi_mask, ex;
  __device__ __forceinline__ DequantConsts() {
    lo_mask = 0x000f000f;
    hi_mask = 0x00f000f0;
    ex = 0x64006400;
    asm volatile("" : "+s"(lo_mask), "+s"(hi_mask), "+v"(ex));
  }
};

// One packed word -> the fp16 weights of column c (lo/hi = k pairs (2t,2t+1)
// and (2t+8,2t+9)) and of column c+8.  fp16(1024+q) - 1032 and
// fp16(1024+16q)/16 - 72 are exact, so the values equal fp16(q - 8) bit for
// bit (the arithmetic of reference marlin_cute_trait.h:20-39).  In group mode
// every weight is then multiplied once by its fp16 scale, rounded to nearest
// (reference marlin_official_kernel.cu:155-159).
template <bool GROUP>
__device__ __forceinline__ void dequant_word(int q, h2 s2, const DequantConsts& dc, h2& lo0,
                                             h2& hi0, h2& lo1, h2& hi1) {
  const h2 sub = {(half_t)1032.f, (half_t)1032.f};
  const h2 mul = {(half_t)0.0625f, (half_t)0.0625f};
  const h2 add = {(half_t)-72.f, (half_t)-72.f};
  int q8 = (int)((unsigned)q >> 8);
  lo0 = as_h2((q & dc.lo_mask) | dc.ex) - sub;
  hi0 = __builtin_elementwise_fma(as_h2((q & dc.hi_mask) | dc.ex), mul, add);
  lo1 = as_h2((q8 & dc.lo_mask) | dc.ex) - sub;
  hi1 = __builtin_elementwise_fma(as_h2((q8 & dc.hi_mask) | dc.ex), mul, add);
  if (GROUP) {
    h2 s0 = {s2[0], s2[0]};
    h2 s1 = {s2[1], s2[1]};
    lo0 *= s0;
    hi0 *= s0;
    lo1 *= s1;
    hi1 *= s1;
  }
}

__device__ __forceinline__ h8 make_h8(h2 a, h2 b, h2 c, h2 d) {
  h8 r = {a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
  return r;
}

// Position, inside a packed per-channel scale row, of the scale of logical
// column n (inverse of the 32-column permutation of reference marlin.py:52-54).
__host__ __device__ __forceinline__ int scale_index_single(int n) {
  int b = n >> 5, u = n & 31;
  return 32 * b + 8 * ((u & 7) >> 1) + 2 * (u >> 3) + (u & 1);
}

__device__ __forceinline__ unsigned pack_half2(float a, float b) {
  h2 v = {(half_t)a, (half_t)b};
  return (unsigned)as_int(v);
}

// ---------------------------------------------------------------------------
// Stream-K partition of the streaming kernel.  The work of one launch is the
// linear space of NT * KG granules (column tile major, k minor); the workgroup
// with work index b owns granules [b*gpb, (b+1)*gpb).  A column tile whose granules fall into
// more than one workgroup is finished by whichever of them arrives last at the
// tile's counter.
//
// Second form (wpt > 0): every column tile is cut into wpt nearly equal runs,
// one per workgroup: work index w owns run w % wpt of tile w / wpt.  This keeps
// every workgroup inside one tile for any KG, where the first form can only do
// so when gpb divides KG.
struct StreamPlan {
  int NT;    // 128-column tiles
  int KG;    // 64-deep granules per tile
  int gpb;   // granules per workgroup (the most, when wpt > 0)
  int grid;  // workgroups launched (all own at least one granule)
  int wpt;   // workgroups per tile, or 0 for the first form
};

__host__ __device__ __forceinline__ int ceil_div(int a, int b) { return (a + b - 1) / b; }

__host__ __device__ inline StreamPlan make_stream_plan(int N, int K, int want_grid) {
  StreamPlan p;
  p.NT = N / kTileN;
  p.KG = K / kGranuleK;
  int total = p.NT * p.KG;
  if (want_grid < 1) want_grid = 1;
  if (want_grid > total) want_grid = total;
  p.gpb = ceil_div(total, want_grid);
  p.grid = ceil_div(total, p.gpb);
  p.wpt = 0;
  return p;
}

// The hardware deals workgroups to the 8 XCDs round-robin (blockIdx % 8) and
// every XCD has an L2 of its own.  Workgroup blockIdx takes the work index
// below, so that consecutive work indices (the sharers of a column tile) sit
// behind one L2 and read the same activation and scale lines through it
// (measured: up to 1 us per launch at 16 rows).  A placement hint only:
// nothing depends on where a workgroup really runs.
__host__ __device__ __forceinline__ int xcd_work_index(int block, int grid) {
  const int x = block & 7, q = grid >> 3, rem = grid & 7;
  return x * q + (x < rem ? x : rem) + (block >> 3);
}
// first / last workgroup (by work index) touching tile t
__host__ __device__ __forceinline__ int tile_first_block(const StreamPlan& p, int t) {
  return (t * p.KG) / p.gpb;
}
__host__ __device__ __forceinline__ int tile_last_block(const StreamPlan& p, int t) {
  return ((t + 1) * p.KG - 1) / p.gpb;
}

// Partial-sum slots: two per workgroup.  In the first form a workgroup owns at
// most two tiles that it shares with others (its first and its last), whose
// partial sums go to slot 2b and 2b+1; in the second form it has one tile and
// uses slot 2b only (slots 16 KiB apart measured 0.1-0.2 us faster per launch
// than slots packed 8 KiB apart at 1-16 rows).
__host__ __device__ __forceinline__ int partial_slot(const StreamPlan& p, int block, int t) {
  if (p.wpt > 0) return 2 * block;
  // block touches tile t; t is its first tile unless the block starts before it
  return 2 * block + (block * p.gpb < t * p.KG ? 1 : 0);
}
// slots a launch of plan p may touch
__host__ __device__ __forceinline__ int stream_slots(const StreamPlan& p) { return 2 * p.grid; }

struct GemmArgs {
  const void* A;    // (M, K) fp16 row-major
  const void* B;    // (K/16, 2N) int32, Marlin format
  void* C;          // (M, N) fp16 row-major
  const void* S;    // (K/128, N) or (1, N) fp16, Marlin-permuted
  int M, N, K;
  int* locks;       // N/128 counters, lock_stride ints apart; zero on entry and on exit
  int lock_stride;  // >= 1; spreads the counters over separate cache lines
  float* scratch;   // partial sums of shared tiles (null if no tile is shared)
  int gpb;          // granules per workgroup (streaming kernel; the most, when wpt > 0)
  int wpt;          // workgroups per column tile, or 0 (see StreamPlan)
  int row_parts;    // streaming kernel, wpt > 0: 1, or the number of parts the rows are cut
                    // into, `part_rows` each (the last one the rest), that separate
                    // workgroups compute: wpt workgroups per column tile and part; needs
                    // lock_stride >= row_parts.  Column-strip kernel: 1, or the number
                    // of 16-row parts, a workgroup per strip set and part
  int part_rows;    // rows of a part: 16 or 32
};

// bytes of fp32 partial sums of mb row blocks of 16 (one slot)
constexpr size_t stream_slot_bytes(int mb) { return (size_t)mb * 4 * 2 * 64 * 16; }

// Result of a kernel launch for the launch helpers below: 0, or 3 with the
// runtime's error kept per thread for the caller's message (reading the
// runtime's error state clears it, so the helper that reads it must keep it).
hipError_t& last_launch_error();
inline int launch_status() {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) last_launch_error() = e;
  return e == hipSuccess ? 0 : 3;
}

// Per-device set-up of the kernels that need more dynamic LDS than the default
// limit; call once with the device current before the first launch on it.
int configure_stream_kernels();
int configure_prefill_kernels();

int launch_stream(const GemmArgs& a, bool group, int grid, hipStream_t stream);
// at most kStripMaxRows rows, 16 x a.row_parts at most; a workgroup per
// `strips` (1 to 4) 16-column strips and 16-row part over the whole k range,
// nothing exchanged between workgroups (w4a16_strip.hip)
constexpr int kStripMaxRows = 1024;
int configure_strip_kernels();
int launch_strip(const GemmArgs& a, bool group, int strips, hipStream_t stream);
// ksplit >= 1 slices of the k range per tile; above 1 the launch needs
// a.scratch (ksplit * tiles * tile bytes of fp32) and a.locks (one zeroed
// counter per tile, zero again afterwards)
// 64-row x 256-column tiles, eight waves (w4a16_prefill.hip)
int launch_prefill(const GemmArgs& a, bool group, int ksplit, hipStream_t stream);
// 128-row x 256-column tiles, four waves with 128 x 128 accumulators
// (w4a16_prefill_wide.hip); same scratch layout and counters
int configure_prefill_wide_kernels();
int launch_prefill_wide(const GemmArgs& a, bool group, int ksplit, hipStream_t stream);

}  // namespace w4a16
