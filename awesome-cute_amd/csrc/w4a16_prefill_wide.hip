// Prefill W4A16 kernel with one wave per SIMD: 128-row x 256-column tiles of C
// for launches that are bound by the matrix pipe and by what competes with it.
//
// A workgroup of four waves owns a 128 x 256 tile (and, like the other prefill
// kernel, one of `ksplit` slices of the k range when tiles alone would leave
// compute units idle).  Wave (nw, kh) computes the 128-column half nw of the
// tile over the k half kh of the workgroup's range: a 128 x 128 fp32
// accumulator, all 256 AGPRs, which is why there is one wave per SIMD.  The
// two k halves are added through LDS at the end.
//
// What this shape buys over eight waves with 128 x 64 accumulators:
//   - The packed weights never pass through LDS.  A wave's 128 columns are two
//     whole 64-column Marlin blocks, so MFMA lane (kg, nu) loads the 16-byte
//     piece of Marlin lane (t = kg, c = nu%8) of block nu/8 straight into
//     registers (coalesced: a wave instruction reads 1 KiB of one packed row),
//     and its four words are the operands of the four 16-column groups.
//   - Every activation operand read from LDS (one ds_read_b128) feeds eight
//     MFMAs instead of four, and every unpacked weight word still meets all
//     eight row blocks.
// Per 32-deep k step a wave issues 64 MFMAs, 8 LDS operand reads, 2 weight
// loads and the unpack of 8 packed words (104 VALU instructions with group
// scales), dealt out two behind every MFMA; the activation slab of a 64-deep
// stage (128 rows, staged through registers into two LDS slabs per k half, in
// the k-slot order of the weight layout) costs a thread 8 loads and 16 LDS
// writes per 128 MFMAs.
//
// Prologue, main loop and the hand-over of the accumulators are one assembly
// statement with fixed registers, written by gen_prefill_wide.py (which also
// documents the register map and the schedule); the build runs it.  The code
// here computes what the statement takes in and finishes the tile.
#include <type_traits>

#include "w4a16_common.hpp"

namespace w4a16 {

namespace {

constexpr int kWdTileM = 128;
constexpr int kWdTileN = 256;
constexpr int kWdRB = 8;                              // row blocks of 16
constexpr int kWdRing = 2;                            // activation slabs in LDS per k half
constexpr int kWdPlane = kWdTileM * 16;               // one k group of a step: rows x 16 bytes
constexpr int kWdStepBytes = 4 * kWdPlane + 128;      // one 32-deep k step of a slab (+pad)
constexpr int kWdSlabBytes = 2 * kWdStepBytes;        // a 64-deep stage
constexpr int kWdRingBytes = kWdRing * kWdSlabBytes;  // per k half
constexpr int kWdPitch = kWdTileN * 2 + 16;           // fp16 tile row in LDS on the way out
// the epilogue reuses the rings: 4 waves x 4 row blocks x 8 KiB of fp32 to
// swap between the k halves, then the fp16 tile with padded rows
constexpr int kWdSwapBytes = 4 * 4 * 8 * 1024;
constexpr int kWdLdsBytes = kWdSwapBytes > 2 * kWdRingBytes ? kWdSwapBytes : 2 * kWdRingBytes;
static_assert(kWdTileM * kWdPitch <= kWdLdsBytes, "");
constexpr int kOobWd = (int)0x80000000;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t wd_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// the four words of a raw buffer resource: 48-bit base, stride 0, size in
// bytes, data format flags
__device__ __forceinline__ i4 wd_rsrc_words(const void* p, unsigned bytes) {
  const unsigned long long a = (unsigned long long)p;
  return (i4){(int)(unsigned)a, (int)(unsigned)((a >> 32) & 0xffffu), (int)bytes, 0x00020000};
}

}  // namespace

template <bool GROUP>
__global__ __launch_bounds__(256) void prefill_wide_kernel(GemmArgs p, int tiles_m, int tiles_n,
                                                           int ksplit) {
  extern __shared__ __attribute__((aligned(16))) char smem_all[];  // kWdLdsBytes
  __shared__ int s_ticket;
  {
    // fetch every kernel argument in one round trip
    const void *a_ = p.A, *b_ = p.B, *s_ = p.S;
    void* c_ = p.C;
    int* l_ = p.locks;
    float* sc_ = p.scratch;
    asm volatile("" ::"s"(a_), "s"(b_), "s"(s_), "s"(c_), "s"(l_), "s"(sc_), "s"(p.M), "s"(p.N),
                 "s"(p.K), "s"(tiles_m), "s"(tiles_n), "s"(ksplit));
  }
  constexpr int RB = kWdRB, HB = RB / 2;

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int kh = wave >> 1;  // k half
  const int nw = wave & 1;   // 128-column half of the tile
  const int tid = threadIdx.x & 127;  // thread within the k half
  const int lane = threadIdx.x & 63;
  const int kg = lane >> 4;
  const int nu = lane & 15;
  char* smem = smem_all + kh * kWdRingBytes;

  // Same numbering of the work as the other prefill kernel: every XCD
  // (workgroup id mod 8) gets a contiguous run of tile numbers, tiles are
  // numbered in panels of 8 column tiles with the row tile next, and the k
  // slices of a tile are consecutive work indices.
  const int total = tiles_m * tiles_n * ksplit;
  int work = (int)blockIdx.x;
  if ((total & 7) == 0) work = (work & 7) * (total >> 3) + (work >> 3);
  const int tile = work / ksplit;
  const int ks = work - tile * ksplit;
  int tm, tn;
  if ((tiles_n & 7) == 0) {
    const int per_panel = 8 * tiles_m;
    const int panel = tile / per_panel, within = tile - panel * per_panel;
    tm = within >> 3;
    tn = panel * 8 + (within & 7);
  } else {
    tm = tile / tiles_n;
    tn = tile - tm * tiles_n;
  }
  const int m0 = tm * kWdTileM;
  const int rows = min(kWdTileM, p.M - m0);

  // raw buffer resources (base, no stride, bytes, flags) as the words the
  // assembly takes; the A resource covers the rows of this tile only
  const i4 rb_words = wd_rsrc_words(p.B, (unsigned)p.K * (unsigned)(p.N / 2));
  const i4 rs_words = wd_rsrc_words(p.S, (unsigned)(GROUP ? p.K / 128 : 1) * (unsigned)p.N * 2u);
  i4 ra_words =
      wd_rsrc_words((const char*)p.A + (size_t)m0 * p.K * 2, (unsigned)rows * (unsigned)p.K * 2u);
  const int b_row = p.N * 8;  // bytes per packed row (16 k of every column)

  // packed weights: piece of Marlin lane (t = kg, c = nu%8) of block 2nw + nu/8
  const int b_lane = 2048 * tn + 1024 * nw + 64 * nu + 16 * kg;
  // group scales: the 8 halfs at 8*nu of the permuted row are those of columns
  // 64(nu/8) + 16j + 8h + nu%8, in the order 2j + h
  const int s_lane = (256 * tn + 128 * nw) * 2 + 16 * nu;

  // slab staging: thread (row = tid/8 + 16 i', chunk x = tid%8) moves 16 bytes,
  // i' = (i + 4 kh) % 8: the second k half keeps its row blocks rotated by four,
  // so that in both halves accumulator blocks 0..3 are the ones the wave
  // finishes and 4..7 the ones it hands to the other half.  Rows past the end
  // of A read as zeros (out-of-range buffer offset).
  const int ax = tid & 7;
  int a_lane[RB];
#pragma unroll
  for (int i = 0; i < RB; i++) {
    const int r = (tid >> 3) + 16 * ((i + 4 * kh) & 7);
    a_lane[i] = r < rows ? r * p.K * 2 + 16 * ax : kOobWd;
  }
  // LDS slab: [step][k group][row][slot] dwords; chunk x -> step x/4, slot x%4
  const int lds_wr =
      (int)(size_t)(smem + (ax >> 2) * kWdStepBytes + (tid >> 3) * 16 + (ax & 3) * 4);
  const int lds_rd = (int)(size_t)(smem + kg * kWdPlane + nu * 16);
  // where this wave leaves accumulator blocks 4..7 for the other k half
  const int lds_swap = (int)(size_t)(smem_all + wave * (HB * 8 * 1024) + lane * 16);

  // this half's stages: [s_begin, s_end) of the K/64 stages; the loop runs the
  // same count in both halves (a stage past s_end fetches zeros)
  const int stages_all = p.K / 64;
  const int st0 = (int)((unsigned)ks * (unsigned)stages_all / (unsigned)ksplit);
  const int st1 = (int)((unsigned)(ks + 1) * (unsigned)stages_all / (unsigned)ksplit);
  const int half_stages = (st1 - st0 + 1) >> 1;
  const int s_begin = st0 + kh * half_stages;
  const int s_end = kh ? st1 : st0 + half_stages;
  const int stages = half_stages;
  const int s_row = p.N * 2;  // bytes per row of group scales

  f4 fin[HB][8];  // accumulator blocks 0..3: row blocks own .. own+3 of the tile
#if defined(__HIP_DEVICE_COMPILE__)
  if constexpr (GROUP) {
#include "w4a16_prefill_wide_group.inc"
  } else {
#include "w4a16_prefill_wide_chan.inc"
  }
#else  // the host pass only needs the launch stub
  (void)rb_words, (void)rs_words, (void)ra_words, (void)b_row, (void)b_lane, (void)s_lane;
  (void)lds_wr, (void)lds_rd, (void)lds_swap, (void)s_begin, (void)s_end, (void)stages;
  (void)s_row, (void)a_lane;
  for (auto& r : fin)
    for (auto& v : r) v = (f4){0.f, 0.f, 0.f, 0.f};
#endif
  // the other k half's sums of the same row blocks
  __syncthreads();
  {
    const f4* in = (const f4*)smem_all + (size_t)(wave ^ 2) * (HB * 8 * 64);
#pragma unroll
    for (int i = 0; i < HB; i++)
#pragma unroll
      for (int o = 0; o < 8; o++) fin[i][o] += in[(i * 8 + o) * 64 + lane];
  }

  // ---- k slices of other workgroups: every slice writes its fp32 tile through
  // to memory (whole 1 KiB lines per wave instruction), waits for the
  // acknowledgement, takes the tile's ticket; the last arrival adds all slices
  // in slice order (its own from registers at its place in that order) and
  // carries on.  Nobody spins.
  if (ksplit > 1) {
    constexpr int part_bytes = kWdTileM * kWdTileN * 4;
    const __amdgpu_buffer_rsrc_t rP = wd_rsrc(p.scratch, 0x7fffffffu);
    const int at = (wave * (HB * 8) * 64 + lane) * 16;
    const int mine = work * part_bytes;
#pragma unroll
    for (int i = 0; i < HB; i++)
#pragma unroll
      for (int o = 0; o < 8; o++)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, fin[i][o]), rP,
                                               at + (i * 8 + o) * 1024, mine, 16 /* sc1 */);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): my stores have been acknowledged
    __syncthreads();
    if (threadIdx.x == 0)
      s_ticket = __hip_atomic_fetch_add(&p.locks[tile], 1, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != ksplit - 1) return;  // a later slice finishes the tile
    // one row block at a time keeps the live registers few
#pragma unroll
    for (int i = 0; i < HB; i++) {
      f4 sum[8];
      for (int k2 = 0; k2 < ksplit; k2++) {
        f4 v[8];
        if (k2 != ks) {
          const int theirs = (tile * ksplit + k2) * part_bytes;
#pragma unroll
          for (int o = 0; o < 8; o++)
            v[o] = __builtin_bit_cast(
                f4, __builtin_amdgcn_raw_buffer_load_b128(rP, at + (i * 8 + o) * 1024, theirs,
                                                          16 /* sc1 */));
        } else {
#pragma unroll
          for (int o = 0; o < 8; o++) v[o] = fin[i][o];
        }
#pragma unroll
        for (int o = 0; o < 8; o++) sum[o] = k2 == 0 ? v[o] : sum[o] + v[o];
      }
#pragma unroll
      for (int o = 0; o < 8; o++) fin[i][o] = sum[o];
    }
    if (threadIdx.x == 0)  // counters are handed back zeroed
      __hip_atomic_store(&p.locks[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();

  // fp16 tile -> LDS in row-major order, then whole 512-byte rows go out with
  // coalesced 16-byte stores.  A lane holds row 16 i + nu and, per operand
  // (j, h), the four consecutive columns 64(q/2) + 16j + 8h + 4(q%2) + r of its
  // wave's 128, q = lane/16.
  const int q = lane >> 4;
  const int own = HB * kh;  // first row block this wave finishes
#pragma unroll
  for (int o = 0; o < 8; o++) {
    const int nloc = 128 * nw + 64 * (q >> 1) + 16 * (o >> 1) + 8 * (o & 1) + 4 * (q & 1);
    h4 sc = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
    if (!GROUP) {
      const half_t* S = (const half_t*)p.S;
#pragma unroll
      for (int r = 0; r < 4; r++) sc[r] = S[scale_index_single(kWdTileN * tn + nloc + r)];
    }
#pragma unroll
    for (int i = 0; i < HB; i++) {
      const int m = 16 * (own + i) + nu;
      h4 v = {(half_t)fin[i][o][0], (half_t)fin[i][o][1], (half_t)fin[i][o][2],
              (half_t)fin[i][o][3]};
      if (!GROUP) v *= sc;
      *(h4*)(smem_all + m * kWdPitch + nloc * 2) = v;
    }
  }
  __syncthreads();
  half_t* C = (half_t*)p.C;
#pragma unroll
  for (int it = 0; it < kWdTileM / 8; it++) {
    const int piece = it * 256 + (int)threadIdx.x;  // 16-byte piece of the tile
    const int m = piece >> 5;
    const int c16 = piece & 31;
    if (m < rows) {
      const i4 v = *(const i4*)(smem_all + m * kWdPitch + c16 * 16);
      // nobody reads C again in this launch: keep it out of the way of A and B in L2
      __builtin_nontemporal_store(v, (i4*)(C + (size_t)(m0 + m) * p.N + kWdTileN * tn + c16 * 8));
    }
  }
}

int configure_prefill_wide_kernels() {
  if (hipFuncSetAttribute((const void*)prefill_wide_kernel<true>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, kWdLdsBytes) != hipSuccess ||
      hipFuncSetAttribute((const void*)prefill_wide_kernel<false>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, kWdLdsBytes) != hipSuccess)
    return 3;
  return 0;
}

int launch_prefill_wide(const GemmArgs& a, bool group, int ksplit, hipStream_t stream) {
  const int tiles_m = ceil_div(a.M, kWdTileM);
  const int tiles_n = a.N / kWdTileN;
  const dim3 grid(tiles_m * tiles_n * ksplit);
  if (group)
    hipLaunchKernelGGL(prefill_wide_kernel<true>, grid, dim3(256), kWdLdsBytes, stream, a, tiles_m,
                       tiles_n, ksplit);
  else
    hipLaunchKernelGGL(prefill_wide_kernel<false>, grid, dim3(256), kWdLdsBytes, stream, a,
                       tiles_m, tiles_n, ksplit);
  return launch_status();
}

}  // namespace w4a16
