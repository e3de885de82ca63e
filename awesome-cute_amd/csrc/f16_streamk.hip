// Dense fp16 GEMM with a stream-K tail for gfx950: C (m x n, row-major) =
// A (m x k, row-major) * B^T with B given as n rows of k ("TN": both operands
// k-contiguous), fp32 accumulation, alpha = 1, beta = 0 -- the problem of the
// reference's gemm/streamk_gemm (gemm_streamk.cu:8-110), with the same split
// of the output tiles into a data-parallel part and a stream-K part
// (dp_sk_block.h:82-128, strategy sk1tile_dp): tiles that fill whole waves of
// compute units are computed by one workgroup each; the tiles of the last,
// partial wave are cut along k into slices, one workgroup per slice, and the
// slices of a tile meet through fp32 partial sums in memory and a counter.
// Unlike the reference's turnstile (gemm_streamk.h:562-590: every block waits
// for the one before it) nobody waits: a slice writes its partial tile through
// to memory, takes a ticket, and the last arrival adds all slices in slice
// order and writes C.
//
// Kernel: a workgroup of 8 waves (2 x 4, two per SIMD) owns a 256 x 256 tile
// of C; a wave holds a 128 x 64 fp32 accumulator (128 registers).  Problems
// with too few such tiles for the compute units run on 128 x 256 or 128 x 128
// tiles (same eight waves, a wave's share 64 x 64 or 64 x 32).  With B as
// the first MFMA operand and A as the second, v_mfma_f32_16x16x32_f16 yields
// D[n][m]; lane l = 16kg + nu of an operand holds k = 8kg ... 8kg+7 of row nu.
// Per 64-deep k stage (two MFMA k steps) the workgroup brings a 256 x 64 slab
// of A and of B into a ring of LDS slabs (two; three or four for the smaller
// tiles, whose stages are shorter than a load's latency) with buffer loads that write LDS
// directly (16 bytes per lane, lane l at 16*l).  Eight lanes fetch the whole
// 128-byte k run of a row -- one cache line; with 64-byte runs every line
// came in twice and the loads alone bounded the kernel -- so a slab is
// row-major with 128-byte rows.  To keep the operand reads (lane (kg, nu):
// 16 bytes at chunk 4h + kg of row nu, one ds_read_b128) free of bank
// conflicts, the chunk stored at position c of row r is chunk c ^ (r % 8);
// since the hardware fixes where a lane's bytes land, the swizzle is applied
// to the address the lane fetches.  A slab is requested at least a whole stage
// before it is needed; one barrier per stage.  The compiler cannot know which slab a
// load in flight writes, so the LDS reads of the main loop and their waits are
// written by hand (LDS reads return in order).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <mutex>
#include <type_traits>
#include <vector>

#include "../../include/streamk_amd.h"
#include "scratch_pool.hpp"
#include "w4a16_common.hpp"

namespace w4a16 {

namespace {

constexpr int kDnTile = 256;     // columns of a tile of C, and rows of the large tile
constexpr int kDnStageK = 64;    // k depth of a stage (two MFMA k steps)
constexpr int kDnOob = (int)0x80000000;

// LDS geometry for tiles of TM rows and TN columns (256 x 256; 128 x 256 or
// 128 x 128 when larger tiles are too few for the compute units): a slab is
// TM rows of A and TN rows of B
template <int TM, int TN>
struct DnShape {
  static constexpr int kSlabA = TM * 128;
  static constexpr int kSlab = kSlabA + TN * 128;
  // slabs in LDS.  A stage of a small tile is shorter than a load's way from
  // L2 (0.4 us of MFMAs for 128 x 128), so its slabs are requested further ahead.
  static constexpr int kRing = TM * TN == 128 * 128 ? 4 : (TM * TN == 128 * 256 ? 3 : 2);
  static constexpr int kLds = kRing * kSlab;
  static constexpr int kRB = TM / 32;  // 16-row blocks per wave
  static constexpr int kNJ = TN / 64;  // 16-column blocks per wave
  static constexpr int kPartBytes = TM * TN * 4;
};
constexpr int kDnMaxSlots = 256;                     // slices in flight per launch
constexpr int kDnMaxSlices = 4;

struct DenseArgs {
  const void* A;
  const void* B;
  void* C;
  int M, N, K;
  int tile_rows;  // 256 or 128
  int tile_cols;  // 256 or 128
  int tiles_m, tiles_n;
  int dp_tiles;  // tiles computed by one workgroup each
  int sk_tiles;  // tiles (the last ones in tile order) cut into ksplit slices
  int ksplit;
  int* locks;      // one zeroed counter per stream-K tile, zero again afterwards
  float* scratch;  // kDnPartBytes per slice
};

// Tiles are numbered panel by panel: a panel is kDnPanel column tiles wide
// (the last one narrower), and inside a panel the column tile runs fastest.
// A run of consecutive tile numbers then covers a compact block of C, so the
// workgroups that share an L2 read few distinct rows of A and B.
constexpr int kDnPanel = 8;
__host__ __device__ __forceinline__ void dn_tile_coord(int t, int tiles_m, int tiles_n, int* tm,
                                                       int* tn) {
  const int per_panel = tiles_m * kDnPanel;
  const int p = t / per_panel;
  const int first = p * kDnPanel;
  const int width = tiles_n - first < kDnPanel ? tiles_n - first : kDnPanel;
  const int o = t - p * per_panel;
  *tm = o / width;
  *tn = first + o - *tm * width;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t dn_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// 16 bytes per lane from a buffer straight into LDS: lane l's bytes land at
// dst + 16*l (dst is wave-uniform).  The instruction's immediate offset stays
// zero: the hardware would add it to the LDS address as well.  (Device pass
// only; the host pass just needs the kernel's launch stub.)
__device__ __forceinline__ void dn_dma16(__amdgpu_buffer_rsrc_t rsrc, char* dst, int voffset,
                                         int soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef __attribute__((address_space(3))) void* lds_ptr;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr)dst, 16, voffset, soffset, 0, 0);
#endif
}

// LDS reads of the main loop, outside the compiler's dependence tracking
template <int OFF>
__device__ __forceinline__ void dn_read16(unsigned at, i4& v) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(OFF) : "memory");
#endif
}
// wait until at most PENDING later LDS reads are outstanding; `v` is the
// operand the wait is for
template <int PENDING>
__device__ __forceinline__ void dn_wait(i4& v) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(PENDING));
#endif
}
// wait for every LDS read in flight; the operand registers are named so that
// they count as in use up to here
__device__ __forceinline__ void drain_reads(i4 (&a)[2], i4 (&b)[2], i4 (&f)[4]) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]), "+v"(f[0]), "+v"(f[1]), "+v"(f[2]),
                 "+v"(f[3]));
#endif
}
__device__ __forceinline__ void drain_reads(i4 (&a)[4], i4 (&b)[4], i4 (&f)[4]) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]),
                 "+v"(b[3]), "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]));
#endif
}
// s_waitcnt vmcnt(n) lgkmcnt(0) (gfx9 encoding)
constexpr int dn_vm_lgkm0(int n) { return (n & 15) | (7 << 4) | (0 << 8) | ((n >> 4) << 14); }
// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding)
constexpr int dn_vmcnt(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

}  // namespace

template <int TM, int TN>
__global__ __launch_bounds__(512) void dense_kernel(DenseArgs p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];  // DnShape<TM, TN>::kLds
  using Shape = DnShape<TM, TN>;
  constexpr int RB = Shape::kRB;
  constexpr int NJ = Shape::kNJ;
  constexpr int kDnSlabA = Shape::kSlabA;
  constexpr int kDnSlab = Shape::kSlab;
  constexpr int kRing = Shape::kRing;
  constexpr int kDnLds = Shape::kLds;
  constexpr int kPart = Shape::kPartBytes;
  __shared__ int s_ticket;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int kg = lane >> 4;
  const int nu = lane & 15;
  const int wm = wave >> 2;  // row half of the tile
  const int wn = wave & 3;   // column quarter of the tile

  // stream-K slices come first in the grid, so that they run beside the first
  // wave of whole tiles
  const int sk_blocks = p.sk_tiles * p.ksplit;
  const int work = (int)blockIdx.x;
  int tile, ks, ksplit;
  if (work < sk_blocks) {
    tile = p.dp_tiles + work / p.ksplit;
    ks = work % p.ksplit;
    ksplit = p.ksplit;
  } else {
    // The hardware deals workgroups to the 8 XCDs round-robin; give every XCD
    // a contiguous run of tile numbers.  A placement hint only.
    tile = work - sk_blocks;
    if (((sk_blocks | p.dp_tiles) & 7) == 0) tile = (tile & 7) * (p.dp_tiles >> 3) + (tile >> 3);
    ks = 0;
    ksplit = 1;
  }
  int tm, tn;
  dn_tile_coord(tile, p.tiles_m, p.tiles_n, &tm, &tn);
  const int m0 = tm * TM;
  const int n0 = tn * TN;
  const int rows = min(TM, p.M - m0);

  const __amdgpu_buffer_rsrc_t rA =
      dn_rsrc((const char*)p.A + (size_t)m0 * p.K * 2, (unsigned)rows * (unsigned)p.K * 2u);
  const __amdgpu_buffer_rsrc_t rB =
      dn_rsrc((const char*)p.B + (size_t)n0 * p.K * 2, (unsigned)TN * (unsigned)p.K * 2u);

  // wave w fetches rows (TM/8) w ... of the A slab and (TN/8) w ... of the
  // B slab, eight rows per instruction: lane (r = lane/8, c = lane%8) lands at
  // [r][c] and fetches chunk c ^ r of its row.  Rows past the end of A repeat
  // the last row (never stored).
  constexpr int TA = TM / 64;  // A instructions per wave and stage
  constexpr int TB = TN / 64;  // B instructions per wave and stage
  int a_src[TA], b_src[TB];
  {
    const int r8 = lane >> 3, c = (lane & 7) ^ r8;
#pragma unroll
    for (int t = 0; t < TA; t++) {
      const int r = 8 * TA * wave + 8 * t + r8;
      a_src[t] = (r < rows ? r : rows - 1) * p.K * 2 + 16 * c;
    }
#pragma unroll
    for (int t = 0; t < TB; t++) b_src[t] = (8 * TB * wave + 8 * t + r8) * p.K * 2 + 16 * c;
  }
  // this workgroup's stages [st0, st1) of the K/64 stages
  const int stages_all = p.K / kDnStageK;
  // (at most 4 slices of at most 2^24 stages: 32 bits do)
  const int st0 = (int)((unsigned)ks * (unsigned)stages_all / (unsigned)ksplit);
  const int st1 = (int)((unsigned)(ks + 1) * (unsigned)stages_all / (unsigned)ksplit);
  const int stages = st1 - st0;

  auto issue_slab = [&](int s, int ring) {
    const int inv = s < stages ? 0 : kDnOob;  // a stage past the end fetches zeros
    const int at = (st0 + s) * (kDnStageK * 2);
    char* base = smem + ring * kDnSlab;
#pragma unroll
    for (int t = 0; t < TA; t++)
      dn_dma16(rA, base + (8 * TA * wave + 8 * t) * 128, a_src[t] | inv, at);
#pragma unroll
    for (int t = 0; t < TB; t++)
      dn_dma16(rB, base + kDnSlabA + (8 * TB * wave + 8 * t) * 128, b_src[t] | inv, at);
  };
  constexpr int kSlabLoads = TA + TB;  // per wave

  f4 acc[RB][NJ];
#pragma unroll
  for (int i = 0; i < RB; i++)
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};

  i4 w[2][NJ];  // B operands of the two k steps of a stage
  i4 af[4];    // ring of A operands, three ahead of the MFMAs
  // operand addresses in slab 0 for the two k steps
  unsigned a_rd[2], b_rd[2];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const unsigned sw = 16 * ((4 * h + kg) ^ (nu & 7));
    a_rd[h] = (unsigned)(size_t)smem + (16 * RB * wm + nu) * 128 + sw;
    b_rd[h] = (unsigned)(size_t)smem + kDnSlabA + (16 * NJ * wn + nu) * 128 + sw;
  }
  // the NJ B operands of a k step: 16 rows of the slab apart
  auto read_b = [&](unsigned at, i4 (&dst)[NJ]) {
    dn_read16<0>(at, dst[0]);
    dn_read16<2048>(at, dst[1]);
    if constexpr (NJ == 4) {
      dn_read16<4096>(at, dst[2]);
      dn_read16<6144>(at, dst[3]);
    }
  };

  // prologue: slabs 0 ... kRing-1 requested; slab 0 landed (loads complete in
  // order); its first operands read
#pragma unroll
  for (int r = 0; r < kRing; r++) issue_slab(r, r);
  __builtin_amdgcn_s_waitcnt(dn_vmcnt((kRing - 1) * kSlabLoads));
  __builtin_amdgcn_s_barrier();
  read_b(b_rd[0], w[0]);
  dn_read16<0>(a_rd[0], af[0]);
  dn_read16<2048>(a_rd[0], af[1]);
  dn_read16<4096>(a_rd[0], af[2]);

  // One k step (H) of the stage in slab `cur`.  LDS reads in issue order, with
  // Ai the operand of row block i and primes the prefetches for the step after
  // (eight row blocks per wave; with four the same three-ahead pattern):
  //   step 0:  | B(step 1) x NJ  A3 | A4 | A5 | A6 | A7 | A0' | A1' | A2' |
  //   step 1:  | A3 | A4 | A5 | A6 | A7 | barrier, B(next stage) x NJ  A0' | A1' | A2' |
  // When row block i is used, the reads issued after Ai may still be pending:
  // three A operands, plus the NJ B reads where those were issued in between
  // (the three row blocks from the one that issues them).
  // The barrier of a stage sits where the first read from the next slab is
  // about to be issued: by then every wave has its own part of that slab (it
  // waits for its loads first) and has issued and received all its reads of
  // the current slab, which the request for the stage after next overwrites.
  auto kstep = [&](auto H, unsigned cur, unsigned nxt, int s, int slot) {
    constexpr int h = decltype(H)::value;
    constexpr int ib = h ? RB - 3 : 0;  // row block that issues the B reads
    const unsigned ac = a_rd[h] + cur;                        // this step, this slab
    const unsigned an = h ? a_rd[0] + nxt : a_rd[1] + cur;    // the step after
    const unsigned bn = h ? b_rd[0] + nxt : b_rd[1] + cur;
#pragma unroll
    for (int i = 0; i < RB; i++) {
      if (i == ib) {
        if (h == 1) {
          // my loads of the next slab (the slabs after it may still be on
          // their way) and my reads of this one
          __builtin_amdgcn_s_waitcnt(dn_vm_lgkm0((kRing - 2) * kSlabLoads));
          __builtin_amdgcn_s_barrier();
          issue_slab(s + kRing, slot);
        }
        read_b(bn, w[h ^ 1]);
      }
      // operand of row block i + 3: of this step, or of the step after
      auto frag = [&](auto I) {
        constexpr int ii = decltype(I)::value;
        if constexpr (ii < RB)
          dn_read16<ii * 2048>(ac, af[ii & 3]);
        else
          dn_read16<(ii - RB) * 2048>(an, af[ii & 3]);
      };
      switch (i) {  // i is a constant after unrolling
        case 0: frag(std::integral_constant<int, 3>{}); break;
        case 1: frag(std::integral_constant<int, 4>{}); break;
        case 2: frag(std::integral_constant<int, 5>{}); break;
        case 3: frag(std::integral_constant<int, 6>{}); break;
        case 4: frag(std::integral_constant<int, 7>{}); break;
        case 5: frag(std::integral_constant<int, 8>{}); break;
        case 6: frag(std::integral_constant<int, 9>{}); break;
        case 7: frag(std::integral_constant<int, 10>{}); break;
      }
      if (i >= ib && i <= ib + 2)
        dn_wait<3 + NJ>(af[i & 3]);
      else
        dn_wait<3>(af[i & 3]);
      if (i == 0) {
        // the B operands of this step were requested before A0 was
#pragma unroll
        for (int j = 0; j < NJ; j++) asm volatile("" : "+v"(w[h][j]));
      }
      const h8 a = __builtin_bit_cast(h8, af[i & 3]);
#pragma unroll
      for (int j = 0; j < NJ; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, w[h][j]), a,
                                                           acc[i][j], 0, 0, 0);
    }
  };

  int slot = 0;  // ring slot of the stage being computed
  for (int s = 0; s < stages; s++) {
    const int slot_next = slot == kRing - 1 ? 0 : slot + 1;
    const unsigned cur = slot * kDnSlab, nxt = slot_next * kDnSlab;
    kstep(std::integral_constant<int, 0>{}, cur, nxt, s, slot);
    kstep(std::integral_constant<int, 1>{}, cur, nxt, s, slot);
    slot = slot_next;
  }
  // The last k step has requested the operands of a stage that does not
  // exist; they are still on their way into w and af.  Those registers stay
  // taken until the reads have landed: the compiler, which believes they were
  // written when the reads were issued and sees no further use, would
  // otherwise hand them to the code below at once, and a late arrival would
  // overwrite what that code keeps there.
  drain_reads(w[0], w[1], af);
  // Nothing of the ring may still be on its way when LDS is reused.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  // ---- slices of other workgroups: every slice writes its fp32 tile through
  // to memory (whole 1 KiB lines per wave instruction), waits for the
  // acknowledgement and takes the tile's ticket; the last arrival adds all
  // slices in slice order (its own from registers at its place in that order).
  if (ksplit > 1) {
    const __amdgpu_buffer_rsrc_t rP = dn_rsrc(p.scratch, 0x7fffffffu);
    const int at = (wave * (RB * NJ) * 64 + lane) * 16;
    const int mine = work * kPart;
#pragma unroll
    for (int i = 0; i < RB; i++)
#pragma unroll
      for (int j = 0; j < NJ; j++)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, acc[i][j]), rP,
                                               at + (i * NJ + j) * 1024, mine, 16 /* sc1 */);
    __builtin_amdgcn_s_waitcnt(dn_vmcnt(0));  // my stores have been acknowledged
    __syncthreads();
    const int sk_tile = tile - p.dp_tiles;
    if (tid == 0)
      s_ticket = __hip_atomic_fetch_add(&p.locks[sk_tile], 1, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != ksplit - 1) return;  // a later slice finishes the tile
    // one row block at a time: the other slices' values are requested
    // together, then added in slice order with my own at its place
#pragma unroll
    for (int i = 0; i < RB; i++) {
      f4 v[kDnMaxSlices][NJ];
#pragma unroll
      for (int k2 = 0; k2 < kDnMaxSlices; k2++) {
        const int theirs = (sk_tile * ksplit + k2) * kPart;
        const int inv = (k2 < ksplit && k2 != ks) ? 0 : kDnOob;  // no traffic for the rest
#pragma unroll
        for (int j = 0; j < NJ; j++)
          v[k2][j] = __builtin_bit_cast(
              f4, __builtin_amdgcn_raw_buffer_load_b128(rP, (at + (i * NJ + j) * 1024) | inv,
                                                        theirs, 16 /* sc1 */));
      }
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        f4 sum = (ks == 0) ? acc[i][j] : v[0][j];
#pragma unroll
        for (int k2 = 1; k2 < kDnMaxSlices; k2++)
          if (k2 < ksplit) sum += (k2 == ks) ? acc[i][j] : v[k2][j];
        acc[i][j] = sum;
      }
    }
    if (tid == 0)  // counters are handed back zeroed
      __hip_atomic_store(&p.locks[sk_tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- C: a lane holds, per (i, j), row 16i + nu and four consecutive
  // columns.  The fp16 tile goes through LDS (the slabs are dead), one half of
  // its rows at a time, and leaves as whole rows (512 or 256 bytes) with
  // 16-byte stores; 8-byte stores straight from the registers cost 13 us more
  // at 4096^3.
  constexpr int kPitch = TN * 2 + 16;  // bytes per tile row in LDS
  constexpr int HR = TM / 2;           // rows of a half
  constexpr int PR = TN / 8;           // 16-byte pieces of a row
  static_assert(HR * kPitch <= kDnLds, "");
  half_t* C = (half_t*)p.C;
  const int q = lane >> 4;
#pragma unroll
  for (int hlf = 0; hlf < 2; hlf++) {
    __syncthreads();
    if (wm == hlf) {
#pragma unroll
      for (int i = 0; i < RB; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
          const h4 o = {(half_t)acc[i][j][0], (half_t)acc[i][j][1], (half_t)acc[i][j][2],
                        (half_t)acc[i][j][3]};
          *(h4*)(smem + (16 * i + nu) * kPitch + (16 * NJ * wn + 16 * j + 4 * q) * 2) = o;
        }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < HR * PR / 512; it++) {
      const int piece = it * 512 + tid;  // 16-byte piece of the half tile
      const int r = piece / PR, c16 = piece % PR;
      const int m = HR * hlf + r;
      if (m < rows) {
        const i4 v = *(const i4*)(smem + r * kPitch + c16 * 16);
        // nobody reads C again in this launch: keep it out of the way of A and B in L2
        __builtin_nontemporal_store(v, (i4*)(C + (size_t)(m0 + m) * p.N + n0 + c16 * 8));
      }
    }
  }
}

// C = 0 for an empty k range (a kernel rather than a memset, so that the call
// can be captured into a HIP graph like any other)
__global__ void dense_zero_kernel(half_t* C, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) C[i] = (half_t)0.f;
}

}  // namespace w4a16

// ---------------------------------------------------------------------------
// Host side: the tile split, the scratch for partial sums, the C ABI.

namespace {

using namespace w4a16;

constexpr int kDnMaxDevices = 16;

thread_local char g_dn_error[256] = "";

void dn_set_error(hipError_t e, const char* what) {
  snprintf(g_dn_error, sizeof(g_dn_error), "%s: %s", what, hipGetErrorString(e));
}

// Partial sums and tile counters of the stream-K tiles come from the scratch
// pool that the W4A16 path uses too: one buffer per (device, stream), sized by
// the launches that need it.
struct DnDevice {
  int cus = 0;
  bool configured = false;
};
std::mutex g_dn_mu;
DnDevice g_dn[kDnMaxDevices];

struct DnPlan {
  int tile_rows, tile_cols, tiles_m, tiles_n, dp_tiles, sk_tiles, ksplit, grid;
};

// Whole waves of tiles go to one workgroup each; the tiles of the partial last
// wave are cut into as many k slices as there are idle compute units per tile
// (at most four: beyond that the partial-sum traffic of the one workgroup that
// finishes a tile costs more than the slices save), each at least 256 deep.
DnPlan dn_plan(int m, int n, int k, int cus) {
  DnPlan pl;
  // 256 x 256 tiles, unless they would occupy at most half of the compute
  // units: then 128 x 256 tiles, twice as many, and 128 x 128 if that holds
  // for those as well (one workgroup per smaller tile beats k slices of a
  // larger one: no partial sums go through memory)
  pl.tile_rows = pl.tile_cols = kDnTile;
  if (2LL * ceil_div(m, kDnTile) * (n / kDnTile) <= cus) {
    pl.tile_rows = 128;
    if (2LL * ceil_div(m, 128) * (n / kDnTile) <= cus) pl.tile_cols = 128;
  }
  pl.tiles_m = ceil_div(m, pl.tile_rows);
  pl.tiles_n = n / pl.tile_cols;
  const int tiles = pl.tiles_m * pl.tiles_n;
  const int rem = cus > 0 ? tiles % cus : 0;
  int s = 1;
  if (rem > 0) {
    s = cus / rem;
    if (s > kDnMaxSlices) s = kDnMaxSlices;
    if (s > k / 256) s = k / 256;
    while (s > 1 && rem * s > kDnMaxSlots) --s;
    if (s < 1) s = 1;
  }
  pl.ksplit = s;
  pl.sk_tiles = s > 1 ? rem : 0;
  pl.dp_tiles = tiles - pl.sk_tiles;
  pl.grid = pl.dp_tiles + pl.sk_tiles * s;
  return pl;
}

int dn_check(int m, int n, int k) {
  if (m < 0 || n < 0 || k < 0) return STREAMK_ERR_SHAPE;
  if (n % kDnTile != 0 || k % kDnStageK != 0) return STREAMK_ERR_SHAPE;
  return STREAMK_OK;
}

}  // namespace

extern "C" {

int streamk_gemm_tn(const void* A, const void* B, void* C, int m, int n, int k, int dev,
                    void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  int rc = dn_check(m, n, k);
  if (rc != STREAMK_OK || m == 0 || n == 0) return rc;
  if (k == 0) {  // an empty sum
    const size_t count = (size_t)m * n;
    hipLaunchKernelGGL(dense_zero_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0,
                       stream, (half_t*)C, count);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      dn_set_error(e, "kernel launch");
      return STREAMK_ERR_RUNTIME;
    }
    return STREAMK_OK;
  }
  // a tile's rows of A and of B are addressed with 32-bit byte offsets
  if ((long long)kDnTile * k * 2 > 0x7fffffffLL) {
    snprintf(g_dn_error, sizeof(g_dn_error), "k = %d is too deep for 32-bit tile offsets", k);
    return STREAMK_ERR_RUNTIME;
  }
  if (dev < 0 || dev >= kDnMaxDevices) {
    snprintf(g_dn_error, sizeof(g_dn_error), "device index %d out of range", dev);
    return STREAMK_ERR_RUNTIME;
  }
  int prev = -1;
  hipError_t e = hipGetDevice(&prev);
  if (e != hipSuccess) {
    dn_set_error(e, "hipGetDevice");
    return STREAMK_ERR_RUNTIME;
  }
  if (prev != dev && (e = hipSetDevice(dev)) != hipSuccess) {
    dn_set_error(e, "hipSetDevice");
    return STREAMK_ERR_RUNTIME;
  }
  rc = STREAMK_ERR_RUNTIME;
  do {
    int cus = 0;
    {
      std::lock_guard<std::mutex> lk(g_dn_mu);
      DnDevice& d = g_dn[dev];
      if (d.cus == 0) {
        e = hipDeviceGetAttribute(&d.cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) {
          d.cus = 0;
          dn_set_error(e, "hipDeviceGetAttribute");
          break;
        }
      }
      cus = d.cus;
      if (!d.configured) {
        e = hipFuncSetAttribute((const void*)dense_kernel<256, 256>,
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                DnShape<256, 256>::kLds);
        if (e == hipSuccess)
          e = hipFuncSetAttribute((const void*)dense_kernel<128, 256>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize,
                                  DnShape<128, 256>::kLds);
        if (e == hipSuccess)
          e = hipFuncSetAttribute((const void*)dense_kernel<128, 128>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize,
                                  DnShape<128, 128>::kLds);
        if (e != hipSuccess) {
          dn_set_error(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
          break;
        }
        d.configured = true;
      }
    }
    const DnPlan pl = dn_plan(m, n, k, cus);
    // only a launch with stream-K tiles exchanges anything
    ScratchView view = {nullptr, nullptr};
    if (pl.sk_tiles > 0 &&
        !scratch_acquire(dev, stream,
                         (size_t)pl.sk_tiles * pl.ksplit * pl.tile_rows * pl.tile_cols * 4, &view,
                         g_dn_error, sizeof(g_dn_error)))
      break;
    (void)hipGetLastError();  // an earlier call's error is not this launch's
    DenseArgs a;
    a.A = A;
    a.B = B;
    a.C = C;
    a.M = m;
    a.N = n;
    a.K = k;
    a.tile_rows = pl.tile_rows;
    a.tile_cols = pl.tile_cols;
    a.tiles_m = pl.tiles_m;
    a.tiles_n = pl.tiles_n;
    a.dp_tiles = pl.dp_tiles;
    a.sk_tiles = pl.sk_tiles;
    a.ksplit = pl.ksplit;
    a.locks = view.counters;
    a.scratch = view.partials;
    constexpr int lds_small = DnShape<128, 128>::kLds, lds_half = DnShape<128, 256>::kLds,
                  lds_large = DnShape<256, 256>::kLds;
    if (pl.tile_cols == 128)
      hipLaunchKernelGGL((dense_kernel<128, 128>), dim3(pl.grid), dim3(512), lds_small, stream, a);
    else if (pl.tile_rows == 128)
      hipLaunchKernelGGL((dense_kernel<128, 256>), dim3(pl.grid), dim3(512), lds_half, stream, a);
    else
      hipLaunchKernelGGL((dense_kernel<256, 256>), dim3(pl.grid), dim3(512), lds_large, stream, a);
    e = hipGetLastError();
    if (e != hipSuccess) {
      dn_set_error(e, "kernel launch");
      break;
    }
    rc = STREAMK_OK;
  } while (false);
  if (prev != dev) (void)hipSetDevice(prev);
  return rc;
}

int streamk_amd_check(int m, int n, int k) { return dn_check(m, n, k); }

int streamk_amd_plan(int m, int n, int k, int cus, int* out) {
  const int rc = dn_check(m, n, k);
  if (rc != STREAMK_OK) return rc;
  const DnPlan pl = dn_plan(m, n, k, cus);
  out[0] = pl.tiles_m;
  out[1] = pl.tiles_n;
  out[2] = pl.dp_tiles;
  out[3] = pl.sk_tiles;
  out[4] = pl.ksplit;
  out[5] = pl.grid;
  out[6] = pl.tile_rows;
  out[7] = pl.tile_cols;
  return STREAMK_OK;
}

void streamk_amd_tile_coord(int tile, int tiles_m, int tiles_n, int* out) {
  dn_tile_coord(tile, tiles_m, tiles_n, &out[0], &out[1]);
}

long long streamk_amd_release(int dev) { return (long long)scratch_release(dev); }

const char* streamk_amd_last_error(void) { return g_dn_error; }

}  // extern "C"
