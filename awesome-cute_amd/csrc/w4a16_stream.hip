// Streaming W4A16 kernel for at most 64 activation rows per workgroup (decode
// and small batch): the weight stream is the roofline, so every wave keeps a
// ring of 128-bit weight loads in flight straight into registers and never
// waits on another wave inside the main loop.  A launch covers up to 64 rows,
// or more where its rows are cut into parts that separate workgroups compute
// (see the PARTS instance below).
//
// Work split (StreamPlan in w4a16_common.hpp): a launch is NT*KG granules of
// 128 columns x 64 k in column-tile-major order.  A workgroup (4 waves) owns a
// contiguous run of granules -- one of wpt runs of a single tile, or an equal
// share of the whole sequence -- chosen by its work index, which follows the
// XCD the hardware deals the workgroup to (xcd_work_index).  Its waves take
// the granules round-robin, each accumulating a private 16*MB x 128 fp32
// tile.  At the end of a tile the four waves are summed through LDS, and if
// other workgroups share the tile the partial sums meet in global memory:
// everybody stores fp32 partials, bumps the tile's counter, and the last
// arrival adds all partials in workgroup order and writes C.  Nobody spins.
//
// All global reads are buffer loads issued unconditionally, DEPTH granules
// ahead, so that the hardware's in-order load counter can be waited on
// exactly; a granule that does not exist is requested at an out-of-range
// offset, which returns zeros without touching memory.  Where a run crosses
// tiles the ring keeps running: the first granules of the next tile are in
// flight while the current tile is reduced and written.
#include "w4a16_common.hpp"

namespace w4a16 {

namespace {

constexpr int kOob = (int)0x80000000;  // offset past any buffer (sizes are < 2 GiB)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// s_waitcnt vmcnt(0) with the other counters left alone (gfx9 encoding)
constexpr int kWaitVm0 = 0x0F70;

// Cache policy of the buffer instructions on gfx950: sc1 is bit 4.  A store
// with sc1 is written through to the memory that all XCDs share (device
// scope) and a load with sc1 never returns a line held by this XCD's L2.
constexpr int kAuxDevice = 16;

// 16 bytes per lane of a partial-sum slot, as whole-line buffer accesses
template <int AUX>
__device__ __forceinline__ void store_partial(__amdgpu_buffer_rsrc_t r, int voffset, int soffset,
                                              f4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, v), r, voffset, soffset, AUX);
}
template <int AUX>
__device__ __forceinline__ f4 load_partial(__amdgpu_buffer_rsrc_t r, int voffset, int soffset) {
  return __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(r, voffset, soffset, AUX));
}

}  // namespace

// The activations of a granule travel through registers and are transposed
// into LDS just before use (2 KiB per wave and row block, inside the memory
// that the cross-wave reduction uses later; barriers separate the two): 8
// registers per row block and ring slot.  Only the form whose workgroups cross
// tile boundaries has no registers left for that with several row blocks (it
// keeps two tiles' bookkeeping alive): there the activations are loaded
// straight into an LDS ring instead (buffer_load ... lds, 16 bytes per lane).
// Those loads are slow to issue -- with four row blocks a wave needs 1.7 us to
// request its first two granules, against 1.0 us through registers -- so the
// one-tile form, which every planned launch uses, does without them (M = 48,
// N = K = 4096: 11.5 -> 10.7 us; M = 64: 13.9 -> 13.2; 8192 x 8192: 20.1 -> 19.7).
template <int MB, int DEPTH, bool ONE_TILE>
struct StreamLds {
  static constexpr bool kDmaA = MB >= 2 && !ONE_TILE;
  static constexpr int kReduceBytes = 32768;
  static constexpr int kRingBytesPerWave = kDmaA ? DEPTH * MB * 2048 : 0;
  // A workgroup that stays inside one tile reduces only once, after its last
  // granule, when the staging memory is dead: all row blocks are then reduced
  // in one pass, kReduceBytes each, which also covers the staging (8 KiB x MB)
  static constexpr bool kOnePass = ONE_TILE && MB >= 2;
  static constexpr int kRingBase = kReduceBytes;
  static constexpr int kBytes =
      kOnePass ? MB * kReduceBytes : kReduceBytes + 4 * kRingBytesPerWave;
};

// 16 bytes per lane from a buffer straight into LDS: lane l's bytes land at
// dst + 16*l (dst is wave-uniform).  The instruction's immediate offset is left
// at zero: the hardware would add it to the LDS address as well.  (This and the
// two helpers below are empty in the host pass, which only needs the kernels'
// launch stubs.)
__device__ __forceinline__ void ring_load(__amdgpu_buffer_rsrc_t rsrc, char* dst, int voffset,
                                          int soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef __attribute__((address_space(3))) void* lds_ptr;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr)dst, 16, voffset, soffset, 0, 0);
#endif
}

// The two halves of an MFMA activation operand from the LDS ring (dword kg of
// chunks 0,1 and of chunks 2,3 of a row), and the wait for them.  Written as
// assembly because the compiler must not treat them as LDS reads that depend
// on every ring load in flight.
__device__ __forceinline__ void ring_read(unsigned at, i2& lo, i2& hi) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile(
      "ds_read2st64_b32 %0, %2 offset1:1\n\t"
      "ds_read2st64_b32 %1, %2 offset0:2 offset1:3"
      : "=v"(lo), "=v"(hi)
      : "v"(at)
      : "memory");
#endif
}
// wait until at most PENDING later LDS reads are outstanding
template <int PENDING>
__device__ __forceinline__ void ring_read_wait(i2& lo, i2& hi) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(lo), "+v"(hi) : "n"(PENDING));
#endif
}

// Workgroup barrier for data exchanged through LDS only: waits for this wave's
// LDS accesses, not for its global loads (__syncthreads would drain the whole
// prefetch ring).
__device__ __forceinline__ void lds_barrier() {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#endif
}

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding)
constexpr int wait_vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

// ONE_TILE: the plan's second form (every column tile cut into p.wpt runs), in
// which a workgroup never leaves its tile: no tile bookkeeping in the main
// loop and exactly one finish at the end.  Otherwise the first form (equal
// runs of the tile-major sequence), where a run may cross tile boundaries.
template <int MB, bool GROUP, int DEPTH, bool ONE_TILE, bool PARTS>
__global__ __launch_bounds__(256) void stream_kernel(GemmArgs p) {
  static_assert(!PARTS || (ONE_TILE && MB <= 2), "rows are only cut in the one-tile form, into parts of 16 or 32");
  extern __shared__ __attribute__((aligned(16))) char smem[];  // StreamLds<MB, DEPTH, ONE_TILE>::kBytes
  __shared__ int s_ticket;
  using Lds = StreamLds<MB, DEPTH, ONE_TILE>;
  constexpr bool kDmaA = Lds::kDmaA;

  {
    // Fetch every kernel argument now, in one round trip: left alone, the
    // compiler fetches the pointers only behind the early exit below, a second
    // trip to memory before the first weight load can be issued (0.2 us).
    const void *a_ = p.A, *b_ = p.B, *s_ = p.S;
    void* c_ = p.C;
    int* l_ = p.locks;
    float* sc_ = p.scratch;
    asm volatile("" ::"s"(a_), "s"(b_), "s"(s_), "s"(c_), "s"(l_), "s"(sc_), "s"(p.M), "s"(p.N),
                 "s"(p.K), "s"(p.gpb), "s"(p.wpt), "s"(p.lock_stride), "s"(p.row_parts), "s"(p.part_rows));
  }
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
  const int lane = tid & 63;
  const int kg = lane >> 4;  // k group of the MFMA operand layout
  const int nu = lane & 15;  // column slot (weights) / row (activations)

  StreamPlan plan;
  plan.NT = p.N / kTileN;
  plan.KG = p.K / kGranuleK;
  plan.gpb = p.gpb;
  plan.grid = (int)gridDim.x;
  plan.wpt = ONE_TILE ? p.wpt : 0;
  const int KG = plan.KG;
  const int total = plan.NT * KG;
  const int wid = xcd_work_index((int)blockIdx.x, plan.grid);
  // my granules [u0, u1) of the tile-major sequence; my_tile = tile of u0
  int u0, u1, my_tile;
  // One-tile form with the rows cut into parts: work index w owns run w % wpt
  // of (tile, part) number w / wpt; a part is a problem of its own (its rows of
  // A and C, its ticket, its partial sums) over the same weights.
  int vt = 0;        // (tile, part) number: my_tile * row_parts + part
  int part = 0;
  int row0 = 0;      // first row of my part
  int rows_m = p.M;  // rows of my part
  if constexpr (ONE_TILE) {
    vt = wid / p.wpt;
    const int run = wid - vt * p.wpt;
    my_tile = vt;
    if constexpr (PARTS) {
      my_tile = vt / p.row_parts;
      part = vt - my_tile * p.row_parts;
      row0 = part * p.part_rows;
      rows_m = min(p.part_rows, p.M - row0);
    }
    u0 = my_tile * KG + (run * KG) / p.wpt;
    u1 = my_tile * KG + ((run + 1) * KG) / p.wpt;
    if (my_tile >= plan.NT || u0 >= u1) return;
  } else {
    u0 = wid * plan.gpb;
    if (u0 >= total) return;
    u1 = min(total, u0 + plan.gpb);
    my_tile = u0 / KG;
  }

  const __amdgpu_buffer_rsrc_t rB = make_rsrc(p.B, (unsigned)p.K * (unsigned)(p.N / 2));
  const __amdgpu_buffer_rsrc_t rA = make_rsrc(p.A, (unsigned)p.M * (unsigned)p.K * 2u);
  const __amdgpu_buffer_rsrc_t rS =
      make_rsrc(p.S, (unsigned)(GROUP ? p.K / 128 : 1) * (unsigned)p.N * 2u);
  const int b_row = p.N * 8;  // bytes per row of B (16 k-values of every column)

  // per-lane parts of the addresses; the rest is wave-uniform
  const int b_lane = 64 * nu + 16 * kg;
  const int s_lane = 16 * nu;
  // Activation staging.  Register path: lane (row = lane/4, ax = lane%4)
  // fetches 16-byte chunks ax and ax+4 of the 128-byte k run of its row and
  // writes their dwords to [step][kg'][row][ax], so that MFMA lane (kg, row nu)
  // reads its operand with one 16-byte access at a_rd.
  // LDS-ring path: lane (kg, nu) fetches chunk kg of the 64-byte k run of row
  // nu; the hardware puts lane l's 16 bytes at 16*l, i.e. [chunk][row].  MFMA
  // lane (kg, nu) then needs dword kg of the four chunks of its row:
  // 256*c + 16*nu + 4*kg, two ds_read2st64_b32 and no bank conflict.
  const int ax = kDmaA ? kg : (lane & 3);
  int a_lane[MB];
#pragma unroll
  for (int i = 0; i < MB; i++) {
    int r = 16 * i + (kDmaA ? nu : (lane >> 2));
    r = r < rows_m ? r : rows_m - 1;  // rows past the end are never written back
    a_lane[i] = (row0 + r) * p.K * 2 + 16 * ax;
  }
  char* lds_a = kDmaA ? smem + Lds::kRingBase + wave * Lds::kRingBytesPerWave
                      : smem + wave * (MB * 2048);
  const int a_wr = ((lane >> 2) * 4 + ax) * 4;
  const int a_rd = kDmaA ? 16 * nu + 4 * kg : (kg * 16 + nu) * 16;
  // (The ring starts with whatever LDS held: a slot is only ever read after a
  // granule that exists was loaded into it -- the arithmetic on slots past the
  // end of the run is skipped below.)

  const DequantConsts dc;

  i4 bq[DEPTH][4];
  i4 sq[DEPTH];
  i4 aq[kDmaA ? 1 : DEPTH][MB][2];  // unused on the LDS-ring path

  // request granule kq of tile t into ring slot `slot`; straight-line code, so
  // that every turn of the ring issues exactly the same loads in the same order
  auto issue = [&](int slot, int t, int kq, bool valid) {
    __builtin_amdgcn_sched_barrier(0);
    const int inv = valid ? 0 : kOob;
    const int vb = b_lane | inv;
    const int sb = (4 * kq) * b_row + 1024 * t;
#pragma unroll
    for (int r = 0; r < 4; r++)
      bq[slot][r] = __builtin_amdgcn_raw_buffer_load_b128(rB, vb, sb + r * b_row, 2);
    if (GROUP)
      sq[slot] = __builtin_amdgcn_raw_buffer_load_b128(rS, s_lane | inv,
                                                       ((kq >> 1) * p.N + kTileN * t) * 2, 0);
#pragma unroll
    for (int i = 0; i < MB; i++) {
      if constexpr (kDmaA) {
        char* dst = lds_a + (slot * MB + i) * 2048;
        ring_load(rA, dst, a_lane[i] | inv, 128 * kq);
        ring_load(rA, dst + 1024, a_lane[i] | inv, 128 * kq + 64);
      } else {
        aq[slot][i][0] = __builtin_amdgcn_raw_buffer_load_b128(rA, a_lane[i] | inv, 128 * kq, 0);
        aq[slot][i][1] =
            __builtin_amdgcn_raw_buffer_load_b128(rA, a_lane[i] | inv, 128 * kq + 64, 0);
      }
    }
    // keep the groups in issue order: the in-order load counter is only exact
    // if a slot's loads are never moved behind those of a later slot
    __builtin_amdgcn_sched_barrier(0);
  };

  f4 acc[MB][8];
  auto clear_acc = [&]() {
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
      for (int j = 0; j < 8; j++) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};
  };

  // loads of one ring slot: 4 weight rows, the scales, 2 per row block
  constexpr int kLoadsPerSlot = 4 + (GROUP ? 1 : 0) + 2 * MB;

  auto compute = [&](int slot) {
    // LDS-ring path: the operands of both k steps are fetched up front; the
    // wait for the second step's comes after the first step's MFMAs
    i2 lo[2][MB], hi[2][MB];
    if constexpr (kDmaA) {
      // The ring loads of this slot are DEPTH-1 slots old: everything but the
      // loads issued since has landed.  (The compiler cannot see that LDS is
      // written by those loads, so the wait and the LDS reads are explicit.)
      __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm((DEPTH - 1) * kLoadsPerSlot));
#pragma unroll
      for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int i = 0; i < MB; i++) {
          const unsigned at =
              (unsigned)(size_t)(lds_a + (slot * MB + i) * 2048 + h * 1024 + a_rd);
          ring_read(at, lo[h][i], hi[h][i]);
        }
      }
      // LDS reads complete in order: all but the 2*MB reads of the second step
#pragma unroll
      for (int i = 0; i < MB; i++) ring_read_wait<2 * MB>(lo[0][i], hi[0][i]);
    } else {
      // activations: registers -> LDS in MFMA k-slot order
#pragma unroll
      for (int i = 0; i < MB; i++)
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
          for (int g = 0; g < 4; g++)
            *(int*)(lds_a + i * 2048 + h * 1024 + g * 256 + a_wr) = aq[slot][i][h][g];
    }
#pragma unroll
    for (int h = 0; h < 2; h++) {
      h8 af[MB];
      if constexpr (kDmaA) {
        if (h == 1) {
          __builtin_amdgcn_sched_barrier(0);  // keep the wait behind the first step's MFMAs
#pragma unroll
          for (int i = 0; i < MB; i++) ring_read_wait<0>(lo[1][i], hi[1][i]);
        }
#pragma unroll
        for (int i = 0; i < MB; i++) {
          i4 v = {lo[h][i][0], lo[h][i][1], hi[h][i][0], hi[h][i][1]};
          af[i] = __builtin_bit_cast(h8, v);
        }
      } else {
#pragma unroll
        for (int i = 0; i < MB; i++)
          af[i] = __builtin_bit_cast(h8, *(const i4*)(lds_a + i * 2048 + h * 1024 + a_rd));
      }
#pragma unroll
      for (int j = 0; j < 4; j++) {
        h2 s2 = GROUP ? as_h2(sq[slot][j]) : (h2){(half_t)1.f, (half_t)1.f};
        h2 l0, h0, l1, h1, m0, n0, m1, n1;
        dequant_word<GROUP>(bq[slot][2 * h][j], s2, dc, l0, h0, l1, h1);
        dequant_word<GROUP>(bq[slot][2 * h + 1][j], s2, dc, m0, n0, m1, n1);
        h8 w0 = make_h8(l0, h0, m0, n0);
        h8 w1 = make_h8(l1, h1, m1, n1);
#pragma unroll
        for (int i = 0; i < MB; i++) {
          acc[i][2 * j] =
              __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, af[i], acc[i][2 * j], 0, 0, 0);
          acc[i][2 * j + 1] =
              __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, af[i], acc[i][2 * j + 1], 0, 0, 0);
        }
      }
    }
  };

  // Finish column tile t: sum the four waves, meet the other workgroups that
  // share the tile, write C.  Every wave calls this exactly once per tile of
  // the workgroup, in tile order.
  auto finish = [&](int t) {
    // ---- sum the four waves; wave w ends up owning the 16-column groups
    // (j = w, h = 0/1) of every row block
    f4 res[MB][2];
    lds_barrier();
    if constexpr (Lds::kOnePass) {
      // room for all row blocks at once: two barriers instead of two per block
#pragma unroll
      for (int i = 0; i < MB; i++) {
        f4* red = (f4*)smem + i * (Lds::kReduceBytes / 16);
#pragma unroll
        for (int j = 0; j < 8; j++) red[(wave * 8 + j) * 64 + lane] = acc[i][j];
      }
      lds_barrier();
#pragma unroll
      for (int i = 0; i < MB; i++) {
        const f4* red = (const f4*)smem + i * (Lds::kReduceBytes / 16);
#pragma unroll
        for (int h = 0; h < 2; h++) {
          f4 v = red[(0 * 8 + 2 * wave + h) * 64 + lane];
#pragma unroll
          for (int w = 1; w < 4; w++) v += red[(w * 8 + 2 * wave + h) * 64 + lane];
          res[i][h] = v;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < MB; i++) {
        f4* red = (f4*)smem;
#pragma unroll
        for (int j = 0; j < 8; j++) red[(wave * 8 + j) * 64 + lane] = acc[i][j];
        lds_barrier();
#pragma unroll
        for (int h = 0; h < 2; h++) {
          f4 v = red[(0 * 8 + 2 * wave + h) * 64 + lane];
#pragma unroll
          for (int w = 1; w < 4; w++) v += red[(w * 8 + 2 * wave + h) * 64 + lane];
          res[i][h] = v;
        }
        lds_barrier();
      }
    }

    // ---- meet the other workgroups of this tile, if any.  Partial sums are
    // written with device-scope (write-through) stores, whole 1 KiB lines per
    // wave instruction, so no cache write-back is needed: a wave waits until
    // its own stores are acknowledged, the barrier collects the four waves, and
    // only then does thread 0 take the tile's ticket.  Whoever draws the last
    // ticket knows every other partial has already landed in memory and reads
    // them with device-scope loads.  (Keeping a second, write-back copy in the
    // XCD's L2 for the reader was measured and dropped: 0.15 us slower.)
    const int bf = ONE_TILE ? vt * p.wpt : tile_first_block(plan, t);
    const int bl = ONE_TILE ? bf + p.wpt - 1 : tile_last_block(plan, t);
    bool writer = true;
    if (bl > bf) {
      constexpr int part_bytes = MB * 4 * 2 * 64 * 16;  // a slot: MB*4*2*64 f4, written through
      const __amdgpu_buffer_rsrc_t rP = make_rsrc(p.scratch, 0x7fffffffu);
      // slot of work index b for this tile
      auto slot_of = [&](int b) { return ONE_TILE ? 2 * b : partial_slot(plan, b, t); };
      const int mine = slot_of(wid) * part_bytes;
#pragma unroll
      for (int i = 0; i < MB; i++)
        if (16 * i + nu < rows_m) {
#pragma unroll
          for (int h = 0; h < 2; h++) {
            const int at = (((i * 4 + wave) * 2 + h) * 64 + lane) * 16;
            store_partial<kAuxDevice>(rP, at, mine, res[i][h]);
          }
        }
      __builtin_amdgcn_s_waitcnt(kWaitVm0);  // my stores have been acknowledged
      __syncthreads();
      if (tid == 0)
        s_ticket = __hip_atomic_fetch_add(&p.locks[t * p.lock_stride + part], 1, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      writer = (s_ticket == bl - bf);
      if (writer) {
        // Add the partials in workgroup order (deterministic).  They are fetched
        // eight workgroups at a time, and the next row block's are requested
        // before this row block's are added, so that the loads overlap.  Rows
        // past M are requested out of range (zeros, no traffic).
        f4 sum[MB][2];
        for (int b0 = bf; b0 <= bl; b0 += 8) {
          f4 v[2][8][2];
          auto fetch = [&](int i, f4 (&dst)[8][2]) {
            const int at = ((((i * 4 + wave) * 2) * 64 + lane) * 16) | (16 * i + nu < rows_m ? 0 : kOob);
#pragma unroll
            for (int u = 0; u < 8; u++) {
              const int b = b0 + u;
              if (b <= bl && b != wid) {
                const int theirs = slot_of(b) * part_bytes;
                dst[u][0] = load_partial<kAuxDevice>(rP, at, theirs);
                dst[u][1] = load_partial<kAuxDevice>(rP, at + 1024, theirs);
              } else {
                dst[u][0] = res[i][0];
                dst[u][1] = res[i][1];
              }
            }
          };
          fetch(0, v[0]);
#pragma unroll
          for (int i = 0; i < MB; i++) {
            if (i + 1 < MB) fetch(i + 1, v[(i + 1) & 1]);
#pragma unroll
            for (int u = 0; u < 8; u++) {
              if (b0 + u <= bl) {
                sum[i][0] = (b0 + u == bf) ? v[i & 1][u][0] : sum[i][0] + v[i & 1][u][0];
                sum[i][1] = (b0 + u == bf) ? v[i & 1][u][1] : sum[i][1] + v[i & 1][u][1];
              }
            }
          }
        }
#pragma unroll
        for (int i = 0; i < MB; i++) {
          res[i][0] = sum[i][0];
          res[i][1] = sum[i][1];
        }
        if (tid == 0)  // counters are handed back zeroed
          __hip_atomic_store(&p.locks[t * p.lock_stride + part], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __syncthreads();  // s_ticket is reused by the next tile
    }

    // ---- write C (fp16); per-channel mode scales the rounded result
    if (writer) {
      half_t* C = (half_t*)p.C;
      const int q = lane >> 4;
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int n0 = kTileN * t + 64 * (q >> 1) + 4 * (q & 1) + 16 * wave + 8 * h;
        h4 sc = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
        if (!GROUP) {
          const half_t* S = (const half_t*)p.S;
#pragma unroll
          for (int r = 0; r < 4; r++) sc[r] = S[scale_index_single(n0 + r)];
        }
#pragma unroll
        for (int i = 0; i < MB; i++) {
          const int m = 16 * i + nu;
          if (m < rows_m) {
            h4 o = {(half_t)res[i][h][0], (half_t)res[i][h][1], (half_t)res[i][h][2],
                    (half_t)res[i][h][3]};
            if (!GROUP) o *= sc;
            *(h4*)(C + (size_t)(row0 + m) * p.N + n0) = o;
          }
        }
      }
    }
  };

  // My granules are u0 + wave, u0 + wave + 4, ... < u1.
  const int n_mine = (u1 - u0 > wave) ? ((u1 - u0 - wave + 3) >> 2) : 0;
  clear_acc();

  if constexpr (ONE_TILE) {
    // one tile: the k position just advances by four granules a turn
    int ikq = u0 - my_tile * KG + wave;  // issue position
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      issue(d, my_tile, ikq, d < n_mine);
      ikq += 4;
    }
    if constexpr (DEPTH == 2 && !kDmaA) {
      // At most two granules per wave (the host picks this instance for no
      // other run) and both are already requested: a rolled loop over one copy
      // of the compute code; the second granule moves into the first's
      // registers in between.
#pragma unroll 1
      for (int i = 0; i < n_mine; i++) {
        compute(0);
#pragma unroll
        for (int r = 0; r < 4; r++) bq[0][r] = bq[1][r];
        sq[0] = sq[1];
#pragma unroll
        for (int m = 0; m < MB; m++) {
          aq[0][m][0] = aq[1][m][0];
          aq[0][m][1] = aq[1][m][1];
        }
      }
    } else {
      for (int base = 0; base < n_mine; base += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
          // the slots past the end hold zeros: skip their arithmetic (the loads
          // are still issued, so the load counter stays exact)
          if (base + d < n_mine) compute(d);
          issue(d, my_tile, ikq, base + d + DEPTH < n_mine);
          ikq += 4;
        }
      }
    }
    finish(my_tile);
  } else {
    // The run is walked in one flat sequence across column tiles; (t, kq) are
    // kept incrementally for the compute position and for the issue position
    // DEPTH granules ahead.
    const int t_last = (u1 - 1) / KG;
    int it = my_tile, ikq = u0 - my_tile * KG + wave;  // issue position
    while (ikq >= KG) {
      ikq -= KG;
      ++it;
    }
    int ct = it, ckq = ikq;  // compute position
    int cur_tile = my_tile;  // tile whose sums are in acc

#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      issue(d, it, ikq, d < n_mine);
      ikq += 4;
      while (ikq >= KG) {
        ikq -= KG;
        ++it;
      }
    }

    for (int base = 0; base < n_mine; base += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; d++) {
        const int i = base + d;
        if (i < n_mine) {
          // entering a new tile: hand over the tiles behind me first
          while (cur_tile < ct) {
            finish(cur_tile);
            ++cur_tile;
            clear_acc();
          }
        }
        if (i < n_mine) compute(d);  // the slots past the end hold zeros
        ckq += 4;
        while (ckq >= KG) {
          ckq -= KG;
          ++ct;
        }
        issue(d, it, ikq, i + DEPTH < n_mine);
        ikq += 4;
        while (ikq >= KG) {
          ikq -= KG;
          ++it;
        }
      }
    }
    while (cur_tile <= t_last) {
      finish(cur_tile);
      ++cur_tile;
      clear_acc();
    }
  }
}

// Ring depth of the deep variant.  Three granules in flight per wave measured
// faster than four for every row-block count (M=16: N=11008 10.3 -> 9.9 us,
// K=11008 10.4 -> 9.6; 64 rows at K=11008 21.2 -> 18.4), and eight slower
// still: the more requests a CU has in flight, the slower the stream.  With
// two row blocks on the LDS ring two are better again (M=32, N=11008:
// 12.7 -> 12.4 us), with three and four they are 2-5 % worse.  In the one-tile
// form the deep variant is never two deep: there the two-slot instance is the
// rolled loop for waves that see at most two granules (see the kernel), which
// launch_form below only picks for such runs.
template <int MB, bool ONE_TILE>
constexpr int deep_ring() {
  return MB == 2 && !ONE_TILE ? 2 : 3;
}

template <int MB, bool GROUP, int DEPTH, bool ONE_TILE>
static int configure_variant() {
  constexpr int lds = StreamLds<MB, DEPTH, ONE_TILE>::kBytes;
  if (lds <= 65536) return 0;  // within the default limit of dynamic LDS
  if (hipFuncSetAttribute((const void*)stream_kernel<MB, GROUP, DEPTH, ONE_TILE, false>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
    return 3;
  if constexpr (ONE_TILE && MB <= 2) {
    if (hipFuncSetAttribute((const void*)stream_kernel<MB, GROUP, DEPTH, ONE_TILE, true>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return 3;
  }
  return 0;
}
template <int MB, bool ONE_TILE>
static int configure_form() {
  return configure_variant<MB, false, 2, ONE_TILE>() | configure_variant<MB, true, 2, ONE_TILE>() |
         configure_variant<MB, false, deep_ring<MB, ONE_TILE>(), ONE_TILE>() |
         configure_variant<MB, true, deep_ring<MB, ONE_TILE>(), ONE_TILE>();
}
template <int MB>
static int configure_row_blocks() {
  return configure_form<MB, false>() | configure_form<MB, true>();
}

int configure_stream_kernels() {
  return (configure_row_blocks<1>() | configure_row_blocks<2>() | configure_row_blocks<3>() |
          configure_row_blocks<4>())
             ? 3
             : 0;
}

template <int MB, bool GROUP, int DEPTH, bool ONE_TILE>
static int launch_variant(const GemmArgs& a, int grid, hipStream_t stream) {
  constexpr int lds = StreamLds<MB, DEPTH, ONE_TILE>::kBytes;
  // (the instance with the rows cut in two is a kernel of its own, so that
  // launches that do not cut them carry none of its bookkeeping)
  if constexpr (ONE_TILE && MB <= 2) {
    if (a.row_parts > 1) {
      hipLaunchKernelGGL((stream_kernel<MB, GROUP, DEPTH, ONE_TILE, true>), dim3(grid), dim3(256),
                         lds, stream, a);
      return launch_status();
    }
  }
  hipLaunchKernelGGL((stream_kernel<MB, GROUP, DEPTH, ONE_TILE, false>), dim3(grid), dim3(256),
                     lds, stream, a);
  return launch_status();
}

template <int MB, bool GROUP, bool ONE_TILE>
static int launch_form(const GemmArgs& a, int grid, hipStream_t stream) {
  // ring depth: shallow when a wave only ever sees a couple of granules
  const int per_wave = (a.gpb + 3) / 4;
  if (per_wave <= 2) return launch_variant<MB, GROUP, 2, ONE_TILE>(a, grid, stream);
  return launch_variant<MB, GROUP, deep_ring<MB, ONE_TILE>(), ONE_TILE>(a, grid, stream);
}

template <int MB, bool GROUP>
static int launch_one(const GemmArgs& a, int grid, hipStream_t stream) {
  return a.wpt > 0 ? launch_form<MB, GROUP, true>(a, grid, stream)
                   : launch_form<MB, GROUP, false>(a, grid, stream);
}

int launch_stream(const GemmArgs& a, bool group, int grid, hipStream_t stream) {
  // row blocks per workgroup: of all rows, or of a part
  const int mb = a.wpt > 0 && a.row_parts > 1 ? a.part_rows / 16 : ceil_div(a.M, 16);
  switch (mb * 2 + (group ? 1 : 0)) {
    case 2: return launch_one<1, false>(a, grid, stream);
    case 3: return launch_one<1, true>(a, grid, stream);
    case 4: return launch_one<2, false>(a, grid, stream);
    case 5: return launch_one<2, true>(a, grid, stream);
    case 6: return launch_one<3, false>(a, grid, stream);
    case 7: return launch_one<3, true>(a, grid, stream);
    case 8: return launch_one<4, false>(a, grid, stream);
    case 9: return launch_one<4, true>(a, grid, stream);
  }
  return 2;
}

}  // namespace w4a16
