// Streaming W4A16 kernel for at most 64 activation rows (decode and small
// batch): the weight stream is the roofline, so every wave keeps a deep queue
// of 128-bit weight loads in flight straight into registers and never waits
// on another wave inside the main loop.
//
// Work split (see make_stream_plan): a launch is NT*KG granules of
// 128 columns x 64 k.  A workgroup (4 waves) owns a contiguous run of
// granules; inside a column tile its waves take granules round-robin, each
// accumulating a private 16*MB x 128 fp32 tile.  At the end of the tile the
// four waves are summed through LDS, and if other workgroups share the tile
// the partial sums meet in global memory: everybody stores fp32 partials,
// bumps the tile's counter, and the last arrival adds all partials in
// workgroup order and writes C.  Nobody ever spins.
#include "w4a16_common.hpp"

namespace w4a16 {

template <int MB, bool GROUP, int DEPTH>
__global__ __launch_bounds__(256) void stream_kernel(GemmArgs p) {
  // A staging (4 waves x MB x 2 KiB) and the cross-wave reduction (32 KiB)
  // use the same LDS; barriers separate the two uses.
  __shared__ __attribute__((aligned(16))) char smem[32768];
  __shared__ int s_ticket;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int kg = lane >> 4;  // k group of the MFMA operand layout
  const int nu = lane & 15;  // column slot (weights) / row (activations)

  StreamPlan plan;
  plan.NT = p.N / kTileN;
  plan.KG = p.K / kGranuleK;
  plan.gpb = p.gpb;
  plan.grid = (int)gridDim.x;
  const int total = plan.NT * plan.KG;
  const int u0 = (int)blockIdx.x * plan.gpb;
  if (u0 >= total) return;
  const int u1 = min(total, u0 + plan.gpb);

  const i4* __restrict__ B4 = (const i4*)p.B;
  const i4* __restrict__ A4 = (const i4*)p.A;
  const i4* __restrict__ S4 = (const i4*)p.S;
  const size_t b_row = (size_t)(p.N / 2);  // int4 per row of B
  const size_t a_row = (size_t)(p.K / 8);  // int4 per row of A

  // activation staging: lane (row = lane/4, ax = lane%4) fetches chunks ax and
  // ax+4 (16 bytes each) of the 128-byte k run of its row
  const int ax = lane & 3;
  size_t a_off[MB];
#pragma unroll
  for (int i = 0; i < MB; i++) {
    int r = 16 * i + (lane >> 2);
    r = r < p.M ? r : p.M - 1;  // rows past M are never written back
    a_off[i] = (size_t)r * a_row + ax;
  }
  char* lds_a = smem + wave * (MB * 2048);
  // write position of dword kg' of a chunk: [step][kg'][row][ax]
  const int a_wr = ((lane >> 2) * 4 + ax) * 4;
  // read position of the operand of MFMA lane (kg, row nu)
  const int a_rd = (kg * 16 + nu) * 16;

  const DequantConsts dc;

  for (int t = u0 / plan.KG; t * plan.KG < u1; ++t) {
    const int seg_a = max(u0, t * plan.KG) - t * plan.KG;
    const int seg_e = min(u1, (t + 1) * plan.KG) - t * plan.KG;
    const int n_my = (seg_e - seg_a > wave) ? ((seg_e - seg_a - wave + 3) >> 2) : 0;
    const int kq0 = seg_a + wave;  // my granules: kq0, kq0+4, ...

    const i4* bptr = B4 + (size_t)64 * t + 4 * nu + kg;
    const i4* sptr = S4 + (size_t)16 * t + nu;

    f4 acc[MB][8];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
      for (int j = 0; j < 8; j++) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};

    i4 bq[DEPTH][4];
    i4 sq[DEPTH];
    i4 aq[DEPTH][MB][2];

    auto issue = [&](int slot, int kq) {
#pragma unroll
      for (int r = 0; r < 4; r++)
        bq[slot][r] = __builtin_nontemporal_load(bptr + (size_t)(4 * kq + r) * b_row);
      if (GROUP) sq[slot] = sptr[(size_t)(kq >> 1) * (p.N / 8)];
#pragma unroll
      for (int i = 0; i < MB; i++) {
        aq[slot][i][0] = A4[a_off[i] + 8 * kq];
        aq[slot][i][1] = A4[a_off[i] + 8 * kq + 4];
      }
    };

    auto compute = [&](int slot) {
      // activations: registers -> LDS in MFMA k-slot order
#pragma unroll
      for (int i = 0; i < MB; i++)
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
          for (int g = 0; g < 4; g++)
            *(int*)(lds_a + i * 2048 + h * 1024 + g * 256 + a_wr) = aq[slot][i][h][g];
#pragma unroll
      for (int h = 0; h < 2; h++) {
        h8 af[MB];
#pragma unroll
        for (int i = 0; i < MB; i++)
          af[i] = __builtin_bit_cast(h8, *(const i4*)(lds_a + i * 2048 + h * 1024 + a_rd));
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

#pragma unroll
    for (int d = 0; d < DEPTH; d++)
      if (d < n_my) issue(d, kq0 + 4 * d);
    for (int base = 0; base < n_my; base += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; d++) {
        if (base + d < n_my) {
          compute(d);
          if (base + d + DEPTH < n_my) issue(d, kq0 + 4 * (base + d + DEPTH));
        }
      }
    }

    // ---- sum the four waves; wave w ends up owning the 16-column groups
    // (j = w, h = 0/1) of every row block
    f4 res[MB][2];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MB; i++) {
      f4* red = (f4*)smem;
#pragma unroll
      for (int j = 0; j < 8; j++) red[(wave * 8 + j) * 64 + lane] = acc[i][j];
      __syncthreads();
#pragma unroll
      for (int h = 0; h < 2; h++) {
        f4 v = red[(0 * 8 + 2 * wave + h) * 64 + lane];
#pragma unroll
        for (int w = 1; w < 4; w++) v += red[(w * 8 + 2 * wave + h) * 64 + lane];
        res[i][h] = v;
      }
      __syncthreads();
    }

    // ---- meet the other workgroups of this tile, if any
    const int bf = tile_first_block(plan, t);
    const int bl = tile_last_block(plan, t);
    bool writer = true;
    if (bl > bf) {
      const size_t slot_f4 = (size_t)MB * 4 * 2 * 64;
      f4* mine = (f4*)p.scratch + (size_t)partial_slot(plan, (int)blockIdx.x, t) * slot_f4;
#pragma unroll
      for (int i = 0; i < MB; i++)
        if (16 * i + nu < p.M) {
#pragma unroll
          for (int h = 0; h < 2; h++) mine[((i * 4 + wave) * 2 + h) * 64 + lane] = res[i][h];
        }
      __threadfence();  // partials visible device-wide before the ticket
      __syncthreads();
      if (tid == 0)
        s_ticket = __hip_atomic_fetch_add(&p.locks[t], 1, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      writer = (s_ticket == bl - bf);
      if (writer) {
        __threadfence();  // see everybody else's partials
#pragma unroll
        for (int i = 0; i < MB; i++) {
          if (16 * i + nu < p.M) {
            f4 sum[2];
            for (int b = bf; b <= bl; b++) {
              f4 v[2];
              if (b == (int)blockIdx.x) {
                v[0] = res[i][0];
                v[1] = res[i][1];
              } else {
                const f4* theirs =
                    (const f4*)p.scratch + (size_t)partial_slot(plan, b, t) * slot_f4;
                v[0] = theirs[((i * 4 + wave) * 2 + 0) * 64 + lane];
                v[1] = theirs[((i * 4 + wave) * 2 + 1) * 64 + lane];
              }
              sum[0] = (b == bf) ? v[0] : sum[0] + v[0];
              sum[1] = (b == bf) ? v[1] : sum[1] + v[1];
            }
            res[i][0] = sum[0];
            res[i][1] = sum[1];
          }
        }
        if (tid == 0) p.locks[t] = 0;  // counters are handed back zeroed
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
          if (m < p.M) {
            h4 o = {(half_t)res[i][h][0], (half_t)res[i][h][1], (half_t)res[i][h][2],
                    (half_t)res[i][h][3]};
            if (!GROUP) o *= sc;
            *(h4*)(C + (size_t)m * p.N + n0) = o;
          }
        }
      }
    }
  }
}

template <int MB, bool GROUP>
static int launch_one(const GemmArgs& a, int grid, hipStream_t stream) {
  constexpr int DEPTH = MB <= 2 ? 4 : 3;
  hipLaunchKernelGGL((stream_kernel<MB, GROUP, DEPTH>), dim3(grid), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

int launch_stream(const GemmArgs& a, bool group, int grid, hipStream_t stream) {
  const int mb = ceil_div(a.M, 16);
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
