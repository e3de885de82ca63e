// Prefill W4A16 kernel (more than 64 activation rows): MFMA-bound, so the
// design minimises everything that competes with the matrix pipe.
//
// One workgroup (4 waves, one per SIMD) owns a 128-row x 256-column tile of C
// over the whole k range.  Wave w keeps a 128 x 64 fp32 accumulator (128
// registers): columns 16j+8h+c of the two 64-column blocks 2p, 2p+1 with
// p = w/2 and j in {2(w%2), 2(w%2)+1}.
//   - Weights never touch LDS: each lane reads the 8 bytes of its Marlin
//     16-byte piece that belong to its two 16-column groups straight from
//     global memory (L2-resident after the first row tile), unpacks them in
//     registers and feeds them to the MFMA as the first operand.  One unpack
//     serves eight MFMAs (the eight 16-row blocks).
//   - Activations are shared by the four waves: the workgroup stages a
//     128 x 64 fp16 slab per k stage through LDS, double buffered, stored in
//     the k-slot order the weight layout dictates so that an operand is one
//     conflict-free ds_read_b128.
// Per 32-deep k step a wave issues 32 MFMAs, 8 LDS reads and the unpack of 4
// weight words (about 52 VALU instructions).
#include "w4a16_common.hpp"

namespace w4a16 {

namespace {

constexpr int kPfTileM = 128;
constexpr int kPfTileN = 256;
constexpr int kPfStageK = 64;
constexpr int kPfStepBytes = 4 * 128 * 16 + 128;       // one 32-deep k step of the slab (+pad)
constexpr int kPfStageBytes = 2 * kPfStepBytes;        // two steps per stage
constexpr int kOobPf = (int)0x80000000;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t pf_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

}  // namespace

template <bool GROUP>
__global__ __launch_bounds__(256) void prefill_kernel(GemmArgs p, int tiles_m, int tiles_n) {
  __shared__ __attribute__((aligned(16))) char smem[2 * kPfStageBytes];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int kg = lane >> 4;
  const int nu = lane & 15;
  const int pr = wave >> 1;  // pair of 64-column blocks
  const int jp = wave & 1;   // pair of 16-column groups inside each block

  // Workgroup ids are dealt round-robin to the 8 XCDs; give every XCD a
  // contiguous run of tiles (column tile fastest) so that the workgroups
  // sharing an L2 read the same rows of A and neighbouring columns of B.
  const int total = tiles_m * tiles_n;
  int tile = (int)blockIdx.x;
  if ((total & 7) == 0) tile = (tile & 7) * (total >> 3) + (tile >> 3);
  const int tm = tile / tiles_n;
  const int tn = tile - tm * tiles_n;
  const int m0 = tm * kPfTileM;
  const int rows = min(kPfTileM, p.M - m0);

  const __amdgpu_buffer_rsrc_t rB = pf_rsrc(p.B, (unsigned)p.K * (unsigned)(p.N / 2));
  const __amdgpu_buffer_rsrc_t rS =
      pf_rsrc(p.S, (unsigned)(GROUP ? p.K / 128 : 1) * (unsigned)p.N * 2u);
  const __amdgpu_buffer_rsrc_t rA =
      pf_rsrc((const char*)p.A + (size_t)m0 * p.K * 2, (unsigned)rows * (unsigned)p.K * 2u);
  const int b_row = p.N * 8;

  const int b_lane = 1024 * (2 * tn + pr) + 64 * nu + 16 * kg + 8 * jp;
  const int s_lane = (256 * tn + 128 * pr + 8 * nu) * 2 + 8 * jp;

  // slab staging: thread (row = tid/8 + 32 i, chunk x = tid%8) moves 16 bytes;
  // rows past the end of A read as zeros (out-of-range buffer offset)
  const int ax = tid & 7;
  int a_lane[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int r = (tid >> 3) + 32 * i;
    a_lane[i] = r < rows ? r * p.K * 2 + 16 * ax : kOobPf;
  }
  // LDS slab: [step][k group][row][slot] dwords; chunk x -> step x/4, slot x%4
  const int a_wr = (ax >> 2) * kPfStepBytes + (tid >> 3) * 16 + (ax & 3) * 4;
  const int a_rd = kg * 2048 + nu * 16;

  const DequantConsts dc;
  const int stages = p.K / kPfStageK;

  i4 areg[4];   // slab of the stage after next, in flight
  i2 breg[2][4];  // weight words of this stage and the next: 4 rows x 8 bytes
  i2 sreg[2];

  auto issue_b = [&](int slot, int s) {
    const int inv = s < stages ? 0 : kOobPf;
#pragma unroll
    for (int r = 0; r < 4; r++)
      breg[slot][r] =
          __builtin_amdgcn_raw_buffer_load_b64(rB, b_lane | inv, (4 * s + r) * b_row, 0);
    if (GROUP)
      sreg[slot] = __builtin_amdgcn_raw_buffer_load_b64(rS, s_lane | inv, (s >> 1) * p.N * 2, 0);
  };
  auto issue_a = [&](int s) {
    const int inv = s < stages ? 0 : kOobPf;
#pragma unroll
    for (int i = 0; i < 4; i++)
      areg[i] = __builtin_amdgcn_raw_buffer_load_b128(rA, a_lane[i] | inv, s * 128, 0);
  };
  auto store_a = [&](int buf) {
    char* base = smem + buf * kPfStageBytes + a_wr;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int g = 0; g < 4; g++) *(int*)(base + g * 2048 + i * 32 * 16) = areg[i][g];
  };

  f4 acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};

  auto step = [&](int buf, int slot, int h) {
    h8 w[4];
#pragma unroll
    for (int j2 = 0; j2 < 2; j2++) {
      h2 s2 = GROUP ? as_h2(sreg[slot][j2]) : (h2){(half_t)1.f, (half_t)1.f};
      h2 l0, h0, l1, h1, m0_, n0_, m1_, n1_;
      dequant_word<GROUP>(breg[slot][2 * h][j2], s2, dc, l0, h0, l1, h1);
      dequant_word<GROUP>(breg[slot][2 * h + 1][j2], s2, dc, m0_, n0_, m1_, n1_);
      w[2 * j2] = make_h8(l0, h0, m0_, n0_);
      w[2 * j2 + 1] = make_h8(l1, h1, m1_, n1_);
    }
    const char* base = smem + buf * kPfStageBytes + h * kPfStepBytes + a_rd;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      h8 af = __builtin_bit_cast(h8, *(const i4*)(base + i * 256));
#pragma unroll
      for (int j = 0; j < 4; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[j], af, acc[i][j], 0, 0, 0);
    }
  };

  // prologue: slab 0 -> LDS, slab 1 and the weights of stages 0, 1 in flight
  issue_a(0);
  issue_b(0, 0);
  store_a(0);
  issue_a(1);
  issue_b(1, 1);
  __syncthreads();

  for (int s = 0; s < stages; s += 2) {
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int cs = s + u;  // stage being computed, slab in buffer u
      step(u, u, 0);
      store_a(u ^ 1);   // slab cs+1 (nobody reads that buffer during stage cs)
      issue_a(cs + 2);
      step(u, u, 1);
      issue_b(u, cs + 2);
      __syncthreads();
    }
  }

  // epilogue: lane holds row m = 16 i + nu and, per (j2, h), four consecutive columns
  half_t* C = (half_t*)p.C;
  const int q = lane >> 4;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int n0 = kPfTileN * tn + 128 * pr + 64 * (q >> 1) + 16 * (2 * jp + (j >> 1)) +
                   8 * (j & 1) + 4 * (q & 1);
    h4 sc = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
    if (!GROUP) {
      const half_t* S = (const half_t*)p.S;
#pragma unroll
      for (int r = 0; r < 4; r++) sc[r] = S[scale_index_single(n0 + r)];
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int m = 16 * i + nu;
      if (m < rows) {
        h4 o = {(half_t)acc[i][j][0], (half_t)acc[i][j][1], (half_t)acc[i][j][2],
                (half_t)acc[i][j][3]};
        if (!GROUP) o *= sc;
        *(h4*)(C + (size_t)(m0 + m) * p.N + n0) = o;
      }
    }
  }
}

int launch_prefill(const GemmArgs& a, bool group, hipStream_t stream) {
  const int tiles_m = ceil_div(a.M, kPfTileM);
  const int tiles_n = a.N / kPfTileN;
  const int grid = tiles_m * tiles_n;
  if (group)
    hipLaunchKernelGGL(prefill_kernel<true>, dim3(grid), dim3(256), 0, stream, a, tiles_m, tiles_n);
  else
    hipLaunchKernelGGL(prefill_kernel<false>, dim3(grid), dim3(256), 0, stream, a, tiles_m,
                       tiles_n);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

}  // namespace w4a16
