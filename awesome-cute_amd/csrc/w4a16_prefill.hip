// Prefill W4A16 kernel on 64-row tiles: 49 to 64 rows over big weights, and
// more rows while twice as many tiles (against the 128-row tiles of
// w4a16_prefill_wide.hip) save k slices.  With four row blocks every unpacked
// weight word meets only four MFMAs, so the loop is bound by the unpack's issue
// slots, not by the matrix pipe; the design keeps everything else out of their
// way.
//
// One workgroup of 8 waves (two per SIMD) owns a 16*RB-row x 256-column tile
// of C (RB = 4 row blocks is the only instantiation) and, when the
// tiles alone would leave compute units idle, one of `ksplit` slices of the k
// range (the slices meet through the same ticketed exchange as the streaming
// kernel's).  Waves 0-3 run the first half of the workgroup's k range and
// waves 4-7 the second half over the same tile, and the two halves are added
// through LDS at the end.  Two waves per SIMD matter: a wave pays 11 to 22
// cycles of its own issue time for every LDS or global instruction, and the
// other wave's MFMAs run there.
// Within a half, wave w keeps a 16*RB x 64 fp32 accumulator (16*RB registers):
// columns 16j+8h+c of the two 64-column blocks 2p, 2p+1 with p = w/2 and
// j in {2(w%2), 2(w%2)+1}.
//   - Packed weights are copied to LDS as they lie in memory (coalesced
//     16-byte loads, four 2 KiB rows per stage and half); each lane then picks
//     the 8 bytes of its Marlin 16-byte piece that belong to its two 16-column
//     groups, unpacks them in registers and feeds them to the MFMA as the
//     first operand.  One unpack serves the RB MFMAs of the tile's row blocks.
//   - Activations are shared by the four waves of a half: they stage a
//     16*RB x 64 fp16 slab per k stage through a ring of three LDS buffers,
//     stored in the k-slot order the weight layout dictates so that an
//     operand is one conflict-free ds_read_b128.
// Per 32-deep k step a wave issues 4*RB MFMAs, RB + 2 LDS reads and the unpack
// of 4 weight words (52 VALU instructions with group scales), software-
// pipelined one step ahead and dealt out four behind every MFMA.
#include "w4a16_common.hpp"

namespace w4a16 {

namespace {

constexpr int kPfTileN = 256;
constexpr int kPfStageK = 64;
constexpr int kPfSlabB = 4 * 2048;  // four 16-deep rows of packed weights
constexpr int kPfRing = 3;          // slabs in LDS per k half
constexpr int kOobPf = (int)0x80000000;

// LDS geometry of a tile of RB row blocks
template <int RB>
struct PfShape {
  static constexpr int kTileM = 16 * RB;
  static constexpr int kPlane = kTileM * 16;            // one k group of a step: rows x 16 bytes
  static constexpr int kStepBytes = 4 * kPlane + 128;   // one 32-deep k step of the A slab (+pad)
  static constexpr int kSlabA = 2 * kStepBytes;         // two steps per stage
  static constexpr int kStageBytes = kSlabA + kPfSlabB;
  static constexpr int kLdsBytes = 2 * kPfRing * kStageBytes;
  // the epilogue reuses the rings: 8 waves x RB/2 row blocks x 4 KiB of fp32
  // to swap, then the fp16 tile with padded rows
  static_assert(8 * (RB / 2) * 4096 <= kLdsBytes && kTileM * (kPfTileN * 2 + 16) <= kLdsBytes, "");
  // (64-row tiles: 8 KiB of bias sums sit behind the 64 KiB that the swap uses)
  static_assert(RB != 4 || 65536 + 8192 <= kLdsBytes, "");
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t pf_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

}  // namespace

template <bool GROUP, int RB>
__global__ __launch_bounds__(512) void prefill_kernel(GemmArgs p, int tiles_m, int tiles_n,
                                                      int ksplit) {
  extern __shared__ __attribute__((aligned(16))) char smem_all[];  // PfShape<RB>::kLdsBytes
  __shared__ int s_ticket;
  {
    // fetch every kernel argument in one round trip (the compiler would fetch
    // the pointers in a second one, just before the first load needs them)
    const void *a_ = p.A, *b_ = p.B, *s_ = p.S;
    void* c_ = p.C;
    int* l_ = p.locks;
    float* sc_ = p.scratch;
    asm volatile("" ::"s"(a_), "s"(b_), "s"(s_), "s"(c_), "s"(l_), "s"(sc_), "s"(p.M), "s"(p.N),
                 "s"(p.K), "s"(tiles_m), "s"(tiles_n), "s"(ksplit));
  }
  constexpr int kPfTileM = PfShape<RB>::kTileM;
  constexpr int kPlane = PfShape<RB>::kPlane;
  constexpr int kPfStepBytes = PfShape<RB>::kStepBytes;
  constexpr int kPfSlabA = PfShape<RB>::kSlabA;
  constexpr int kPfStageBytes = PfShape<RB>::kStageBytes;
  constexpr int HB = RB / 2;  // row blocks a wave finishes after the halves are added
  // Per-channel scales with 64-row tiles: every unpacked word meets only four
  // row blocks, so the loop is bound by the unpack's issue slots (36 VALU to 16
  // MFMAs per k step), not by the matrix pipe.  There the unpack stops at the
  // biased integers -- (q & 0x000f000f) | 0x6400 is fp16(1024 + n) and
  // (q & 0x00f000f0) | 0x5400 is fp16(64 + n) for the nibbles n of a word, five
  // instructions per word instead of nine -- and the biases and the zero point
  // (1032 and 72 per activation) are summed by one more MFMA per k step on a
  // constant weight operand, in a chain of exactly the shape of the weights'
  // chains, and subtracted at the end: what is left is sum a (n - 8), exact
  // integers times activations in fp32; a one-hot row returns fp16(n - 8)
  // exactly, and where every nibble is the zero point the two chains are the
  // same computation, so the difference is exactly zero.  The four waves of a
  // k half share the rows, so each sums the bias of one row block (the one it
  // visits first: wave w walks the row blocks starting from block w).
  constexpr bool BIAS = !GROUP && RB == 4;

  const int kh = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8);  // k half
  const int tid = threadIdx.x & 255;  // thread within the half
  char* smem = smem_all + kh * (kPfRing * kPfStageBytes);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int kg = lane >> 4;
  const int nu = lane & 15;
  const int pr = wave >> 1;  // pair of 64-column blocks
  const int jp = wave & 1;   // pair of 16-column groups inside each block

  // Workgroup ids are dealt round-robin to the 8 XCDs; give every XCD a
  // contiguous run of tile numbers so that the workgroups sharing an L2 read
  // the same rows of A and neighbouring columns of B.
  // The k slices of a tile are consecutive work indices, so they share an XCD.
  const int total = tiles_m * tiles_n * ksplit;
  int work = (int)blockIdx.x;
  if ((total & 7) == 0) work = (work & 7) * (total >> 3) + (work >> 3);
  const int tile = work / ksplit;
  const int ks = work - tile * ksplit;
  int tm, tn;
  if ((tiles_n & 7) == 0) {
    // tiles numbered in panels of 8 column tiles, row tile next: an XCD's run
    // of tiles is then closer to square (4 x 8 instead of 2 x 16 at M = 2048,
    // N = 4096) and shares more of A and B (8192 x 8192, M = 2048: 226 -> 221 us)
    const int per_panel = 8 * tiles_m;
    const int panel = tile / per_panel, within = tile - panel * per_panel;
    tm = within >> 3;
    tn = panel * 8 + (within & 7);
  } else {
    tm = tile / tiles_n;
    tn = tile - tm * tiles_n;
  }
  const int m0 = tm * kPfTileM;
  const int rows = min(kPfTileM, p.M - m0);

  const __amdgpu_buffer_rsrc_t rB = pf_rsrc(p.B, (unsigned)p.K * (unsigned)(p.N / 2));
  const __amdgpu_buffer_rsrc_t rS =
      pf_rsrc(p.S, (unsigned)(GROUP ? p.K / 128 : 1) * (unsigned)p.N * 2u);
  const __amdgpu_buffer_rsrc_t rA =
      pf_rsrc((const char*)p.A + (size_t)m0 * p.K * 2, (unsigned)rows * (unsigned)p.K * 2u);
  const int b_row = p.N * 8;

  // Packed weights go through LDS too: the 256 threads of a half copy the
  // stage's four 2 KiB rows with coalesced 16-byte loads, and every lane then
  // picks its 8 bytes (Marlin piece (t = kg, c = nu%8) of block 2p + nu/8,
  // words 2jp, 2jp+1).  In LDS the two halves of the pieces of a pair of
  // 64-column blocks lie apart -- 64 x 8 bytes of words 0,1, then 64 x 8 bytes
  // of words 2,3 -- so that the 64 lanes of a wave read 512 contiguous bytes,
  // and the pieces are rotated inside each group of four so that each half of
  // the wave touches every bank once (with the halves interleaved a wave used
  // half of the banks: 12 cycles per read instead of 4).
  const int bx = tid & 127;  // 16-byte piece inside a row, for the copy
  const int b_ld = 2048 * tn + 16 * bx;
  const int b_a = (bx & 63) >> 2;
  const int b_wr = kPfSlabA + (wave >> 1) * 2048 + (bx >> 6) * 1024 +
                   8 * (4 * b_a + (((bx & 3) + (b_a >> 2)) & 3));
  const int b_rd = kPfSlabA + pr * 1024 + 8 * (4 * nu + ((kg + (nu >> 2)) & 3)) + 512 * jp;
  const int s_lane = (256 * tn + 128 * pr + 8 * nu) * 2 + 8 * jp;

  // slab staging: thread (row = tid/8 + 32 i, chunk x = tid%8) moves 16 bytes;
  // rows past the end of A read as zeros (out-of-range buffer offset)
  const int ax = tid & 7;
  int a_lane[HB];
#pragma unroll
  for (int i = 0; i < HB; i++) {
    const int r = (tid >> 3) + 32 * i;
    a_lane[i] = r < rows ? r * p.K * 2 + 16 * ax : kOobPf;
  }
  // LDS slab: [step][k group][row][slot] dwords; chunk x -> step x/4, slot x%4
  const int a_wr = (ax >> 2) * kPfStepBytes + (tid >> 3) * 16 + (ax & 3) * 4;
  const int a_rd = kg * kPlane + nu * 16;
  // row block visited in turn i: (i + rot) % RB
  const int rot = BIAS ? wave : 0;
  auto row_block = [&](int i) { return BIAS ? ((i + rot) & (RB - 1)) : i; };

  const DequantConsts dc;
  // this half's stages: [s_begin, s_end) of the K/64 stages; the loop runs the
  // same count in both halves (a stage past s_end fetches zeros)
  const int stages_all = p.K / kPfStageK;
  // this workgroup's slice (at most 8 slices of at most 2^18 stages: 32 bits do)
  const int st0 = (int)((unsigned)ks * (unsigned)stages_all / (unsigned)ksplit);
  const int st1 = (int)((unsigned)(ks + 1) * (unsigned)stages_all / (unsigned)ksplit);
  const int half_stages = (st1 - st0 + 1) >> 1;
  const int s_begin = st0 + kh * half_stages;
  const int s_end = kh ? st1 : st0 + half_stages;
  const int stages = half_stages;

  i4 areg[HB];  // A slab of the stage after next, in flight
  i4 bcopy[2];  // its packed weights
  i2 sreg[2];   // group scales of this stage and the next

  auto issue_s = [&](int slot, int s) {
    const int sg = s_begin + s;  // stage in the whole k range
    const int inv = sg < s_end ? 0 : kOobPf;
    if (GROUP)
      sreg[slot] = __builtin_amdgcn_raw_buffer_load_b64(rS, s_lane | inv,
                                                        (sg >> 1) * p.N * 2, 0);
  };
  auto issue_a = [&](int s) {
    const int sg = s_begin + s;
    const int inv = sg < s_end ? 0 : kOobPf;
#pragma unroll
    for (int i = 0; i < HB; i++)
      areg[i] = __builtin_amdgcn_raw_buffer_load_b128(rA, a_lane[i] | inv, sg * 128, 0);
#pragma unroll
    for (int i = 0; i < 2; i++)
      bcopy[i] = __builtin_amdgcn_raw_buffer_load_b128(
          rB, b_ld | inv, (4 * sg + 2 * i + (wave >> 1)) * b_row, 0);
  };
  auto store_a = [&](int ring) {
    char* base = smem + ring * kPfStageBytes;
#pragma unroll
    for (int i = 0; i < HB; i++)
#pragma unroll
      for (int g = 0; g < 4; g++) *(int*)(base + a_wr + g * kPlane + i * 32 * 16) = areg[i][g];
#pragma unroll
    for (int i = 0; i < 2; i++) {
      *(i2*)(base + b_wr + i * 4096) = (i2){bcopy[i][0], bcopy[i][1]};
      *(i2*)(base + b_wr + i * 4096 + 512) = (i2){bcopy[i][2], bcopy[i][3]};
    }
  };

  f4 acc[RB][4];
#pragma unroll
  for (int i = 0; i < RB; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};

  // the biases of the sums of row block `rot` (see BIAS above) and the constant
  // weight operand that sums them: (1032, 72) per (low, high) nibble pair
  f4 bias = {0.f, 0.f, 0.f, 0.f};
  const i4 wbias_i = {0x64086408, 0x54805480, 0x64086408, 0x54805480};
  const h8 wbias = __builtin_bit_cast(h8, wbias_i);
  h8 w[2][4];  // unpacked weights of the current and the next k step
  i4 af[4];    // ring of activation operands, three ahead of the MFMAs
  i2 bw[2];    // packed weight words of the next k step (its two 16-deep rows)

  // unpack the two words of 16-column group j2 of k step (slot, h) into w[buf]
  const int ex_hi = dc.ex - 0x10001000;  // 0x54005400: fp16(64 + n) for a nibble at bit 4
  auto dequant_pair = [&](int buf, int slot, int h, int j2) {
    (void)h;
    if constexpr (BIAS) {
      const int q0 = bw[0][j2], q1 = bw[1][j2];
      const int r0 = (int)((unsigned)q0 >> 8), r1 = (int)((unsigned)q1 >> 8);
      const i4 lo = {(q0 & dc.lo_mask) | dc.ex, (q0 & dc.hi_mask) | ex_hi,
                     (q1 & dc.lo_mask) | dc.ex, (q1 & dc.hi_mask) | ex_hi};
      const i4 hi = {(r0 & dc.lo_mask) | dc.ex, (r0 & dc.hi_mask) | ex_hi,
                     (r1 & dc.lo_mask) | dc.ex, (r1 & dc.hi_mask) | ex_hi};
      w[buf][2 * j2] = __builtin_bit_cast(h8, lo);
      w[buf][2 * j2 + 1] = __builtin_bit_cast(h8, hi);
      return;
    }
    h2 s2 = GROUP ? as_h2(sreg[slot][j2]) : (h2){(half_t)1.f, (half_t)1.f};
    h2 l0, h0, l1, h1, m0_, n0_, m1_, n1_;
    dequant_word<GROUP>(bw[0][j2], s2, dc, l0, h0, l1, h1);
    dequant_word<GROUP>(bw[1][j2], s2, dc, m0_, n0_, m1_, n1_);
    w[buf][2 * j2] = make_h8(l0, h0, m0_, n0_);
    w[buf][2 * j2 + 1] = make_h8(l1, h1, m1_, n1_);
  };
  // fetch the packed words of k step h of the slab at `stage_base`
  auto read_bw = [&](const char* stage_base, int h) {
    bw[0] = *(const i2*)(stage_base + b_rd + (2 * h) * 2048);
    bw[1] = *(const i2*)(stage_base + b_rd + (2 * h + 1) * 2048);
  };
  auto read_frag = [&](int idx, const char* step_base, int i) {
    af[idx] = *(const i4*)(step_base + a_rd + row_block(i) * 256);
  };

  // One operation of the unpack of word bw[r][j2] into w[buf] (the sequence of
  // dequant_word, cut up so that it can be dealt out between the MFMAs):
  // op 0 the shift, 1-4 the four mask-and-exponent words, 5-8 the bias
  // removal, 9-12 (group mode) the scale.
  int wt[2];  // the shifted words
  auto dq_op = [&](int buf, int slot, int j2, int r, int op) {
    const h2 sub = {(half_t)1032.f, (half_t)1032.f};
    const h2 mul = {(half_t)0.0625f, (half_t)0.0625f};
    const h2 add = {(half_t)-72.f, (half_t)-72.f};
    i4& lo = *(i4*)&w[buf][2 * j2];      // column c: dwords 2r (k pair 2t), 2r+1 (k pair 2t+8)
    i4& hi = *(i4*)&w[buf][2 * j2 + 1];  // column c+8
    const int q = bw[r][j2];
    switch (op) {
      case 0: wt[r] = (int)((unsigned)q >> 8); break;
      case 1: lo[2 * r] = (q & dc.lo_mask) | dc.ex; break;
      case 2: lo[2 * r + 1] = (q & dc.hi_mask) | (BIAS ? ex_hi : dc.ex); break;
      case 3: hi[2 * r] = (wt[r] & dc.lo_mask) | dc.ex; break;
      case 4: hi[2 * r + 1] = (wt[r] & dc.hi_mask) | (BIAS ? ex_hi : dc.ex); break;
      case 5: lo[2 * r] = as_int(as_h2(lo[2 * r]) - sub); break;
      case 6: lo[2 * r + 1] = as_int(__builtin_elementwise_fma(as_h2(lo[2 * r + 1]), mul, add)); break;
      case 7: hi[2 * r] = as_int(as_h2(hi[2 * r]) - sub); break;
      case 8: hi[2 * r + 1] = as_int(__builtin_elementwise_fma(as_h2(hi[2 * r + 1]), mul, add)); break;
      default: {
        const h2 s2 = as_h2(sreg[slot][j2]);
        const h2 s0 = {s2[0], s2[0]};
        const h2 s1 = {s2[1], s2[1]};
        if (op == 9) lo[2 * r] = as_int(as_h2(lo[2 * r]) * s0);
        if (op == 10) lo[2 * r + 1] = as_int(as_h2(lo[2 * r + 1]) * s0);
        if (op == 11) hi[2 * r] = as_int(as_h2(hi[2 * r]) * s1);
        if (op == 12) hi[2 * r + 1] = as_int(as_h2(hi[2 * r + 1]) * s1);
      }
    }
  };

  // One 32-deep k step: 4*RB MFMAs on w[h] and the operand ring, while the
  // operands of the next step are fetched from LDS and its weights unpacked
  // into w[h^1].  Two VALU instructions issued behind an MFMA cost nothing, a
  // third costs its full four cycles, so the unpack is dealt out two (with 64
  // rows: four) operations per MFMA instead of standing in blocks between
  // them; scheduling fences keep it that way.  `extra(m)` runs behind MFMA m.
  auto step = [&](int h, const char* cur_base, const char* nxt_base, const char* nxt_stage,
                  int nslot, int nh, auto&& extra) {
    constexpr int kOpsPerWord = GROUP ? 13 : (BIAS ? 5 : 9);
    constexpr int kPairsPerMfma = RB == 8 ? 1 : 2;  // one operation of each word of a pair
    constexpr int kFirst = RB == 8 ? 6 : 3;         // the words are read from LDS behind MFMA 0
#pragma unroll
    for (int i = 0; i < RB; i++) {
      if (i == 0) read_bw(nxt_stage, nh);
      if (i + 3 < RB)
        read_frag((i + 3) & 3, cur_base, i + 3);
      else
        read_frag((i + 3) & 3, nxt_base, i + 3 - RB);
      const h8 a = __builtin_bit_cast(h8, af[i & 3]);
      if constexpr (BIAS) {
        if (i == 0) bias = __builtin_amdgcn_mfma_f32_16x16x32_f16(wbias, a, bias, 0, 0, 0);
      }
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int m = 4 * i + j;
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[h][j], a, acc[i][j], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < kPairsPerMfma; u++) {
          const int t = (m - kFirst) * kPairsPerMfma + u;
          if (t >= 0 && t < 2 * kOpsPerWord) {
            dq_op(h ^ 1, nslot, t / kOpsPerWord, 0, t % kOpsPerWord);
            dq_op(h ^ 1, nslot, t / kOpsPerWord, 1, t % kOpsPerWord);
          }
        }
        extra(m);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // The slab traffic of a stage, dealt out behind the MFMAs of its first step:
  // each staging register is written to LDS (slab cs+1) and then requested
  // again (slab cs+2), so every load has a whole stage to arrive.
  auto stage_traffic = [&](int m, int ring_next, int s_next2) {
    constexpr int kPerA = 3;  // two pairs of dword writes and the reload of one register
    constexpr int kBegin = 4 * RB - (HB * kPerA + 2 * 2);
    const int x = m - kBegin;
    if (x < 0) return;
    char* base = smem + ring_next * kPfStageBytes;
    const int sg = s_begin + s_next2;
    const int inv = sg < s_end ? 0 : kOobPf;
    if (x < HB * kPerA) {
      const int i = x / kPerA, g = x % kPerA;
      if (g < 2) {
        // two planes per slot: the pair becomes one ds_write2st64_b32
        *(int*)(base + a_wr + (2 * g) * kPlane + i * 32 * 16) = areg[i][2 * g];
        *(int*)(base + a_wr + (2 * g + 1) * kPlane + i * 32 * 16) = areg[i][2 * g + 1];
      } else
        areg[i] = __builtin_amdgcn_raw_buffer_load_b128(rA, a_lane[i] | inv, sg * 128, 0);
    } else {
      const int y = x - HB * kPerA, i = y >> 1;
      if ((y & 1) == 0)
      {
        *(i2*)(base + b_wr + i * 4096) = (i2){bcopy[i][0], bcopy[i][1]};
        *(i2*)(base + b_wr + i * 4096 + 512) = (i2){bcopy[i][2], bcopy[i][3]};
      }
      else
        bcopy[i] = __builtin_amdgcn_raw_buffer_load_b128(
            rB, b_ld | inv, (4 * sg + 2 * i + (wave >> 1)) * b_row, 0);
    }
  };

  // prologue: slab 0 in LDS, slab 1 in flight, scales of stages 0 and 1
  issue_a(0);
  issue_s(0, 0);
  issue_s(1, 1);
  store_a(0);
  issue_a(1);
  __syncthreads();
  read_bw(smem, 0);
  dequant_pair(0, 0, 0, 0);
  dequant_pair(0, 0, 0, 1);
  read_frag(0, smem, 0);
  read_frag(1, smem, 1);
  read_frag(2, smem, 2);

  // The instruction arbiter favours the older waves (the first k half); a
  // higher priority for the second half evens the two out (measured: never
  // slower, up to 4 % faster depending on the schedule of the loop).
  if (kh) __builtin_amdgcn_s_setprio(1);
  int ring = 0;  // LDS slab of the stage being computed
  for (int s = 0; s < stages; s += 2) {
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int cs = s + u;
      // (an odd count of stages computes one stage of zeros in the second copy
      // of the last turn: an exit here costs this loop more than it saves)
      const int ring_next = ring == kPfRing - 1 ? 0 : ring + 1;
      const char* cur = smem + ring * kPfStageBytes;
      const char* nxt = smem + ring_next * kPfStageBytes;
      // step 0: meanwhile slab cs+1 goes to LDS and slab cs+2 is requested.
      // The slab written here was last read two stages ago, and every wave
      // has passed the previous barrier since, so one barrier per stage is
      // enough; it sits mid-stage, where no wave needs the new slab yet.
      step(0, cur, cur + kPfStepBytes, cur, u, 1,
           [&](int m) { stage_traffic(m, ring_next, cs + 2); });
      __syncthreads();
      // step 1: the scales of this stage are spent, request those of stage cs+2
      step(1, cur + kPfStepBytes, nxt, nxt, u ^ 1, 0, [](int) {});
      issue_s(u, cs + 2);
      ring = ring_next;
    }
  }

  // ---- epilogue.  The k halves swap the row blocks they will not write
  // (half 0 keeps blocks 0..HB-1, half 1 the rest) through LDS and add; the
  // slab rings are dead by now.
  const int own = HB * kh;  // first row block this wave finishes
  __syncthreads();
  if constexpr (BIAS) {
    // every wave of a k half needs the bias of all four row blocks: wave w has
    // summed that of block w
    f4* bx = (f4*)(smem_all + 65536);
    bx[(kh * 4 + wave) * 64 + lane] = bias;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < RB; i++) {
      const f4 b = bx[(kh * 4 + row_block(i)) * 64 + lane];
#pragma unroll
      for (int j = 0; j < 4; j++) acc[i][j] -= b;
    }
  }
  {
    f4* out = (f4*)smem_all + (size_t)(kh * 4 + wave) * (HB * 4 * 64);
#pragma unroll
    for (int i = 0; i < HB; i++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        out[(i * 4 + j) * 64 + lane] = kh ? acc[i][j] : acc[HB + i][j];
  }
  __syncthreads();
  f4 fin[HB][4];
  {
    const f4* in = (const f4*)smem_all + (size_t)((kh ^ 1) * 4 + wave) * (HB * 4 * 64);
#pragma unroll
    for (int i = 0; i < HB; i++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        fin[i][j] = (kh ? acc[HB + i][j] : acc[i][j]) + in[(i * 4 + j) * 64 + lane];
  }

  // ---- k slices of other workgroups.  Same exchange as the streaming
  // kernel's: every slice writes its fp32 tile through to memory (whole 1 KiB
  // lines per wave instruction), waits for the acknowledgement, takes the
  // tile's ticket; the last arrival adds all slices in slice order (its own
  // from registers at its place in that order) and carries on.  Nobody spins.
  if (ksplit > 1) {
    constexpr int part_bytes = kPfTileM * kPfTileN * 4;
    const __amdgpu_buffer_rsrc_t rP = pf_rsrc(p.scratch, 0x7fffffffu);
    const int at = ((kh * 4 + wave) * (HB * 4) * 64 + lane) * 16;
    const int mine = work * part_bytes;
#pragma unroll
    for (int i = 0; i < HB; i++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, fin[i][j]), rP,
                                               at + (i * 4 + j) * 1024, mine, 16 /* sc1 */);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): my stores have been acknowledged
    __syncthreads();
    if (threadIdx.x == 0)
      s_ticket = __hip_atomic_fetch_add(&p.locks[tile], 1, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != ksplit - 1) return;  // a later slice finishes the tile
    f4 sum[HB][4];
    for (int k2 = 0; k2 < ksplit; k2++) {
      f4 v[HB][4];
      if (k2 != ks) {
        const int theirs = (tile * ksplit + k2) * part_bytes;
#pragma unroll
        for (int i = 0; i < HB; i++)
#pragma unroll
          for (int j = 0; j < 4; j++)
            v[i][j] = __builtin_bit_cast(
                f4, __builtin_amdgcn_raw_buffer_load_b128(rP, at + (i * 4 + j) * 1024, theirs,
                                                          16 /* sc1 */));
      } else {
#pragma unroll
        for (int i = 0; i < HB; i++)
#pragma unroll
          for (int j = 0; j < 4; j++) v[i][j] = fin[i][j];
      }
#pragma unroll
      for (int i = 0; i < HB; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) sum[i][j] = k2 == 0 ? v[i][j] : sum[i][j] + v[i][j];
    }
#pragma unroll
    for (int i = 0; i < HB; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) fin[i][j] = sum[i][j];
    if (threadIdx.x == 0)  // counters are handed back zeroed
      __hip_atomic_store(&p.locks[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();

  // fp16 tile -> LDS in row-major order, then whole 512-byte rows go out with
  // coalesced 16-byte stores.  Lane holds row 16 i + nu and, per (j2, h), four
  // consecutive columns.
  constexpr int kPitch = kPfTileN * 2 + 16;  // bytes per tile row in LDS
  const int q = lane >> 4;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int nloc = 128 * pr + 64 * (q >> 1) + 16 * (2 * jp + (j >> 1)) + 8 * (j & 1) + 4 * (q & 1);
    h4 sc = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
    if (!GROUP) {
      const half_t* S = (const half_t*)p.S;
#pragma unroll
      for (int r = 0; r < 4; r++) sc[r] = S[scale_index_single(kPfTileN * tn + nloc + r)];
    }
#pragma unroll
    for (int i = 0; i < HB; i++) {
      const int m = 16 * row_block(own + i) + nu;
      h4 o = {(half_t)fin[i][j][0], (half_t)fin[i][j][1], (half_t)fin[i][j][2],
              (half_t)fin[i][j][3]};
      if (!GROUP) o *= sc;
      *(h4*)(smem_all + m * kPitch + nloc * 2) = o;
    }
  }
  __syncthreads();
  half_t* C = (half_t*)p.C;
#pragma unroll
  for (int it = 0; it < kPfTileM / 16; it++) {
    const int piece = it * 512 + (int)threadIdx.x;  // 16-byte piece of the tile
    const int m = piece >> 5;
    const int c16 = piece & 31;
    if (m < rows) {
      const i4 v = *(const i4*)(smem_all + m * kPitch + c16 * 16);
      // nobody reads C again in this launch: keep it out of the way of A and B in L2
      __builtin_nontemporal_store(v, (i4*)(C + (size_t)(m0 + m) * p.N + kPfTileN * tn + c16 * 8));
    }
  }
}

template <int RB>
static int configure_rb() {
  // more LDS than the default per-workgroup limit: opt in per kernel and device
  constexpr int lds = PfShape<RB>::kLdsBytes;
  if (hipFuncSetAttribute((const void*)prefill_kernel<true, RB>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess ||
      hipFuncSetAttribute((const void*)prefill_kernel<false, RB>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
    return 3;
  return 0;
}

int configure_prefill_kernels() { return configure_rb<4>() ? 3 : 0; }

template <bool GROUP, int RB>
static void launch_rb(const GemmArgs& a, int ksplit, hipStream_t stream) {
  const int tiles_m = ceil_div(a.M, PfShape<RB>::kTileM);
  const int tiles_n = a.N / kPfTileN;
  constexpr int lds = PfShape<RB>::kLdsBytes;
  hipLaunchKernelGGL((prefill_kernel<GROUP, RB>), dim3(tiles_m * tiles_n * ksplit), dim3(512), lds,
                     stream, a, tiles_m, tiles_n, ksplit);
}

int launch_prefill(const GemmArgs& a, bool group, int ksplit, hipStream_t stream) {
  if (group) launch_rb<true, 4>(a, ksplit, stream); else launch_rb<false, 4>(a, ksplit, stream);
  return launch_status();
}

}  // namespace w4a16
