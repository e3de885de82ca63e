// Column-strip W4A16 kernel, 16 activation rows per workgroup (decode, small
// batches, and more rows over small weights): a workgroup owns 16*CS columns
// over the whole k range, so no two workgroups ever meet -- no partial sums in
// global memory, no counters, no last arrival.  What that exchange costs a launch of a few microseconds
// (store, acknowledge, ticket, read back: four trips to memory one after the
// other) is more than what narrow strips cost the weight stream.
//
// A strip is the unit the packed layout allows (reference marlin.py:119-129):
// in every row of B (16 k-values of every column) the 128 bytes of Marlin lanes
// 8s..8s+7 of a 64-column block hold exactly the 16 columns
// {16j + 8h + 2s + e : j < 4, h < 2, e < 2} of that block, one whole cache
// line.  MFMA lane (kg, nu = 8e + 2j + h) needs from that line one word --
// word j of Marlin lane (t = kg, c = 2s + e), its low or high byte pairs by h
// -- of rows 2ks and 2ks+1 per 32-deep k step.  A wave fetches the lines 16
// bytes per lane, eight rows per instruction, passes them through LDS as they
// are and reads its words back in MFMA order (one ds_read2_b32 per k step, no
// bank conflict).  Fetching the words straight into MFMA order with 4-byte
// loads costs four times the load instructions, which the compute unit issues
// one per ten cycles or so: its youngest wave then had requested its weights
// 1.4 us into the kernel instead of 0.9.
//
// The eight waves of a workgroup split the k range into contiguous runs of
// chunks (256/CS k-values); each keeps one or two chunks in flight in registers,
// stages the activations of a chunk through LDS into operand order by itself
// (no barrier in the loop), and the eight partial strips are summed through
// LDS once, at the end.  Every workgroup reads all activation rows it
// computes, M*K*2 bytes against 8*CS*K bytes of weights, so narrow strips pay
// off for few rows.
//
// More than 16 rows are cut into parts of 16, each a workgroup of its own over
// the same strips: grid = strip sets x parts.  The parts of a strip set have
// neighbouring work indices (one L2), so the weights come from memory once and
// mostly from the L2 for the other parts (M = 64, N = K = 4096: 13.5 MB of
// memory traffic per launch, 9.7 MB algorithmic); every part unpacks them again, which a
// launch of a few microseconds over small weights can afford.  (Several row
// blocks inside one workgroup, sharing every unpacked weight, were slower
// wherever they were tried: a workgroup then reads 16 x row blocks rows of
// activations, and eight waves' rows of a chunk fill LDS.  M = 64: N = 2048,
// K = 4096 12.9 us with four row blocks per workgroup, 7.0 in parts; N = 512,
// K = 1024 5.4 / 3.6; N = K = 4096 13.1 / 9.5.)
#include "w4a16_common.hpp"

namespace w4a16 {

namespace {

constexpr int kStripOob = (int)0x80000000;  // offset past any buffer (sizes are < 2 GiB)
constexpr int kStripWaves = 8;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t strip_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

}  // namespace

// CS: 16-column strips per workgroup (1 to 4; three where N's strips fill the
// compute units better in threes, the last workgroup then with fewer).
// MR: activation rows staged (2, 4, 8 or 16; rows past M are read as zeros).
template <int CS, int MR>
struct StripShape {
  // a chunk is two weight loads of 1 KiB per wave (three for three strips): 16
  // (24) lines of 128 bytes, CS lines per row of B, two rows per k step
  static constexpr int kLoads = CS == 3 ? 3 : 2;
  static constexpr int kSteps = 4 * kLoads / CS;      // 32-deep k steps per chunk
  static constexpr int kChunkK = 32 * kSteps;         // k-values per chunk
  static constexpr int kRowBytes = 2 * kChunkK;       // of one activation row per chunk
  static constexpr int kLanesPerRow = kRowBytes / 16;
  static constexpr int kRowsPerLoad = 64 / kLanesPerRow;
  static constexpr int kALoads = (MR + kRowsPerLoad - 1) / kRowsPerLoad;
  static constexpr int kRowsStaged = kALoads * kRowsPerLoad;
  // 16 bytes of padding per row: MFMA lanes (kg, row) then read 64 distinct banks
  static constexpr int kStride = kRowBytes + 16;
  // per wave: the activation rows of a chunk, then its 2 (3) KiB of weights
  static constexpr int kWeightBase = kRowsStaged * kStride;
  static constexpr int kStagePerWave = kWeightBase + 1024 * kLoads;
  static constexpr int kReduceBase = kStripWaves * kStagePerWave;
  static constexpr int kBytes = kReduceBase + kStripWaves * CS * 1024;
};

template <int CS, int MR, bool GROUP, int DEPTH>
__global__ __launch_bounds__(64 * kStripWaves) void strip_kernel(GemmArgs p) {
  using Sh = StripShape<CS, MR>;
  constexpr int KC = Sh::kSteps;
  constexpr int NL = Sh::kLoads;
  constexpr int NSC = GROUP ? (CS == 1 ? 2 : 1) : 0;  // scale rows a chunk touches
  // Group scales, up to 8 rows: applied to the sums of a group instead of to
  // its weights (below).  With 16 rows staged the two forms are within 1.5 %
  // of each other either way (M = 16: N = 11008, K = 4096 9.3 us against 9.2,
  // N = K = 4096 5.85 / 5.83, N = 8192, K = 2048 5.0 / 5.1) and the weights
  // keep their scales.
  constexpr bool kScaleSums = GROUP && MR <= 8;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  {
    // all kernel arguments in one trip to memory, ahead of the first load
    const void *a_ = p.A, *b_ = p.B, *s_ = p.S;
    void* c_ = p.C;
    asm volatile("" ::"s"(a_), "s"(b_), "s"(s_), "s"(c_), "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.gpb),
                 "s"(p.row_parts));
  }
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int kg = lane >> 4;
  const int nu = lane & 15;
  // (p.gpb carries the grid: the launch's own record of it is a second trip to memory)
  const int wid = xcd_work_index((int)blockIdx.x, p.gpb);
  // rows in parts (p.row_parts > 1): work index w computes rows [16 part, 16
  // part + 16) of strip set w / row_parts, part = w % row_parts
  const int set = p.row_parts > 1 ? wid / p.row_parts : wid;
  const int row0 = p.row_parts > 1 ? 16 * (wid - set * p.row_parts) : 0;
  const int strip0 = set * CS;  // my first strip; strip S holds bytes [128 S, 128 S + 128) of a row of B
  const int n_strips = p.N >> 4;  // (three strips per workgroup: the last one may hold fewer)

  // my chunks [c0, c1) of the k range
  const int n_chunks = ceil_div(p.K, Sh::kChunkK);
  const int c0 = (wave * n_chunks) / kStripWaves;
  const int c1 = ((wave + 1) * n_chunks) / kStripWaves;

  const __amdgpu_buffer_rsrc_t rB = strip_rsrc(p.B, (unsigned)p.K * (unsigned)(p.N / 2));
  const __amdgpu_buffer_rsrc_t rA = strip_rsrc(p.A, (unsigned)p.M * (unsigned)p.K * 2u);
  const __amdgpu_buffer_rsrc_t rS =
      strip_rsrc(p.S, (unsigned)(GROUP ? p.K / 128 : 1) * (unsigned)p.N * 2u);
  const int b_row = p.N * 8;  // bytes per row of B

  // weights, fetched: the 128 (192) lanes of a chunk's loads take 16 bytes each
  // in the order [row][strip][Marlin lane]; used: word j = (nu/2)%4 of Marlin
  // lane (t = kg, c = 2s + e), e = nu/8
  int b_lane[NL];
  bool b_mine[NL];  // (a strip past the last one would be the next row's first)
#pragma unroll
  for (int i = 0; i < NL; i++) {
    const int idx = 64 * i + lane;
    const int strip = strip0 + (idx / 8) % CS;
    b_lane[i] = (idx / (8 * CS)) * b_row + 128 * strip + 16 * (idx % 8);
    b_mine[i] = CS != 3 || strip < n_strips;
  }
  const int b_rd = (4 * (nu >> 3) + kg) * 16 + 4 * ((nu >> 1) & 3);
  const int shift = 8 * (nu & 1);  // h = nu%2 picks the low or the high byte pairs
  // group scales: a group's row holds the column of slot nu of strip S at
  // position 16S + 8e + 2j + h = 16S + nu (the 64-column permutation of
  // reference marlin.py:50-51 puts the 8 columns of a Marlin lane side by side).
  // Applied to the weights, MFMA lane (kg, nu) needs the scale of slot nu;
  // applied to the sums, result lane (row, kg) needs those of the slots 4 kg
  // ... 4 kg + 3, four scales in 8 bytes.
  const int s_lane = 2 * (16 * strip0 + (kScaleSums ? 4 * kg : nu));
  // activations: lane (row, piece) fetches 16 bytes (8 k-values)
  const int a_row = lane / Sh::kLanesPerRow;
  const int a_piece = lane % Sh::kLanesPerRow;
  int a_lane[Sh::kALoads];
#pragma unroll
  for (int i = 0; i < Sh::kALoads; i++) {
    const int r = i * Sh::kRowsPerLoad + a_row;
    a_lane[i] = row0 + r < p.M ? (row0 + r) * p.K * 2 + 16 * a_piece : kStripOob;
  }
  char* stage = smem + wave * Sh::kStagePerWave;
  const int a_wr = a_row * Sh::kStride + 16 * a_piece;
  // MFMA lane (kg, row nu) reads dwords kg, kg+4, kg+8, kg+12 of the 64 bytes
  // of its row and k step; rows that are not staged read row 0 (never stored)
  const int a_rd = (nu < Sh::kRowsStaged ? nu : 0) * Sh::kStride + 4 * kg;

  // Result lane (row m = lane%16, q = lane/16) holds in register r the column
  // slot nu = 4q + r, i.e. e = q/2, j = 2(q%2) + r/2, h = r%2: column
  // 16j + 8h + 2s' + e of the block, s' the strip's place in the block.  The
  // per-channel scales of those columns are fetched now (wave s < CS writes
  // strip s in the end).
  const int res_strip = strip0 + wave;
  const int res_col = 64 * (res_strip >> 2) + 2 * (res_strip & 3) + 32 * (kg & 1) + (kg >> 1);
  unsigned short chan[4] = {0, 0, 0, 0};
  if constexpr (!GROUP) {
    if (wave < CS && res_strip < n_strips) {
#pragma unroll
      for (int r = 0; r < 4; r++)
        chan[r] = __builtin_amdgcn_raw_buffer_load_b16(
            rS, 2 * scale_index_single(res_col + 16 * (r >> 1) + 8 * (r & 1)), 0, 0);
    }
  }

  const DequantConsts dc;

  i4 bq[DEPTH][NL];
  i2 sq[DEPTH][NSC > 0 ? NSC * CS : 1];
  i4 aq[DEPTH][Sh::kALoads];

  // Request chunk c into ring slot `slot`.  The per-lane part of an address is
  // what the hardware checks against the buffer's size, so it carries the row:
  // rows of B and of the scales past the end of K then read as zeros by
  // themselves, and a chunk that is not mine is requested at an offset past
  // everything, which touches no memory.  (Only the rows of A need a test of
  // their own: past the end of a row lies the next row.)
  auto issue = [&](int slot, int c, bool valid) {
    __builtin_amdgcn_sched_barrier(0);
    const int inv = valid ? 0 : kStripOob;
    const int k0 = c * Sh::kChunkK;
#pragma unroll
    for (int i = 0; i < Sh::kALoads; i++) {
      const int off = (k0 + 8 * a_piece < p.K) ? a_lane[i] : kStripOob;
      aq[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(rA, off | inv, 2 * k0, 0);
    }
    if constexpr (GROUP) {
      int vs = s_lane + (valid ? (k0 >> 7) * p.N * 2 : kStripOob);
#pragma unroll
      for (int g = 0; g < NSC; g++) {
#pragma unroll
        for (int s = 0; s < CS; s++)
          if constexpr (kScaleSums)
            sq[slot][g * CS + s] = __builtin_amdgcn_raw_buffer_load_b64(rS, vs + 32 * s, 0, 0);
          else
            sq[slot][g * CS + s][0] = __builtin_amdgcn_raw_buffer_load_b16(rS, vs + 32 * s, 0, 0);
        vs += p.N * 2;
      }
    }
    // the weights last: what comes back first is small and near
    const int b_chunk = valid ? c * (KC * 2) * b_row : kStripOob;
#pragma unroll
    for (int i = 0; i < NL; i++)
      bq[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(
          rB, b_mine[i] ? b_lane[i] + b_chunk : kStripOob, 0, 2);
    __builtin_amdgcn_sched_barrier(0);
  };

  f4 acc[CS][2];
#pragma unroll
  for (int s = 0; s < CS; s++) acc[s][0] = acc[s][1] = (f4){0.f, 0.f, 0.f, 0.f};

  // Group scales applied to the sums of a group: its k steps are summed from
  // zero (`part`) and the sums scaled (fp32) into the accumulators -- four
  // multiply-adds per group and strip instead of four packed multiplies per k
  // step (M = 1: N = K = 4096 4.31 -> 4.22 us, 8192 x 8192 8.6 -> 8.2, N =
  // 11008, K = 4096 7.5 -> 6.95; M = 8, N = K = 4096 5.04 -> 4.91).  One strip
  // has a group per half chunk, more strips have one per chunk or two.  A
  // one-hot row still returns fp16((q - 8) s), with its one rounding; sums of
  // several weights are rounded once instead of once per weight.  (Scaling the
  // sums only after the next operands have been read from LDS, when the
  // group's last MFMA has long finished, was no faster: 4.29, 8.2, 7.1.)
  f4 part[CS];
#pragma unroll
  for (int s = 0; s < CS; s++) part[s] = (f4){0.f, 0.f, 0.f, 0.f};

  auto compute = [&](int slot) {
    // activations of the chunk: registers -> LDS, rows as they are
#pragma unroll
    for (int i = 0; i < Sh::kALoads; i++)
      *(i4*)(stage + i * Sh::kRowsPerLoad * Sh::kStride + a_wr) = aq[slot][i];
    const h2 sub = {(half_t)1032.f, (half_t)1032.f};
    const h2 mul = {(half_t)0.0625f, (half_t)0.0625f};
    const h2 add = {(half_t)-72.f, (half_t)-72.f};
    // Each of the chunk's two weight loads holds half its k steps and is used
    // as it lands (of three loads the first two hold the first half): registers
    // -> LDS as fetched ([row][strip][Marlin lane]), then all operands of the
    // half back from LDS before the first of them is used (read one k step at
    // a time, every step would wait out a trip to LDS).
    constexpr int KH = KC / 2;
#pragma unroll
    for (int half = 0; half < 2; half++) {
#pragma unroll
      for (int i = (half == 0 ? 0 : NL - 1); i < (half == 0 ? NL - 1 : NL); i++)
        *(i4*)(stage + Sh::kWeightBase + (64 * i + lane) * 16) = bq[slot][i];
      i4 av[KH];
      int wv[KH][CS][2];
#pragma unroll
      for (int u = 0; u < KH; u++) {
        const int q = half * KH + u;
        const int* ap = (const int*)(stage + a_rd + 64 * q);
        av[u] = (i4){ap[0], ap[4], ap[8], ap[12]};
#pragma unroll
        for (int s = 0; s < CS; s++) {
          const int* wp = (const int*)(stage + Sh::kWeightBase + (2 * q * CS + s) * 128 + b_rd);
          wv[u][s][0] = wp[0];
          wv[u][s][1] = wp[32 * CS];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < KH; u++) {
        const int q = half * KH + u;
        const h8 af = __builtin_bit_cast(h8, av[u]);
#pragma unroll
        for (int s = 0; s < CS; s++) {
          const int wa = (int)((unsigned)wv[u][s][0] >> shift);
          const int wb = (int)((unsigned)wv[u][s][1] >> shift);
          h2 la = as_h2((wa & dc.lo_mask) | dc.ex) - sub;
          h2 ha = __builtin_elementwise_fma(as_h2((wa & dc.hi_mask) | dc.ex), mul, add);
          h2 lb = as_h2((wb & dc.lo_mask) | dc.ex) - sub;
          h2 hb = __builtin_elementwise_fma(as_h2((wb & dc.hi_mask) | dc.ex), mul, add);
          if constexpr (GROUP && !kScaleSums) {
            const int g = CS == 1 ? q / 4 : 0;
            const half_t sc = __builtin_bit_cast(half_t, (unsigned short)sq[slot][g * CS + s][0]);
            const h2 s2 = {sc, sc};
            la *= s2;
            ha *= s2;
            lb *= s2;
            hb *= s2;
          }
          if constexpr (kScaleSums) {
            const bool first = CS == 1 ? u == 0 : q == 0;
            const f4 from = first ? (f4){0.f, 0.f, 0.f, 0.f} : part[s];
            part[s] = __builtin_amdgcn_mfma_f32_16x16x32_f16(make_h8(la, ha, lb, hb), af, from, 0, 0, 0);
          } else {
            acc[s][q & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(make_h8(la, ha, lb, hb), af,
                                                                   acc[s][q & 1], 0, 0, 0);
          }
        }
      }
      // (a group ends with every half chunk of one strip, else with the chunk)
      if (kScaleSums && (CS == 1 || half == 1)) {
#pragma unroll
        for (int s = 0; s < CS; s++) {
          const h4 sc = __builtin_bit_cast(h4, sq[slot][(CS == 1 ? half : 0) * CS + s]);
#pragma unroll
          for (int r = 0; r < 4; r++)
            acc[s][0][r] = __builtin_fmaf((float)sc[r], part[s][r], acc[s][0][r]);
        }
      }
    }
  };

#pragma unroll
  for (int d = 0; d < DEPTH; d++) issue(d, c0 + d, c0 + d < c1);
  for (int c = c0; c < c1; c += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      if (c + d < c1) compute(d);
      issue(d, c + d + DEPTH, c + d + DEPTH < c1);
    }
  }

  // ---- sum the eight waves; wave s < CS writes strip s
  f4* red = (f4*)(smem + Sh::kReduceBase);
#pragma unroll
  for (int s = 0; s < CS; s++) red[(wave * CS + s) * 64 + lane] = acc[s][0] + acc[s][1];
  __syncthreads();
  if (wave < CS && res_strip < n_strips) {
    const int s = wave;
    f4 v = red[s * 64 + lane];
#pragma unroll
    for (int w = 1; w < kStripWaves; w++) v += red[(w * CS + s) * 64 + lane];
    const int m = row0 + nu;
    if (m < p.M) {
      half_t* crow = (half_t*)p.C + (size_t)m * p.N + res_col;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        half_t o = (half_t)v[r];
        if constexpr (!GROUP) o *= __builtin_bit_cast(half_t, chan[r]);
        crow[16 * (r >> 1) + 8 * (r & 1)] = o;
      }
    }
  }
}

template <int CS, int MR, bool GROUP>
static int configure_strip_variant() {
  constexpr int lds = StripShape<CS, MR>::kBytes;
  if (lds <= 65536) return 0;
  if (hipFuncSetAttribute((const void*)strip_kernel<CS, MR, GROUP, 1>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess ||
      hipFuncSetAttribute((const void*)strip_kernel<CS, MR, GROUP, 2>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
    return 3;
  return 0;
}
template <int CS>
static int configure_strip_width() {
  return configure_strip_variant<CS, 2, false>() | configure_strip_variant<CS, 2, true>() |
         configure_strip_variant<CS, 4, false>() | configure_strip_variant<CS, 4, true>() |
         configure_strip_variant<CS, 8, false>() | configure_strip_variant<CS, 8, true>() |
         configure_strip_variant<CS, 16, false>() | configure_strip_variant<CS, 16, true>();
}

int configure_strip_kernels() {
  return (configure_strip_width<1>() | configure_strip_width<2>() | configure_strip_width<3>() |
          configure_strip_width<4>())
             ? 3
             : 0;
}

template <int CS, int MR, bool GROUP>
static int launch_strip_variant(const GemmArgs& a, hipStream_t stream) {
  constexpr int lds = StripShape<CS, MR>::kBytes;
  const dim3 grid(ceil_div(a.N / 16, CS) * (a.row_parts > 1 ? a.row_parts : 1)),
      block(64 * kStripWaves);
  GemmArgs b = a;
  b.gpb = (int)grid.x;
  // Chunks in flight per wave: one where a wave has two at most, else two.
  // The fewer requests the compute units have outstanding, the sooner each
  // comes back: with everything requested at once M = 1, N = K = 4096 (two
  // chunks per wave) took 4.36 us against 4.28, 16 rows 6.33 against 5.80;
  // N = 4096, K = 11008 (five to six chunks per wave) 8.6 us with one chunk
  // in flight, 7.8 with two, 8.5 with three, 9.2 with four, 9.6 with six.
  const int per_wave = ceil_div(ceil_div(a.K, StripShape<CS, MR>::kChunkK), kStripWaves);
  if (per_wave <= 2)
    hipLaunchKernelGGL((strip_kernel<CS, MR, GROUP, 1>), grid, block, lds, stream, b);
  else
    hipLaunchKernelGGL((strip_kernel<CS, MR, GROUP, 2>), grid, block, lds, stream, b);
  return launch_status();
}
template <int CS, bool GROUP>
static int launch_strip_rows(const GemmArgs& a, hipStream_t stream) {
  if (a.row_parts > 1) return launch_strip_variant<CS, 16, GROUP>(a, stream);  // parts of 16 rows
  if (a.M <= 2) return launch_strip_variant<CS, 2, GROUP>(a, stream);
  if (a.M <= 4) return launch_strip_variant<CS, 4, GROUP>(a, stream);
  if (a.M <= 8) return launch_strip_variant<CS, 8, GROUP>(a, stream);
  return launch_strip_variant<CS, 16, GROUP>(a, stream);
}

// strips: 16-column strips per workgroup (1, 2 or 4 with N a multiple of
// 16*strips, or 3 with any N)
int launch_strip(const GemmArgs& a, bool group, int strips, hipStream_t stream) {
  const int parts = a.row_parts > 1 ? a.row_parts : 1;
  if (a.M > 16 * parts || a.M > kStripMaxRows || (strips != 3 && a.N % (16 * strips) != 0))
    return 2;
  switch (strips * 2 + (group ? 1 : 0)) {
    case 2: return launch_strip_rows<1, false>(a, stream);
    case 3: return launch_strip_rows<1, true>(a, stream);
    case 4: return launch_strip_rows<2, false>(a, stream);
    case 5: return launch_strip_rows<2, true>(a, stream);
    case 6: return launch_strip_rows<3, false>(a, stream);
    case 7: return launch_strip_rows<3, true>(a, stream);
    case 8: return launch_strip_rows<4, false>(a, stream);
    case 9: return launch_strip_rows<4, true>(a, stream);
  }
  return 2;
}

}  // namespace w4a16
