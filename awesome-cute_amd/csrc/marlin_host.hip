// Host launcher and C ABI of the gfx950 W4A16 Marlin GEMM.
//
// Mirrors the host side of the reference path: the argument contract and
// shape checks of marlin_cute (marlin_cute_kernel.cu:28-115) and the checks
// of the tensor binding mul (marlin_gemm.cpp:19-56).  Kernel choice, grid and
// partition are this library's own.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <vector>

#include "../../include/marlin_amd.h"
#include "../../include/marlin_amd_tools.h"
#include "scratch_pool.hpp"
#include "w4a16_common.hpp"

// Scratch for partial sums and tile counters that marlin_gemm_static uses in
// place of the pool's allocations: a fixed array in device memory, one copy per
// GPU, addressed through the pointer hipGetSymbolAddress returns for the
// current device (the name itself is not a device address in host code).
constexpr size_t kStaticPartialBytes = (size_t)32 << 20;
constexpr size_t kStaticScratchBytes = w4a16::kCounterBytes + kStaticPartialBytes;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace w4a16 {
hipError_t& last_launch_error() {
  thread_local hipError_t e = hipSuccess;
  return e;
}
}  // namespace w4a16

namespace {

using namespace w4a16;

constexpr int kMaxStreamGrid = 1024;  // workgroups of the streaming kernel
constexpr int kMaxDevices = 16;

thread_local char g_last_error[256] = "";

void set_error(hipError_t e, const char* what) {
  snprintf(g_last_error, sizeof(g_last_error), "%s: %s", what, hipGetErrorString(e));
}

struct DeviceState {
  int cus = 0;
  bool configured = false;          // kernels' LDS limits raised on this device
  unsigned char* static_scratch = nullptr;  // this device's copy of `scratch`
};
std::mutex g_mu;
DeviceState g_dev[kMaxDevices];

// What the planner may assume about the partial-sum buffer: the pool grows up
// to this much for one call; the fixed array of marlin_gemm_static is smaller.
constexpr size_t kPoolPartialLimit = (size_t)64 << 20;

// With `dev` current: raise the dynamic-LDS limit of the kernels that need it.
bool configure_device(int dev) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_dev[dev].configured) return true;
  if (configure_stream_kernels() != 0 || configure_prefill_kernels() != 0 ||
      configure_prefill_wide_kernels() != 0 || configure_strip_kernels() != 0) {
    set_error(hipGetLastError(), "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    return false;
  }
  g_dev[dev].configured = true;
  return true;
}

int device_cus(int dev) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_dev[dev].cus == 0) {
    int cus = 0;
    hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) {
      set_error(e, "hipDeviceGetAttribute");
      return -1;
    }
    g_dev[dev].cus = cus;
  }
  return g_dev[dev].cus;
}

// Shape checks in the order the reference performs them
// (marlin_cute_kernel.cu:39-60, 95-107).
int check_shape(int m, int n, int k, int groupsize, int& thread_k, int& thread_n) {
  if (thread_k == -1 || thread_n == -1) {
    if (m <= 16) {
      thread_k = 128;
      thread_n = 128;
    } else {
      thread_k = 64;
      thread_n = 256;
    }
  }
  if (thread_k <= 0 || thread_n <= 0) return MARLIN_ERR_PROB_SHAPE;
  if (groupsize == 0 || groupsize < -1) return MARLIN_ERR_KERN_SHAPE;
  const int group_blocks = groupsize == -1 ? -1 : groupsize / 16;
  if (group_blocks == 0) return MARLIN_ERR_KERN_SHAPE;
  if (m < 0 || n < 0 || k < 0) return MARLIN_ERR_PROB_SHAPE;
  if (n % thread_n != 0 || k % thread_k != 0 || (group_blocks != -1 && k % group_blocks != 0))
    return MARLIN_ERR_PROB_SHAPE;
  if (m == 0 || n == 0 || k == 0) return MARLIN_OK;
  // kernel table: tiles (128 k x 128 n) for one 16-row block, (64 k x 256 n)
  // for one to four; group size 128 or per-channel
  if (groupsize != -1 && groupsize != 128) return MARLIN_ERR_KERN_SHAPE;
  const bool small = thread_k == 128 && thread_n == 128;
  const bool wide = thread_k == 64 && thread_n == 256;
  if (!small && !wide) return MARLIN_ERR_KERN_SHAPE;
  if (small && m > 16) return MARLIN_ERR_KERN_SHAPE;
  if (groupsize == 128 && k % 128 != 0) return MARLIN_ERR_PROB_SHAPE;
  return MARLIN_OK;
}

struct Plan {
  int kernel;  // 1 streaming, 2 prefill, 3 column strips
  int grid;
  StreamPlan sp;
  int launches;
  int ksplit;            // prefill: slices of the k range per tile
  int tile_rows;         // prefill: rows of C per workgroup
  size_t partial_bytes;  // fp32 partial sums the launch exchanges through scratch (0: none)
  int row_parts;         // streaming, one-tile form: parts the rows are cut into (1: uncut)
  int part_rows;         // rows of a part (the last one has the rest)
  int strips;            // column-strip kernel: 16-column strips per workgroup (else 0)
};

constexpr int kStreamMaxRows = 64;

// Overrides of the planner for the calling thread (tests and tools; see
// marlin_amd_force_*): which kernel (0 = by cost, 1 = streaming in chunks of
// 64 rows, 2 = prefill, 3 = column strips, 4 = by cost without the column
// strips), slices of the k range per prefill tile (0 = by cost),
// rows of C per prefill workgroup (0 = by cost, 64 or 128).
struct Force {
  int kernel = 0, k_slices = 0, tile_rows = 0;
  int row_halves = 0;  // streaming kernel: 0 = by cost, 1 = never cut the rows, 2 = cut them where possible
  int strips = 0;      // column-strip kernel: 0 = by cost, or 1 to 4 strips per workgroup
};
thread_local Force t_force;

// What a plan is made for: the device's compute units, the room for partial
// sums, and the thread's overrides.
struct PlanCtx {
  int cus;
  size_t partial_limit;
  Force force;
  int counters = 16;  // ints of the workspace per column tile: min(max_par, 16)
};

// Cost in us of the prefill kernel with `tiles` tiles of tile_rows rows cut into
// s slices, fitted to measurements on MI355X.  A full-depth tile takes
// 6 + 0.0130 k with 128 rows and 5 + 0.0080 k with 64 (every unpacked weight
// then meets four row blocks instead of eight, so a 64-row tile costs more than
// half of a 128-row one) when the launch fills the CUs; k slices divide that
// and add their exchange, 3 + 2 s (128 rows: 128 KiB of partial sums per
// workgroup) or 3 + 1.5 s (64 rows).
double prefill_cost_slices(int tiles, int tile_rows, int k, int cus, int s) {
  // more workgroups than CUs run in rounds, the last of which is faster the
  // emptier it is: half way between whole rounds and the plain ratio fits
  // (N = K = 4096, M = 3072: 384 tiles of 128 rows, 102.7 us, where one round
  // of 256 takes 59.3)
  const double ratio = (double)tiles * s / cus;
  const double rounds = ratio <= 1.0 ? 1.0 : 0.5 * (ceil_div(tiles * s, cus) + ratio);
  // ... and a launch that leaves CUs idle runs its tiles faster (clock, and
  // fewer workgroups at the memory): 0.9 of the time at three quarters full
  const double fill = ratio < 1.0 ? 0.6 + 0.4 * ratio : 1.0;
  const double tile = (tile_rows == 64 ? 5.0 + 0.0080 * k : 6.0 + 0.0130 * k) * fill;
  const double exchange = s > 1 ? 3.0 + (tile_rows == 64 ? 1.5 : 2.0) * s : 0.0;
  return rounds * (tile / s + exchange);
}

// Slices of the k range per tile: the cheapest count among those that keep
// the launch within one workgroup per CU, slices at least 256 deep (two
// 64-deep stages for each half of the workgroup), and the partial sums and
// tile counters within the scratch.  Up to eight; in practice four, six where
// k is deep (N = 4096, K = 11008, M = 128: 24.8 us with six against 26.9 with
// four).
int prefill_k_slices(int tiles, int tile_rows, int k, const PlanCtx& cx) {
  int most = k / 256;
  if (most > 8) most = 8;
  while (most > 1 && (size_t)tiles * most * tile_rows * 256 * 4 > cx.partial_limit) --most;
  if (most < 1 || tiles > kMaxCounters) return 1;
  if (cx.force.k_slices > 0) return cx.force.k_slices < most ? cx.force.k_slices : most;
  if (most > cx.cus / tiles) most = cx.cus / tiles;
  int best = 1;
  double best_cost = prefill_cost_slices(tiles, tile_rows, k, cx.cus, 1);
  for (int s = 2; s <= most; s++) {
    const double c = prefill_cost_slices(tiles, tile_rows, k, cx.cus, s);
    if (c < best_cost) {
      best = s;
      best_cost = c;
    }
  }
  return best;
}

// Either kernel can do any problem whose n is a multiple of 256: the prefill
// kernel once, or the streaming kernel once per 64 rows, reading the weights
// again every time.
double prefill_cost_rows(int m, int n, int k, const PlanCtx& cx, int tile_rows) {
  const int tiles = ceil_div(m, tile_rows) * (n / 256);
  return prefill_cost_slices(tiles, tile_rows, k, cx.cus,
                             prefill_k_slices(tiles, tile_rows, k, cx));
}

// Rows of C per prefill workgroup.  64-row tiles are twice as many, so they
// need fewer k slices to fill the CUs (or none), which wins while the problem
// is small: at N = K = 4096 up to about 512 rows (M = 128: 16.0 against
// 21.9 us), at N = 4096, K = 11008 up to 256 (27.5 against 38.9 us at M = 128).
int prefill_tile_rows(int m, int n, int k, const PlanCtx& cx) {
  if (cx.force.tile_rows == 64 || cx.force.tile_rows == 128) return cx.force.tile_rows;
  if (m <= 64) return 64;
  return prefill_cost_rows(m, n, k, cx, 64) < prefill_cost_rows(m, n, k, cx, 128) ? 64 : 128;
}

double prefill_cost(int m, int n, int k, const PlanCtx& cx) {
  // (the tile fits were made at K >= 4096: at K <= 1024 the prefill kernels
  // measure a third more, 56 and 64 rows at every N from 256 to 11008)
  return prefill_cost_rows(m, n, k, cx, prefill_tile_rows(m, n, k, cx)) * (k < 2048 ? 1.33 : 1.0);
}

// The streaming kernel's split of the granule sequence over the compute units
// for `mb` row blocks.  Measured on MI355X: a split that keeps every workgroup
// inside one column tile (or gives it whole tiles) costs about 0.1 us x row
// blocks per granule of the longest workgroup; a split that leaves workgroups
// straddling tile boundaries is several us slower (a second exchange per
// workgroup, and workgroups that read different weight rows at the same
// time), about 1 + 2.5 x row blocks us.  Candidates: every tile cut into c
// nearly equal runs (c tiles' worth of workgroups <= CUs), whole tiles per
// workgroup, and the evenly balanced uniform split.
struct StreamSplit {
  int gpb;        // granules of the longest workgroup
  int wpt;        // workgroups per column tile, or 0 for the uniform form
  bool straddle;  // workgroups cross tile boundaries
};
// The last arrival of a tile fetches its sharers eight at a time: beyond 8
// every sharer costs (M = 16, N = 2048, K = 4096: 8 runs per tile 6.1 us, 16
// 6.7, 32 10.7; N = 1024, K = 8192: 8 7.9, 16 7.1, 32 8.9)
double sharer_cost(int c) { return c <= 8 ? 0.0 : c <= 16 ? 0.1 * (c - 8) : 0.8 + 0.25 * (c - 16); }

StreamSplit choose_stream_split(int mb, int n, int k, int cus) {
  const int NT = n / kTileN;
  const int KG = k / kGranuleK;
  const int total = NT * KG;
  if (cus > kMaxStreamGrid) cus = kMaxStreamGrid;  // the grid the kernel's slots allow
  const double per_granule = 0.1 * mb, straddle = 1.0 + 2.5 * mb;
  StreamSplit sp;
  sp.gpb = ceil_div(total, cus);
  sp.wpt = 0;
  sp.straddle = !(sp.gpb % KG == 0 || KG % sp.gpb == 0);
  auto sharers = sharer_cost;
  double best_cost = per_granule * sp.gpb + (sp.straddle ? straddle : 0.0) +
                     sharers(ceil_div(KG, sp.gpb));
  for (int c = 1; c <= KG && NT * c <= cus; c++) {
    const int g = ceil_div(KG, c);
    const double cost = per_granule * g + sharers(c);
    if (cost < best_cost + 1e-9) {  // on a tie the one-tile form: its kernel is leaner
      sp.gpb = g;
      sp.wpt = c;
      sp.straddle = false;
      best_cost = cost;
    }
  }
  for (int mult = 2; mult * KG <= total; mult++) {
    const int g = mult * KG;
    if (ceil_div(total, g) > cus) continue;  // more workgroups than CUs never paid off
    const double cost = per_granule * g;
    if (cost < best_cost - 1e-9) {
      sp.gpb = g;
      sp.wpt = 0;
      sp.straddle = false;
      best_cost = cost;
    }
  }
  return sp;
}

// What cutting the rows of a streaming launch in two saves (us; negative: a
// loss), fitted on MI355X over N = 2048...11008, K = 4096...13824, 17 to 64
// rows.  The halves have half the row blocks to sum, store and read back and
// half the sharers per tile, which is worth S; their runs are twice as long,
// and a granule of one or two row blocks costs more than half a granule of two
// to four, which costs p per granule of the uncut run.  S jumps where the last
// arrival of the uncut launch would fetch its sharers in more than one round
// (more than 8).  E.g. M = 64, N = K = 4096 (8 sharers, 8 granules): 12.9 ->
// 10.2 us; N = 2048: 14.9 -> 8.5; 8192 x 8192 (4 sharers, 32 granules): 20.0
// -> 19.5; M = 48 there 17.1 -> 19.1 (not cut).
double halves_gain(int rows, int wpt, int gpb) {
  const int mb = ceil_div(rows, 16);
  const bool rounds = wpt > 8;
  const double p = 0.06;
  double s;
  if (mb <= 2)
    s = rounds ? 2.8 : 1.0 + 0.045 * (rows - 16);
  else if (mb == 3)
    s = rounds ? 4.0 : 1.0 + 0.027 * (rows - 33);
  else
    s = rounds ? 6.5 : 3.2;
  return s - p * gpb;
}

// Fitted time (us) of the streaming kernel with uncut rows: a pass over 49-64
// rows takes 11.3 + 0.28 per granule of the longest workgroup (N=K=4096: 8
// granules, 12.9; N=8192, K=4096: 16, 15.5; N=4096, K=11008: 22, 18.0;
// N=11008, K=4096 or 8192^2: 32, 18.5-20; N=28672, K=8192: 128, 46), fewer
// rows a share of that, up to 16 rows 4.9 + 0.17 per granule (1.4 less where
// no tile is shared: N=28672, K=8192, 128 granules, 23 us); every launch
// after the first waits a microsecond for the one before (65 rows at N=4096,
// K=11008: 18.0 + 9.0 alone, 27.0 in a row).
double stream_cost(int m, int n, int k, int cus) {
  const StreamSplit s4 = choose_stream_split(4, n, k, cus);
  const double full = 11.3 + 0.28 * s4.gpb + (s4.straddle ? 11.0 : 0.0);
  const int tail = m % kStreamMaxRows;
  double t = (m / kStreamMaxRows) * full;
  if (tail > 16) {
    t += full * (tail > 48 ? 1.0 : tail > 32 ? 0.9 : 0.65);
  } else if (tail > 0) {
    const StreamSplit s1 = choose_stream_split(1, n, k, cus);
    // (refitted over M = 1, 4, 8, 16 on N = 256...28672, K = 512...11008, 6 %
    // rms: a workgroup that shares its tiles with no other exchanges nothing)
    const int sharers = s1.wpt > 0 ? s1.wpt : ceil_div(k / kGranuleK, s1.gpb);
    t += 4.94 + 0.167 * s1.gpb + (tail > 8 ? 0.23 : 0.0) + (s1.straddle ? 3.5 : 0.0) +
         (sharers == 1 && !s1.straddle ? -1.39 : sharer_cost(sharers));
  }
  return t + 1.0 * (ceil_div(m, kStreamMaxRows) - 1);
}

// More than 64 rows in one streaming launch: the rows cut into parts of 32,
// every (tile, part) a problem of its own for wpt workgroups.  Possible while
// there is a CU per (tile, part) and a counter per part; costs what a 32-row
// launch of that split costs (0.65 of the fit above; measured 12.6 us against
// 13.2 for M = 128 at N = K = 4096, 22.9 / 23.0 at K = 11008, 17.1 / 17.0 for
// M = 256 with one workgroup per tile and part).  Sets wpt
// and the granules per run; returns the cost in us, or a negative number where
// it cannot be done.
double stream_parts_cost(int m, int n, int k, const PlanCtx& cx, int* parts, int* wpt, int* gpb) {
  const int NT = n / kTileN, KG = k / kGranuleK;
  const int P = ceil_div(m, 32);
  if (m <= kStreamMaxRows || P > cx.counters || NT * P > cx.cus || cx.force.row_halves == 1)
    return -1.0;
  int w = cx.cus / (NT * P);
  if (w > KG) w = KG;
  // more than 8 sharers would be fetched in two rounds by the last arrival
  if (w > 8) w = 8;
  *parts = P;
  *wpt = w;
  *gpb = ceil_div(KG, w);
  // (a launch that exchanges nothing saves the 2 us the fit holds for that)
  return 0.65 * (11.3 + 0.28 * *gpb) - (w == 1 ? 2.0 : 0.0);
}

// The streaming kernel's cost as make_plan would launch it: with the rows cut
// in two or into parts of 32 where that is cheaper.
double stream_cost_as_planned(int m, int n, int k, const PlanCtx& cx) {
  double stream = stream_cost(m, n, k, cx.cus);
  if (m <= kStreamMaxRows && cx.force.row_halves != 1 && cx.counters >= 2) {
    // what the launch gains where make_plan cuts its rows in two
    const StreamSplit split = choose_stream_split(ceil_div(m, 16), n, k, cx.cus);
    const int half = 16 * ceil_div(ceil_div(m, 2), 16);
    const StreamSplit hs = choose_stream_split(half / 16, 2 * n, k, cx.cus);
    const double gain = split.wpt >= 2 && hs.wpt >= 1 && half < m
                            ? halves_gain(m, 2 * hs.wpt, ceil_div(k / kGranuleK, 2 * hs.wpt))
                            : 0.0;
    if (gain > 0.25) {
      // (the halves take no less than a launch of half the rows over twice the
      // tiles: the gain was fitted where the uncut launch fetches its sharers
      // in rounds, which the fit of the uncut launch does not hold -- M = 64,
      // N = 2048, K = 4096: 12.1 - 6.3 by the fits, 8.7 us measured, 8.1 by this)
      const double alone = stream_cost(half, 2 * n, k, cx.cus);
      stream = stream - gain > alone ? stream - gain : alone;
    }
    // 17 to 64 rows over short, wide weights: tiles of at most 16 granules that
    // two to four workgroups share finish in three quarters of the fit's time
    // (K = 512 and 1024 at N = 4096...28672: 0.6 to 0.9 of it; N <= 2048, more
    // sharers per tile: 1.05 to 1.4)
    if (m > 16 && k < 2048 && n >= 4096) stream *= 0.75;
  }
  int parts, wpt, gpb;
  const double cut = stream_parts_cost(m, n, k, cx, &parts, &wpt, &gpb);
  if (cut > 0.0 && cut < stream) stream = cut;
  return stream;
}

bool prefer_prefill(int m, int n, int k, const PlanCtx& cx) {
  // no measurement favours 64-row prefill tiles below four row blocks
  if (m <= 48) return false;
  // ... nor, up to 64 rows, over weights that are neither wide nor deep: 56 and
  // 64 rows at N = 256...11008 with K = 512...4096 stream in 0.6 to 0.95 of
  // the prefill kernel's time (N = 28672: 1.07 to 1.1 at every K; N = 11008:
  // 1.1 at K = 8192, 1.5 at 11008), which the two fits, 15 % apart there in
  // opposite directions, do not resolve
  if (m <= kStreamMaxRows && n < 16384 && k < 8192) return false;
  return prefill_cost(m, n, k, cx) <= stream_cost_as_planned(m, n, k, cx);
}

// Fitted time (us) of the column-strip kernel with `cs` strips per workgroup.
// Up to 16 rows a launch costs 2.7 us.  A workgroup takes in its 8 cs k bytes
// of weights at about 23 GB/s, what its eight waves unpack and multiply, and
// workgroups beyond one per compute unit queue up behind each other, 0.3 us
// each; all together they draw 4.8 TB/s from memory at most.  Every workgroup
// also reads all rows of activations, which a compute unit takes from the L2s
// at about 87 GB/s.  Measured (M = 1, one strip): N = K = 2048 3.2 us, 4096 x
// 4096 4.3, N = 11008, K = 4096 7.8, N = 1024, K = 8192 5.5, N = 4096, K =
// 11008 7.5, 8192 x 8192 10.4 (two strips 9.1), N = 13824, K = 5120 11.4 (four
// strips 10.0); M = 16: 4096 x 4096 5.8, N = 11008, K = 4096 15.0 (four strips
// 9.4), N = 4096, K = 11008 11.8.
// More rows are cut into parts of 16, a workgroup per strip set and part, and
// fitted on their own: 1.8 us, and per round of workgroups over the compute
// units 1.27 us, the weights at 32.7 GB/s and the part's 16 rows at 67.8 GB/s,
// a quarter of which later rounds hide behind the one before.  Measured: M =
// 32, N = K = 1024 3.9 us, 2048 x 2048 4.6, 4096 x 4096 7.6; M = 64: N = 512,
// K = 1024 3.6, N = 2048, K = 4096 7.7, 4096 x 4096 9.7; M = 128: N = 256, K =
// 512 3.4, 2048 x 2048 6.8; M = 512: N = 256, K = 1024 3.7; M = 1024: N =
// 256, K = 512 3.8.
double strip_cost(int m, int n, int k, int cs, int cus) {
  // a wave's chunk is 256 / cs k-values (128 with three strips): a k range of
  // fewer than eight chunks leaves waves idle (K = 1024: one strip 0.2 to 0.3
  // us behind two at every N from 8 rows on; fewer rows are no slower for it)
  const int chunks = ceil_div(k, cs == 3 ? 128 : 256 / cs);
  const double idle = m >= 8 && chunks < 8 ? 0.7 * (1.0 - chunks / 8.0) : 0.0;
  if (m > 16) {
    // rows in parts of 16, a workgroup each: fitted to 17...128 rows over N =
    // 256...28672, K = 512...11008 (8 % rms where the strips are within 1.6
    // times the other kernels' time)
    const int wgs = ceil_div(n / 16, cs) * ceil_div(m, 16);
    const int rounds = ceil_div(wgs, cus);
    const double per_wg = 1.27 + 8.0 * cs * k / 32.7e3 + 32.0 * k / 67.8e3;
    const double by_cu = rounds * per_wg * (1.0 - 0.24 * (1.0 - 1.0 / rounds));
    const double by_memory = 0.5 * k * n / 4.8e6;
    return 1.8 + (by_cu > by_memory ? by_cu : by_memory) + idle;
  }
  // Up to 8 rows the group scales go to the sums, not to the weights, and the
  // constants are fitted on their own (M = 1, 4, 8: 7 % rms): the launch, the
  // rate a compute unit unpacks at, the rate it reads rows at, a queued
  // workgroup, and memory -- 5.85 TB/s while every round of workgroups fills
  // the compute units.
  const bool few = m <= 8;
  const int wgs = ceil_div(n / 16, cs);
  const int per_cu = ceil_div(wgs, cus);
  const double last_round = wgs > cus ? (double)wgs / (per_cu * cus) : 1.0;
  const double by_cu = per_cu * 8.0 * cs * k / (few ? 28.0e3 : 23e3);
  const double by_memory = 0.5 * k * n / (few ? 5.85e6 * last_round : 4.8e6);
  // (with 172 of 256 compute units reading 16 rows the rows came in a third
  // sooner than this: N = 11008, K = 4096 with four strips)
  const double rows =
      per_cu * 2.0 * m * k / (few ? 72.5e3 : 87e3) * (wgs < cus ? (0.5 + 0.5 * wgs / cus) : 1.0);
  // (a little of by_cu always: it decides between widths that memory bounds alike)
  return (few ? 2.88 : 2.7) + (by_cu > by_memory ? by_cu : by_memory) + rows +
         (few ? 0.43 : 0.3) * (per_cu - 1) + 0.02 * by_cu + idle;
}

// 16-column strips per workgroup of the column-strip kernel: the cheapest of
// 1, 2 and 4 where they divide n's strips, and for up to 16 rows of 3, which
// leaves the last workgroup with fewer (N = 11008, K = 4096, 230 workgroups
// of three strips against 172 of four: M = 16 9.2 against 9.3 us, M = 8 8.2 /
// 8.5, M = 1 7.5 / 7.7 with one strip; K = 8192: M = 1 12.3 against 13.6, M =
// 4 11.7 / 13.6, M = 16 14.4 / 15.2; N = 5120, K = 5120: 10.3 against 8.4 with
// two)
// (0 where the planner's own rules leave none; a forced launch takes any)
int strips_per_workgroup(int m, int n, int k, const PlanCtx& cx) {
  const bool forced = cx.force.kernel == 3 || cx.force.strips != 0;
  int best = 0;
  double best_cost = 0.0;
  for (int cs = 1; cs <= 4; cs++) {
    // (three strips: not over k ranges of a chunk or two per wave, where their
    // three loads per chunk cost 8 % against two or four strips)
    if (cs == 3 ? ((m > 16 || k < 1024) && !forced) : n % (16 * cs) != 0) continue;
    // Rows in parts: at most two workgroups per compute unit (with three and
    // more the streaming kernel was 1.1 to 1.6 times faster wherever the fits,
    // its own 20 to 40 % high over short k ranges, promised otherwise: 48 rows
    // at N = 28672, K = 512 11.8 against 7.3 us, 64 rows at N = 11008, K = 2048
    // 13.5 against 11.2)
    if (m > 16 && !forced && ceil_div(n / 16, cs) * ceil_div(m, 16) > 2 * cx.cus) continue;
    if (cx.force.strips != 0 && cx.force.strips != cs && best != 0) continue;
    const double c = strip_cost(m, n, k, cs, cx.cus);
    if (best == 0 || cx.force.strips == cs || c < best_cost) {
      best = cs;
      best_cost = c;
      if (cx.force.strips == cs) break;
    }
  }
  return best;
}

// The column-strip kernel against the other two: the streaming kernel reaches
// more of the memory's bandwidth (its workgroups share a column tile's k
// range, so every compute unit has work whatever n is), the strips pay nothing
// for the exchange between workgroups -- 2 us of a launch that takes 6.  The
// strips win while the weights are a few MiB per launch (M = 1: 4096 x 4096
// 4.3 against 6.3 us, N = 11008, K = 4096 8.5 against 9.7, N = 4096, K = 11008
// 7.5 against 9.1, 8192 x 8192 9.1 against 10.4, N = 28672, K = 8192 27.6
// against 23.9 -- there no more; M = 16: 4096 x 4096 5.8 against 6.6, N =
// 11008, K = 4096 9.4 against 9.9, N = 4096, K = 11008 11.8 against 9.6), and
// with more rows, in parts, while the parts fill the compute units at most
// twice (M = 32: N = K = 1024 3.9 against 5.6, 4096 x 4096 7.6 against 8.5, N =
// 8192, K = 4096 9.5 against 10.3, N = 4096, K = 8192 11.0 against 10.7; M =
// 64: N = 512, K = 1024 3.6 against 6.9, N = 2048, K = 4096 7.7 against 8.7,
// 4096 x 4096 9.7 against 10.5, N = 8192, K = 4096 15.0 against 13.3; M =
// 128: N = 256, K = 512 3.4 against 7.0, 2048 x 2048 6.8 against 8.1, 4096 x
// 4096 14.6 against 12.9; M = 1024: N = 256, K = 512 3.8 against 7.7, N = 512,
// K = 1024 6.6 against 11.4).
bool prefer_strips(int m, int n, int k, const PlanCtx& cx) {
  const int cs = strips_per_workgroup(m, n, k, cx);
  // (beyond one row block the fits are looser, the streaming kernel's above all
  // over short k ranges: the strips have to win by a margin)
  if (cs == 0) return false;
  const double strips = strip_cost(m, n, k, cs, cx.cus) * (m > 16 ? 1.05 : 1.0);
  if (strips >= stream_cost_as_planned(m, n, k, cx)) return false;
  return !(n % 256 == 0 && m > 48 && prefill_cost(m, n, k, cx) <= strips);
}

Plan make_plan(int m, int n, int k, int sms, const PlanCtx& cx) {
  Plan pl;
  // (the column-strip kernel does at most kStripMaxRows rows and takes no
  // hint: forced onto anything else it leaves the choice to the costs)
  const int force = cx.force.kernel == 3 && (m > kStripMaxRows || sms > 0) ? 0 : cx.force.kernel;
  // the prefill kernel's tiles are 256 columns wide (n is a multiple of 256
  // whenever m > 16, by the shape contract)
  const bool by_cost = force == 0 || force == 4;
  const bool prefill = n % 256 == 0 && (force == 2 || (by_cost && prefer_prefill(m, n, k, cx)));
  pl.ksplit = 1;
  pl.tile_rows = 0;
  pl.partial_bytes = 0;
  pl.row_parts = 1;
  pl.part_rows = 0;
  pl.strips = 0;
  if (m <= kStripMaxRows && sms <= 0 &&
      (force == 3 || (force == 0 && prefer_strips(m, n, k, cx)))) {
    pl.kernel = 3;
    pl.strips = strips_per_workgroup(m, n, k, cx);
    if (m > 16) {
      pl.row_parts = ceil_div(m, 16);
      pl.part_rows = 16;
    }
    pl.grid = ceil_div(n / 16, pl.strips) * pl.row_parts;
    pl.sp = make_stream_plan(n, k, 1);
    pl.launches = 1;
    return pl;
  }
  if (prefill) {
    // one workgroup per (tile of C, slice of k)
    pl.kernel = 2;
    pl.tile_rows = prefill_tile_rows(m, n, k, cx);
      const int tiles = ceil_div(m, pl.tile_rows) * (n / 256);
    pl.ksplit = prefill_k_slices(tiles, pl.tile_rows, k, cx);
    pl.grid = tiles * pl.ksplit;
    pl.sp = make_stream_plan(n, k, 1);
    pl.launches = 1;
    if (pl.ksplit > 1) pl.partial_bytes = (size_t)pl.grid * pl.tile_rows * 256 * 4;
    return pl;
  }
  pl.kernel = 1;
  const int rows = m < kStreamMaxRows ? m : kStreamMaxRows;
  const int mb = ceil_div(rows, 16);
  {
    // more than 64 rows: one launch with the rows cut into parts of 32 where
    // that is cheaper than a launch per 64 rows
    int parts = 0, wpt = 0, gpb = 0;
    const double cut = sms > 0 ? -1.0 : stream_parts_cost(m, n, k, cx, &parts, &wpt, &gpb);
    if (cut > 0.0 && (cx.force.row_halves == 2 || cut < stream_cost(m, n, k, cx.cus))) {
      pl.sp.NT = n / kTileN;
      pl.sp.KG = k / kGranuleK;
      pl.sp.gpb = gpb;
      pl.sp.wpt = wpt;
      pl.sp.grid = pl.sp.NT * parts * wpt;
      pl.row_parts = parts;
      pl.part_rows = 32;
      pl.grid = pl.sp.grid;
      pl.launches = 1;
      if (wpt > 1) pl.partial_bytes = (size_t)stream_slots(pl.sp) * stream_slot_bytes(2);
      return pl;
    }
  }
  if (sms > 0) {
    pl.sp = make_stream_plan(n, k, sms > kMaxStreamGrid ? kMaxStreamGrid : sms);
  } else {
    const StreamSplit split = choose_stream_split(mb, n, k, cx.cus);
    pl.sp.NT = n / kTileN;
    pl.sp.KG = k / kGranuleK;
    pl.sp.gpb = split.gpb;
    pl.sp.wpt = split.wpt;
    pl.sp.grid = split.wpt > 0 ? pl.sp.NT * split.wpt : ceil_div(pl.sp.NT * pl.sp.KG, split.gpb);
    // Many rows and many workgroups per tile: cut the rows in two instead of
    // the k range once more.  Each half is finished by half as many sharers,
    // with half the rows to sum, store and read back.
    const int half = 16 * ceil_div(ceil_div(rows, 2), 16);
    // the halves' own split: twice the tiles, half the row blocks
    const StreamSplit hs = choose_stream_split(half / 16, 2 * n, k, cx.cus);
    const bool can = m <= kStreamMaxRows && half < rows && split.wpt >= 2 && hs.wpt >= 1 &&
                     cx.counters >= 2;
    const bool want =
        can && (cx.force.row_halves == 2 ||
                (cx.force.row_halves == 0 &&
                 halves_gain(rows, 2 * hs.wpt, ceil_div(pl.sp.KG, 2 * hs.wpt)) > 0.25));
    if (want) {
      pl.row_parts = 2;
      pl.part_rows = half;
      pl.sp.wpt = hs.wpt;
      pl.sp.gpb = ceil_div(pl.sp.KG, pl.sp.wpt);
      pl.sp.grid = pl.sp.NT * 2 * pl.sp.wpt;
    }
  }
  pl.grid = pl.sp.grid;
  pl.launches = ceil_div(m, kStreamMaxRows);
  // column tiles that several workgroups share are finished through one
  // partial-sum slot per workgroup (cut tiles) or two (runs that may start and
  // end inside a tile)
  const bool shared = pl.sp.wpt > 0 ? pl.sp.wpt > 1 : pl.sp.gpb % pl.sp.KG != 0;
  if (shared)
    pl.partial_bytes = (size_t)stream_slots(pl.sp) *
                       stream_slot_bytes(pl.row_parts > 1 ? pl.part_rows / 16 : mb);
  return pl;
}

// Enqueue the launches of plan pl with the scratch of `view` (null pointers
// when the plan exchanges nothing through scratch).
int enqueue(const Plan& pl, const ScratchView& view, const void* A, const void* B, void* C,
            const void* s, int m, int n, int k, void* workspace, int groupsize, int max_par,
            hipStream_t stream) {
  // the caller's workspace holds at least n/128 * max_par zero ints
  // (reference marlin_gemm.cpp:29-31, marlin_cute_kernel.cu:68); one counter
  // per column tile is used (two where the rows are cut in halves: the plan
  // only does that when max_par >= 2), and the counters are spread max_par
  // ints apart (64 bytes at the launcher's default of 16)
  const int lock_stride = max_par > 16 ? 16 : max_par;
  (void)hipGetLastError();  // an earlier call's error is not this launch's
  int rc = MARLIN_OK;
  if (pl.kernel == 3) {
    GemmArgs a;
    const int strip_parts = pl.row_parts;
    a.A = A;
    a.B = B;
    a.C = C;
    a.S = s;
    a.M = m;
    a.N = n;
    a.K = k;
    a.locks = nullptr;
    a.lock_stride = 1;
    a.scratch = nullptr;
    a.gpb = 0;
    a.wpt = 0;
    a.row_parts = strip_parts;
    a.part_rows = strip_parts > 1 ? 16 : 0;
    rc = launch_strip(a, groupsize != -1, pl.strips, stream);
  } else if (pl.kernel == 2) {
    GemmArgs a;
    a.A = A;
    a.B = B;
    a.C = C;
    a.S = s;
    a.M = m;
    a.N = n;
    a.K = k;
    a.locks = view.counters;
    a.lock_stride = 1;
    a.scratch = view.partials;
    a.gpb = 0;
    a.wpt = 0;
    a.row_parts = 1;
    a.part_rows = 0;
    // 128-row tiles: four waves with 128 x 128 accumulators; 64-row tiles: eight
    // waves with 64 x 64
    rc = pl.tile_rows == 128 ? launch_prefill_wide(a, groupsize != -1, pl.ksplit, stream)
                             : launch_prefill(a, groupsize != -1, pl.ksplit, stream);
  } else {
    // a launch per 64 rows, or one launch over all rows cut into parts
    const int rows_per_launch = pl.launches == 1 ? m : kStreamMaxRows;
    for (int m0 = 0; m0 < m && rc == MARLIN_OK; m0 += rows_per_launch) {
      GemmArgs a;
      a.A = (const char*)A + (size_t)m0 * k * 2;
      a.B = B;
      a.C = (char*)C + (size_t)m0 * n * 2;
      a.S = s;
      a.M = m - m0 < rows_per_launch ? m - m0 : rows_per_launch;
      a.N = n;
      a.K = k;
      a.locks = (int*)workspace;
      a.lock_stride = lock_stride;
      a.scratch = view.partials;
      a.gpb = pl.sp.gpb;
      a.wpt = pl.sp.wpt;
      a.row_parts = pl.row_parts;
      a.part_rows = pl.part_rows;
      rc = launch_stream(a, groupsize != -1, pl.grid, stream);
    }
  }
  if (rc == MARLIN_ERR_RUNTIME) set_error(w4a16::last_launch_error(), "kernel launch");
  return rc;
}

// With `dev` current: this device's copy of the fixed scratch array.  Its
// counters need no clearing: the array is zero when the module is loaded and
// every launch hands its counters back zeroed.  (A clearing kernel on the first
// caller's stream could land in the middle of another stream's first launch.)
unsigned char* static_scratch_for(int dev) {
  std::lock_guard<std::mutex> lk(g_mu);
  DeviceState& d = g_dev[dev];
  if (d.static_scratch) return d.static_scratch;
  void* ptr = nullptr;
  hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) {
    set_error(e, "hipGetSymbolAddress(scratch)");
    return nullptr;
  }
  d.static_scratch = (unsigned char*)ptr;
  return d.static_scratch;
}

// use_static: marlin_gemm_static -- the fixed array instead of the pool, a
// plan made for its size, and no allocation on any path.
int run(const void* A, const void* B, void* C, const void* s, int m, int n, int k,
        void* workspace, int groupsize, int dev, hipStream_t stream, int thread_k, int thread_n,
        int sms, int max_par, bool use_static) {
  int rc = check_shape(m, n, k, groupsize, thread_k, thread_n);
  if (rc != MARLIN_OK || m == 0 || n == 0 || k == 0) return rc;
  if (max_par < 1) {
    // the tile counters live in the caller's workspace, max_par ints apart
    snprintf(g_last_error, sizeof(g_last_error), "max_par = %d: must be at least 1", max_par);
    return MARLIN_ERR_WORKSPACE;
  }
  // the kernels address A, B and C with 32-bit byte offsets
  const long long lim = 0x7fffffffLL;
  if ((long long)k * n / 2 > lim || (long long)m * k * 2 > lim || (long long)m * n * 2 > lim) {
    snprintf(g_last_error, sizeof(g_last_error),
             "operand of more than 2 GiB (m=%d n=%d k=%d): split the call", m, n, k);
    return MARLIN_ERR_RUNTIME;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    snprintf(g_last_error, sizeof(g_last_error), "device index %d out of range", dev);
    return MARLIN_ERR_RUNTIME;
  }
  int prev = -1;
  hipError_t e = hipGetDevice(&prev);
  if (e != hipSuccess) {
    set_error(e, "hipGetDevice");
    return MARLIN_ERR_RUNTIME;
  }
  if (prev != dev && (e = hipSetDevice(dev)) != hipSuccess) {
    set_error(e, "hipSetDevice");
    return MARLIN_ERR_RUNTIME;
  }
  const int cus = device_cus(dev);
  rc = MARLIN_ERR_RUNTIME;
  if (cus > 0 && configure_device(dev)) {
    PlanCtx cx = {cus, use_static ? kStaticPartialBytes : kPoolPartialLimit, t_force};
    cx.counters = max_par > 16 ? 16 : max_par;  // the counters of a tile sit that many ints apart
    const Plan pl = make_plan(m, n, k, sms, cx);
    ScratchView view = {nullptr, nullptr};
    bool ok = true;
    if (use_static) {
      if (pl.partial_bytes > kStaticPartialBytes) {
        snprintf(g_last_error, sizeof(g_last_error),
                 "marlin_gemm_static: this call (m=%d n=%d k=%d sms=%d) needs %zu bytes of "
                 "partial sums, the fixed scratch holds %zu: use marlin_gemm",
                 m, n, k, sms, pl.partial_bytes, kStaticPartialBytes);
        ok = false;
      } else if (pl.partial_bytes > 0) {
        unsigned char* base = static_scratch_for(dev);
        ok = base != nullptr;
        if (ok) {
          view.counters = (int*)base;
          view.partials = (float*)(base + kCounterBytes);
        }
      }
    } else if (pl.partial_bytes > 0) {
      ok = scratch_acquire(dev, stream, pl.partial_bytes, &view, g_last_error,
                           sizeof(g_last_error));
    }
    if (ok)
      rc = enqueue(pl, view, A, B, C, s, m, n, k, workspace, groupsize, max_par, stream);
  }
  if (prev != dev) (void)hipSetDevice(prev);
  return rc;
}

}  // namespace

extern "C" {

int marlin_gemm(const void* A, const void* B, void* C, const void* s, int prob_m, int prob_n,
                int prob_k, void* workspace, int groupsize, int dev, void* stream, int thread_k,
                int thread_n, int sms, int max_par) {
  return run(A, B, C, s, prob_m, prob_n, prob_k, workspace, groupsize, dev, (hipStream_t)stream,
             thread_k, thread_n, sms, max_par, false);
}

int marlin_cute(const void* A, const void* B, void* C, void* s, int prob_m, int prob_n,
                int prob_k, void* workspace, int groupsize, int dev, void* stream, int thread_k,
                int thread_n, int sms, int max_par) {
  return marlin_gemm(A, B, C, s, prob_m, prob_n, prob_k, workspace, groupsize, dev, stream,
                     thread_k, thread_n, sms, max_par);
}

int marlin_official(const void* A, const void* B, void* C, void* s, int prob_m, int prob_n,
                    int prob_k, void* workspace, int groupsize, int dev, void* stream,
                    int thread_k, int thread_n, int sms, int max_par) {
  return marlin_gemm(A, B, C, s, prob_m, prob_n, prob_k, workspace, groupsize, dev, stream,
                     thread_k, thread_n, sms, max_par);
}

int marlin_gemm_static(const void* A, const void* B, void* C, const void* s, int prob_m,
                       int prob_n, int prob_k, void* workspace, int groupsize, int dev,
                       void* stream, int thread_k, int thread_n, int sms, int max_par) {
  return run(A, B, C, s, prob_m, prob_n, prob_k, workspace, groupsize, dev, (hipStream_t)stream,
             thread_k, thread_n, sms, max_par, true);
}

long long marlin_gemm_static_capacity(void) { return (long long)kStaticPartialBytes; }

int marlin_mul(const void* A, const void* B, void* C, const void* s, int prob_m, int prob_n,
               int prob_k, int s_rows, void* workspace, long long workspace_numel, int dev,
               void* stream, int thread_k, int thread_n, int sms, int max_par, int cute_version,
               char* err, int err_len) {
  (void)cute_version;  // one implementation serves both reference variants
  auto fail = [&](int code, const char* fmt, auto... args) {
    if (err && err_len > 0) snprintf(err, (size_t)err_len, fmt, args...);
    return code;
  };
  if (err && err_len > 0) err[0] = 0;
  if (s_rows <= 0) return fail(MARLIN_ERR_GROUPS, "k=%d not compatible with %d groups.", prob_k, s_rows);
  int groupsize = s_rows == 1 ? -1 : prob_k / s_rows;
  if (groupsize != -1 && groupsize * s_rows != prob_k)
    return fail(MARLIN_ERR_GROUPS, "k=%d not compatible with %d groups.", prob_k, s_rows);
  // (the reference's comparison, marlin_gemm.cpp:29-31, lets any workspace pass
  // when max_par < 1; the tile counters need at least one int per tile)
  const int par = max_par < 1 ? 1 : max_par;
  if (workspace_numel < (long long)(prob_n / 128) * par)
    return fail(MARLIN_ERR_WORKSPACE, "workspace must be of size at least %d.",
                prob_n / 128 * par);
  int rc = marlin_gemm(A, B, C, s, prob_m, prob_n, prob_k, workspace, groupsize, dev, stream,
                       thread_k, thread_n, sms, par);
  if (rc == MARLIN_ERR_PROB_SHAPE)
    return fail(rc, "Problem (m=%d, n=%d, k=%d) not compatible with thread_k=%d, thread_n=%d.",
                prob_m, prob_n, prob_k, thread_k, thread_n);
  if (rc == MARLIN_ERR_KERN_SHAPE)
    return fail(rc, "No kernel implementation for thread_k=%d, thread_n=%d, groupsize=%d.",
                thread_k, thread_n, groupsize);
  if (rc == MARLIN_ERR_RUNTIME) return fail(rc, "HIP runtime error: %s", g_last_error);
  if (rc != MARLIN_OK) return fail(rc, "%s", g_last_error);
  return rc;
}

int marlin_amd_check(int prob_m, int prob_n, int prob_k, int groupsize, int thread_k,
                     int thread_n) {
  return check_shape(prob_m, prob_n, prob_k, groupsize, thread_k, thread_n);
}

int marlin_amd_plan(int prob_m, int prob_n, int prob_k, int groupsize, int thread_k,
                    int thread_n, int sms, int cus, int* out) {
  for (int i = 0; i < 13; i++) out[i] = 0;
  int rc = check_shape(prob_m, prob_n, prob_k, groupsize, thread_k, thread_n);
  if (rc != MARLIN_OK || prob_m == 0 || prob_n == 0 || prob_k == 0) return rc;
  const PlanCtx cx = {cus, kPoolPartialLimit, t_force};
  Plan pl = make_plan(prob_m, prob_n, prob_k, sms, cx);
  out[0] = pl.kernel;
  out[1] = pl.grid;
  out[2] = pl.sp.gpb;
  out[3] = pl.sp.NT;
  out[4] = pl.sp.KG;
  out[5] = pl.launches;
  out[6] = pl.ksplit;
  out[7] = pl.tile_rows;
  out[8] = pl.kernel == 1 ? pl.sp.wpt : 0;
  out[9] = (int)(pl.partial_bytes >> 10);
  out[10] = pl.kernel == 1 || pl.kernel == 3 ? pl.row_parts : 1;
  out[11] = pl.kernel == 1 || pl.kernel == 3 ? pl.part_rows : 0;
  out[12] = pl.strips;
  return rc;
}

int marlin_amd_plan_costs(int prob_m, int prob_n, int prob_k, int groupsize, int cus, double* out) {
  for (int i = 0; i < 4; i++) out[i] = -1.0;
  int thread_k = -1, thread_n = -1;
  int rc = check_shape(prob_m, prob_n, prob_k, groupsize, thread_k, thread_n);
  if (rc != MARLIN_OK || prob_m == 0 || prob_n == 0 || prob_k == 0) return rc;
  const PlanCtx cx = {cus, kPoolPartialLimit, t_force};
  out[0] = stream_cost_as_planned(prob_m, prob_n, prob_k, cx);
  if (prob_n % 256 == 0) out[1] = prefill_cost(prob_m, prob_n, prob_k, cx);
  if (prob_m <= kStripMaxRows) {
    const int cs = strips_per_workgroup(prob_m, prob_n, prob_k, cx);
    if (cs > 0) out[2] = strip_cost(prob_m, prob_n, prob_k, cs, cx.cus);
    out[3] = cs;
  }
  return rc;
}

void marlin_amd_force_kernel(int which) { t_force.kernel = which >= 1 && which <= 4 ? which : 0; }
void marlin_amd_force_strips(int strips) {
  t_force.strips = strips >= 1 && strips <= 4 ? strips : 0;
}

void marlin_amd_force_k_slices(int slices) { t_force.k_slices = slices > 0 ? slices : 0; }

void marlin_amd_force_row_halves(int mode) { t_force.row_halves = mode == 1 || mode == 2 ? mode : 0; }

void marlin_amd_force_tile_rows(int rows) { t_force.tile_rows = rows == 64 || rows == 128 ? rows : 0; }

void marlin_amd_work_order(int grid, int* out) {
  for (int b = 0; b < grid; b++) out[b] = xcd_work_index(b, grid);
}

long long marlin_amd_scratch_bytes(int dev, int* buffers) {
  return (long long)scratch_bytes_held(dev, buffers);
}

long long marlin_amd_release(int dev) { return (long long)scratch_release(dev); }

int marlin_amd_device_info(int dev, int* out) {
  const hipDeviceAttribute_t what[5] = {
      hipDeviceAttributeMultiprocessorCount, hipDeviceAttributeClockRate,
      hipDeviceAttributeMemoryClockRate, hipDeviceAttributeMemoryBusWidth,
      hipDeviceAttributeL2CacheSize};
  for (int i = 0; i < 5; i++) {
    out[i] = 0;
    hipError_t e = hipDeviceGetAttribute(&out[i], what[i], dev);
    if (e != hipSuccess) {
      set_error(e, "hipDeviceGetAttribute");
      return MARLIN_ERR_RUNTIME;
    }
  }
  return MARLIN_OK;
}

const char* marlin_amd_last_error(void) { return g_last_error; }

const char* marlin_amd_version(void) { return "marlin_amd 0.2 (gfx950)"; }

}  // extern "C"
