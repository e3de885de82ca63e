// Measurement probes (libmarlin_amd_probe.so, include/marlin_amd_probe.h): what
// a launch and a plain read of the packed weights cost on this device, with no
// arithmetic, and what the matrix pipes sustain by themselves, to judge the
// GEMM kernels against.  A library of its own, beside libmarlin_amd.so, which
// it asks for the plan of the shape (marlin_amd_plan): the product library
// carries no measurement code.
//
// probe_read_kernel walks the packed weights exactly as the streaming kernel
// does for the same plan -- same work split, same workgroup-to-XCD order, same
// 128-bit streaming buffer loads of 1 KiB per wave instruction, four rows per
// granule -- keeps up to kProbeDepth granules in flight per wave, and throws
// the data away; probe_read_strips_kernel does the same for the column-strip
// kernel's split (a workgroup of eight waves per 16, 32 or 64 columns over the
// whole k range, eight rows of a strip per wave instruction).
// probe_empty_kernel does nothing at all.  probe_mfma_kernel is
// a loop of nothing but v_mfma_f32_16x16x32_f16 on pseudo-random operands, two
// waves per SIMD and 32 independent accumulators per wave: what the matrix
// pipes of this board sustain when nothing competes with them.
#include <cstdio>

#include "../../include/marlin_amd_probe.h"
#include "../../include/marlin_amd_tools.h"
#include "w4a16_common.hpp"

namespace w4a16 {

namespace {
constexpr int kProbeDepth = 4;
constexpr int kProbeOob = (int)0x80000000;
}  // namespace

__global__ __launch_bounds__(512) void probe_empty_kernel() {}

__global__ __launch_bounds__(256) void probe_read_kernel(GemmArgs p, int* sink) {
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int kg = lane >> 4, nu = lane & 15;
  const int NT = p.N / kTileN, KG = p.K / kGranuleK;
  const int total = NT * KG;
  const int wid = xcd_work_index((int)blockIdx.x, (int)gridDim.x);
  int u0, u1;
  if (p.wpt > 0) {
    const int t = wid / p.wpt, run = wid - t * p.wpt;
    u0 = t * KG + (run * KG) / p.wpt;
    u1 = t * KG + ((run + 1) * KG) / p.wpt;
    if (t >= NT) return;
  } else {
    u0 = wid * p.gpb;
    u1 = min(total, u0 + p.gpb);
  }
  const __amdgpu_buffer_rsrc_t rB = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void*>(p.B), 0, (int)((unsigned)p.K * (unsigned)(p.N / 2)), 0x00020000);
  const int b_row = p.N * 8;
  const int b_lane = 64 * nu + 16 * kg;
  i4 acc = {0, 0, 0, 0};
  i4 buf[kProbeDepth][4];
  auto issue = [&](int slot, int u) {
    const bool valid = u < u1;
    const int t = u / KG, kq = u - t * KG;
    const int vb = b_lane | (valid ? 0 : kProbeOob);
    const int sb = valid ? (4 * kq) * b_row + 1024 * t : 0;
#pragma unroll
    for (int r = 0; r < 4; r++)
      buf[slot][r] = __builtin_amdgcn_raw_buffer_load_b128(rB, vb, sb + r * b_row, 2);
  };
  int u = u0 + wave;
#pragma unroll
  for (int d = 0; d < kProbeDepth; d++) issue(d, u + 4 * d);
  for (; u < u1; u += 4 * kProbeDepth) {
#pragma unroll
    for (int d = 0; d < kProbeDepth; d++) {
#pragma unroll
      for (int r = 0; r < 4; r++) acc |= buf[d][r];
      issue(d, u + 4 * (d + kProbeDepth));
    }
  }
  // uniform packed nibbles never OR to this pattern: nothing is written
  if ((acc[0] & acc[1] & acc[2] & acc[3]) == 0x12345678 && sink) sink[0] = 1;
}

template <int CS>
__global__ __launch_bounds__(512) void probe_read_strips_kernel(GemmArgs p, int* sink) {
  // rows of B per chunk: two loads of 1 KiB per wave (three for three strips)
  constexpr int NL = CS == 3 ? 3 : 2;
  constexpr int kRows = 8 * NL / CS;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wid = xcd_work_index((int)blockIdx.x, (int)gridDim.x);
  // (rows in parts: every part of a strip set reads the set's weights)
  const int strip0 = (p.row_parts > 1 ? wid / p.row_parts : wid) * CS;
  const int n_chunks = ceil_div(p.K, 16 * kRows);
  const int c0 = (wave * n_chunks) / 8, c1 = ((wave + 1) * n_chunks) / 8;
  const __amdgpu_buffer_rsrc_t rB = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void*>(p.B), 0, (int)((unsigned)p.K * (unsigned)(p.N / 2)), 0x00020000);
  const int b_row = p.N * 8;
  int b_lane[NL];
#pragma unroll
  for (int i = 0; i < NL; i++) {
    const int idx = 64 * i + lane;
    const int strip = strip0 + (idx / 8) % CS;
    // (a strip past the last one, of a last workgroup of three, is not read)
    b_lane[i] = strip < (p.N >> 4)
                    ? (idx / (8 * CS)) * b_row + 128 * strip + 16 * (idx % 8)
                    : kProbeOob;
  }
  i4 acc = {0, 0, 0, 0};
  i4 buf[kProbeDepth][NL];
  auto issue = [&](int slot, int c) {
    const int inv = c < c1 ? 0 : kProbeOob;
#pragma unroll
    for (int i = 0; i < NL; i++)
      buf[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(
          rB, (b_lane[i] + c * kRows * b_row) | inv, 0, 2);
  };
#pragma unroll
  for (int d = 0; d < kProbeDepth; d++) issue(d, c0 + d);
  for (int c = c0; c < c1; c += kProbeDepth) {
#pragma unroll
    for (int d = 0; d < kProbeDepth; d++) {
#pragma unroll
      for (int i = 0; i < NL; i++) acc |= buf[d][i];
      issue(d, c + d + kProbeDepth);
    }
  }
  if ((acc[0] & acc[1] & acc[2] & acc[3]) == 0x12345678 && sink) sink[0] = 1;
}

__global__ __launch_bounds__(512) void probe_mfma_kernel(int iters, float* sink) {
  // operands: fp16 values in (-1, 1) from a hash of the lane and the register
  unsigned x = (unsigned)(blockIdx.x * 512 + threadIdx.x) * 2654435761u + 12345u;
  auto next = [&]() {
    x = x * 1664525u + 1013904223u;
    return (half_t)((float)(int)(x >> 8) * (1.0f / 8388608.0f) - 1.0f);
  };
  h8 w[8], a[4];
#pragma unroll
  for (int o = 0; o < 8; o++)
#pragma unroll
    for (int e = 0; e < 8; e++) w[o][e] = next();
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) a[i][e] = next();
  f4 acc[4][8];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int o = 0; o < 8; o++) acc[i][o] = (f4){0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int o = 0; o < 8; o++)
        acc[i][o] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[o], a[i], acc[i][o], 0, 0, 0);
  }
  f4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int o = 0; o < 8; o++) sum += acc[i][o];
  // sums of products of values below one stay far from this: nothing is written
  if (sum[0] + sum[1] + sum[2] + sum[3] == 1.2345e30f && sink) sink[0] = 1.f;
}

// What a lone wave per SIMD can issue beside its MFMAs: 32 independent
// v_mfma_f32_16x16x32_f16 per turn, each followed by NV independent packed-fp16
// VALU operations, NL 16-byte LDS reads and NG 16-byte global loads (per 8
// MFMAs for the two memory kinds).  Thread 0 of every workgroup writes the
// cycles one turn took, averaged over the run; one workgroup of four waves per
// CU (the LDS request keeps a second one out).
template <int NV, int NL, int NG>
__global__ __launch_bounds__(256) void probe_issue_kernel(int iters, const i4* src, float* out) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  unsigned x = (unsigned)(blockIdx.x * 256 + threadIdx.x) * 2654435761u + 12345u;
  auto next = [&]() {
    x = x * 1664525u + 1013904223u;
    return (half_t)((float)(int)(x >> 8) * (1.0f / 8388608.0f) - 1.0f);
  };
  h8 w[8], a[4];
#pragma unroll
  for (int o = 0; o < 8; o++)
#pragma unroll
    for (int e = 0; e < 8; e++) w[o][e] = next();
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) a[i][e] = next();
  f4 acc[4][8];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int o = 0; o < 8; o++) acc[i][o] = (f4){0.f, 0.f, 0.f, 0.f};
  h2 v[8];
#pragma unroll
  for (int r = 0; r < 8; r++) v[r] = (h2){next(), next()};
  const h2 mul = {(half_t)0.999f, (half_t)1.001f};
  i4 sink = {0, 0, 0, 0};
  const unsigned lds_at = (unsigned)(size_t)(lds + threadIdx.x * 16);
  const i4* g = src + threadIdx.x;
  __syncthreads();
  const unsigned long long t0 = __builtin_readcyclecounter();
  // the loads of a row block are consumed one row block later (eight MFMAs,
  // more than their latency from LDS or a cache hit), so that what is measured
  // is what issuing them costs, not the wait for them
  i4 got_l[2][NL > 0 ? NL : 1] = {}, got_g[2][NG > 0 ? NG : 1] = {};
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int o = 0; o < 8; o++) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[i][o]) : "v"(w[o]), "v"(a[i]));
#pragma unroll
        for (int r = 0; r < NV; r++)
          asm volatile("v_pk_mul_f16 %0, %0, %1" : "+v"(v[(o * NV + r) & 7]) : "v"(mul));
        if (o < NL)
          asm volatile("ds_read_b128 %0, %1" : "=v"(got_l[i & 1][o]) : "v"(lds_at) : "memory");
        if (o < NG)
          asm volatile("global_load_dwordx4 %0, %1, off"
                       : "=v"(got_g[i & 1][o])
                       : "v"(g + 256 * o)
                       : "memory");
      }
      // all but this row block's loads have landed
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(%1)" ::"n"(NG), "n"(NL) : "memory");
#pragma unroll
      for (int o = 0; o < NL; o++) sink |= got_l[(i & 1) ^ 1][o];
#pragma unroll
      for (int o = 0; o < NG; o++) sink |= got_g[(i & 1) ^ 1][o];
    }
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  const unsigned long long t1 = __builtin_readcyclecounter();
  f4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int o = 0; o < 8; o++) sum += acc[i][o];
  float keep = sum[0] + sum[1] + sum[2] + sum[3];
#pragma unroll
  for (int r = 0; r < 8; r++) keep += (float)v[r][0] + (float)v[r][1];
  if (threadIdx.x == 0)
    out[blockIdx.x] = (float)(t1 - t0) / (float)iters +
                      ((keep == 1.2345e30f || sink[0] == 0x12345678) ? 1.f : 0.f);
}

// What one CU pulls from memory: every workgroup of 256 threads reads its own
// `bytes_per_wg` of `src` with `depth` 16-byte loads in flight per thread and
// writes the time it took in ticks of the 100 MHz constant clock (thread 0) --
// with one workgroup the figure is one CU's, with one per CU the whole chip's.
template <int DEPTH>
__global__ __launch_bounds__(256) void probe_pull_kernel(const i4* src, int pieces_per_thread,
                                                         float* out) {
  const i4* g = src + (size_t)blockIdx.x * 256 * pieces_per_thread + threadIdx.x;
  i4 acc = {0, 0, 0, 0};
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
  for (int p = 0; p < pieces_per_thread; p += DEPTH) {
    i4 got[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
      got[d] = __builtin_nontemporal_load(g + (size_t)(p + d) * 256);
#pragma unroll
    for (int d = 0; d < DEPTH; d++) acc |= got[d];
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0)
    out[blockIdx.x] = (float)(t1 - t0) + ((acc[0] & acc[1]) == 0x12345678 ? 1.f : 0.f);
}

}  // namespace w4a16

namespace {
thread_local char g_probe_error[256] = "";

bool probe_fail(const char* what, hipError_t e) {
  snprintf(g_probe_error, sizeof(g_probe_error), "%s: %s", what, hipGetErrorString(e));
  return false;
}

// launch `fn` (which enqueues one kernel writing n floats to dev_out), wait,
// bring the floats to `host_out`
template <class F>
bool run_and_fetch(int n, float* host_out, F fn) {
  float* dev_out = nullptr;
  hipError_t e = hipMalloc((void**)&dev_out, (size_t)n * sizeof(float));
  if (e != hipSuccess) return probe_fail("hipMalloc", e);
  (void)hipGetLastError();
  fn(dev_out);
  e = hipGetLastError();
  if (e == hipSuccess) e = hipDeviceSynchronize();
  if (e == hipSuccess) e = hipMemcpy(host_out, dev_out, (size_t)n * sizeof(float), hipMemcpyDeviceToHost);
  (void)hipFree(dev_out);
  return e == hipSuccess ? true : probe_fail("probe launch", e);
}
}  // namespace

extern "C" {

int marlin_amd_probe(int kind, const void* B, int prob_m, int prob_n, int prob_k, int dev,
                     void* stream_) {
  using namespace w4a16;
  hipStream_t stream = (hipStream_t)stream_;
  g_probe_error[0] = 0;
  if (prob_m <= 0 || prob_n <= 0 || prob_k <= 0 || dev < 0 || kind < 0 || kind > 2)
    return MARLIN_ERR_PROB_SHAPE;
  int info[5] = {0, 0, 0, 0, 0};
  if (marlin_amd_device_info(dev, info) != MARLIN_OK || info[0] <= 0) {
    snprintf(g_probe_error, sizeof(g_probe_error), "device %d: %s", dev, marlin_amd_last_error());
    return MARLIN_ERR_RUNTIME;
  }
  const int cus = info[0];
  // the grid and the work split of a launch of this shape with prob_m rows; where
  // that is the prefill kernel's, of a launch with 16 rows
  int plan[13];
  int rc = marlin_amd_plan(prob_m, prob_n, prob_k, -1, -1, -1, -1, cus, plan);
  if (rc == MARLIN_OK && plan[0] == 2)
    rc = marlin_amd_plan(16, prob_n, prob_k, -1, -1, -1, -1, cus, plan);
  if (rc != MARLIN_OK) return rc;
  int prev = -1;
  hipError_t e = hipGetDevice(&prev);
  if (e == hipSuccess && prev != dev) e = hipSetDevice(dev);
  if (e != hipSuccess) {
    snprintf(g_probe_error, sizeof(g_probe_error), "hipSetDevice: %s", hipGetErrorString(e));
    return MARLIN_ERR_RUNTIME;
  }
  (void)hipGetLastError();
  const int grid = plan[1];
  const int strips = plan[0] == 3 ? plan[12] : 0;
  if (kind == 0) {
    hipLaunchKernelGGL(probe_empty_kernel, dim3(grid), dim3(strips ? 512 : 256), 0, stream);
  } else if (kind == 1 && strips) {
    GemmArgs a = {};
    a.B = B;
    a.M = 1;
    a.N = prob_n;
    a.K = prob_k;
    a.row_parts = plan[10];
    if (strips == 1)
      hipLaunchKernelGGL(probe_read_strips_kernel<1>, dim3(grid), dim3(512), 0, stream, a, (int*)nullptr);
    else if (strips == 2)
      hipLaunchKernelGGL(probe_read_strips_kernel<2>, dim3(grid), dim3(512), 0, stream, a, (int*)nullptr);
    else if (strips == 3)
      hipLaunchKernelGGL(probe_read_strips_kernel<3>, dim3(grid), dim3(512), 0, stream, a, (int*)nullptr);
    else
      hipLaunchKernelGGL(probe_read_strips_kernel<4>, dim3(grid), dim3(512), 0, stream, a, (int*)nullptr);
  } else if (kind == 1) {
    GemmArgs a = {};
    a.B = B;
    a.M = 1;
    a.N = prob_n;
    a.K = prob_k;
    a.gpb = plan[2];
    a.wpt = plan[8];
    hipLaunchKernelGGL(probe_read_kernel, dim3(grid), dim3(256), 0, stream, a, (int*)nullptr);
  } else {
    // one workgroup of 8 waves per CU; n*k/8192 MFMAs per wave (a multiple of 32)
    const long long per_wave = (long long)prob_n * prob_k / 8192;
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(cus), dim3(512), 0, stream,
                       (int)(per_wave / 32 > 0 ? per_wave / 32 : 1), (float*)nullptr);
  }
  e = hipGetLastError();
  if (prev != dev) (void)hipSetDevice(prev);
  if (e != hipSuccess) {
    snprintf(g_probe_error, sizeof(g_probe_error), "probe launch: %s", hipGetErrorString(e));
    return MARLIN_ERR_RUNTIME;
  }
  return MARLIN_OK;
}

int marlin_amd_probe_issue(int n_valu, int n_lds, int n_global, int iters, int workgroups,
                           float* cycles_out) {
  using namespace w4a16;
  g_probe_error[0] = 0;
  if (iters <= 0 || workgroups <= 0 || workgroups > 4096 || !cycles_out)
    return MARLIN_ERR_PROB_SHAPE;
  i4* src = nullptr;
  hipError_t e = hipMalloc((void**)&src, 256 * 8 * sizeof(i4));
  if (e != hipSuccess) {
    probe_fail("hipMalloc", e);
    return MARLIN_ERR_RUNTIME;
  }
  (void)hipMemset(src, 0, 256 * 8 * sizeof(i4));
  const int lds = 96 * 1024;  // more than half a CU's: one workgroup per CU
  bool ok = false, known = true;
  auto go = [&](auto kernel) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) !=
        hipSuccess)
      return probe_fail("hipFuncSetAttribute", hipGetLastError());
    return run_and_fetch(workgroups, cycles_out, [&](float* out) {
      hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(256), lds, 0, iters, (const i4*)src, out);
    });
  };
  const int key = n_valu * 100 + n_lds * 10 + n_global;
  switch (key) {
    case 0: ok = go(probe_issue_kernel<0, 0, 0>); break;
    case 100: ok = go(probe_issue_kernel<1, 0, 0>); break;
    case 200: ok = go(probe_issue_kernel<2, 0, 0>); break;
    case 300: ok = go(probe_issue_kernel<3, 0, 0>); break;
    case 400: ok = go(probe_issue_kernel<4, 0, 0>); break;
    case 10: ok = go(probe_issue_kernel<0, 1, 0>); break;
    case 20: ok = go(probe_issue_kernel<0, 2, 0>); break;
    case 1: ok = go(probe_issue_kernel<0, 0, 1>); break;
    case 2: ok = go(probe_issue_kernel<0, 0, 2>); break;
    case 210: ok = go(probe_issue_kernel<2, 1, 0>); break;
    case 201: ok = go(probe_issue_kernel<2, 0, 1>); break;
    default: known = false;
  }
  (void)hipFree(src);
  if (!known) return MARLIN_ERR_PROB_SHAPE;
  return ok ? MARLIN_OK : MARLIN_ERR_RUNTIME;
}

int marlin_amd_probe_pull(const void* src, long long src_bytes, long long bytes_per_workgroup,
                          int depth, int workgroups, float* cycles_out) {
  using namespace w4a16;
  g_probe_error[0] = 0;
  const long long pieces = bytes_per_workgroup / (256 * 16);
  if (!src || !cycles_out || workgroups <= 0 || workgroups > 4096 || pieces <= 0 ||
      pieces > (1 << 20) || pieces % 16 != 0 || pieces * 256 * 16 * workgroups > src_bytes)
    return MARLIN_ERR_PROB_SHAPE;
  bool ok;
  auto go = [&](auto kernel) {
    return run_and_fetch(workgroups, cycles_out, [&](float* out) {
      hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(256), 0, 0, (const i4*)src, (int)pieces, out);
    });
  };
  switch (depth) {
    case 1: ok = go(probe_pull_kernel<1>); break;
    case 4: ok = go(probe_pull_kernel<4>); break;
    case 16: ok = go(probe_pull_kernel<16>); break;
    default: return MARLIN_ERR_PROB_SHAPE;
  }
  return ok ? MARLIN_OK : MARLIN_ERR_RUNTIME;
}

const char* marlin_amd_probe_last_error(void) { return g_probe_error; }

}  // extern "C"
