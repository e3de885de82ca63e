// Scratch pool: see scratch_pool.hpp.  Host code only.
#include "scratch_pool.hpp"

#include <atomic>
#include <cstdio>
#include <mutex>
#include <vector>

namespace w4a16 {

namespace {

struct Buffer {
  hipStream_t stream;
  char* ptr;
  size_t partial_bytes;  // capacity behind the counters
  bool retired;          // replaced by a larger one; kept because launches in
                         // flight and captured graphs may still name it
};

std::mutex g_mu;
std::vector<Buffer> g_buffers[kPoolMaxDevices];
// bumped whenever a buffer is added or freed: invalidates the per-thread cache
std::atomic<unsigned> g_generation{1};

// The last buffer this thread was handed: a call on the same (device, stream)
// with no larger need takes it without the lock.
struct Cached {
  unsigned generation = 0;
  int dev = -1;
  hipStream_t stream = nullptr;
  char* ptr = nullptr;
  size_t partial_bytes = 0;
};
thread_local Cached t_cached;

constexpr size_t kGrain = (size_t)1 << 20;  // capacities are whole MiB

void view_of(char* ptr, ScratchView* out) {
  out->counters = (int*)ptr;
  out->partials = (float*)(ptr + kCounterBytes);
}

void fail(char* err, size_t err_len, const char* what, hipError_t e) {
  if (err && err_len) snprintf(err, err_len, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace

bool scratch_acquire(int dev, hipStream_t stream, size_t partial_bytes, ScratchView* out,
                     char* err, size_t err_len) {
  if (dev < 0 || dev >= kPoolMaxDevices) {
    if (err && err_len) snprintf(err, err_len, "device index %d out of range", dev);
    return false;
  }
  Cached& c = t_cached;
  if (c.generation == g_generation.load(std::memory_order_acquire) && c.dev == dev &&
      c.stream == stream && c.partial_bytes >= partial_bytes) {
    view_of(c.ptr, out);
    return true;
  }
  std::lock_guard<std::mutex> lk(g_mu);
  Buffer* live = nullptr;
  for (Buffer& b : g_buffers[dev])
    if (b.stream == stream && !b.retired) live = &b;
  if (!live || live->partial_bytes < partial_bytes) {
    // nothing may be allocated under a capture: the allocation would become
    // part of nothing, and a synchronising call would break the capture
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    hipError_t e = hipStreamIsCapturing(stream, &cap);
    if (e != hipSuccess) {
      fail(err, err_len, "hipStreamIsCapturing", e);
      return false;
    }
    if (cap != hipStreamCaptureStatusNone) {
      if (err && err_len)
        snprintf(err, err_len,
                 "the stream is being captured and this call needs %zu bytes of scratch that "
                 "are not allocated yet: run the same call once on this stream before the "
                 "capture, or use marlin_gemm_static",
                 partial_bytes + kCounterBytes);
      return false;
    }
    // buffers are keyed by stream handle and kept until scratch_release (a
    // launch in flight or a captured graph may still name them), so a process
    // that keeps making streams would grow without bound: refuse beyond a cap
    if (g_buffers[dev].size() >= kPoolMaxBuffers) {
      if (err && err_len)
        snprintf(err, err_len,
                 "%zu scratch buffers are held on device %d (one per stream that shared tiles, "
                 "plus outgrown ones): call marlin_amd_release(%d) when those streams are idle",
                 g_buffers[dev].size(), dev, dev);
      return false;
    }
    size_t want = (partial_bytes + kGrain - 1) / kGrain * kGrain;
    if (live && want < 2 * live->partial_bytes) want = 2 * live->partial_bytes;
    if (want < kGrain) want = kGrain;
    // Another stream of this process may be under capture in the default
    // (global) mode, in which an allocation from any thread invalidates that
    // capture: this thread's calls below are made in relaxed mode.
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    char* p = nullptr;
    e = hipMalloc((void**)&p, kCounterBytes + want);
    // Cleared on the caller's stream, ahead of the launch that will use the
    // counters: a clear on the null stream is not ordered against a
    // non-blocking stream and could land in the middle of that launch.
    hipError_t e2 = e == hipSuccess ? hipMemsetAsync(p, 0, kCounterBytes, stream) : hipSuccess;
    if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode);
    if (e != hipSuccess) {
      fail(err, err_len, "hipMalloc(scratch)", e);
      return false;
    }
    if (e2 != hipSuccess) {
      fail(err, err_len, "hipMemsetAsync(scratch)", e2);
      (void)hipFree(p);
      return false;
    }
    if (live) live->retired = true;
    g_buffers[dev].push_back({stream, p, want, false});
    live = &g_buffers[dev].back();
    g_generation.fetch_add(1, std::memory_order_acq_rel);
  }
  c.generation = g_generation.load(std::memory_order_acquire);
  c.dev = dev;
  c.stream = stream;
  c.ptr = live->ptr;
  c.partial_bytes = live->partial_bytes;
  view_of(live->ptr, out);
  return true;
}

size_t scratch_release(int dev) {
  std::lock_guard<std::mutex> lk(g_mu);
  size_t freed = 0;
  int prev = -1;
  const bool have_prev = hipGetDevice(&prev) == hipSuccess;
  for (int d = 0; d < kPoolMaxDevices; d++) {
    if ((dev >= 0 && d != dev) || g_buffers[d].empty()) continue;
    if (hipSetDevice(d) != hipSuccess) continue;
    (void)hipDeviceSynchronize();
    for (Buffer& b : g_buffers[d]) {
      if (hipFree(b.ptr) == hipSuccess) freed += kCounterBytes + b.partial_bytes;
    }
    g_buffers[d].clear();
  }
  if (have_prev) (void)hipSetDevice(prev);
  g_generation.fetch_add(1, std::memory_order_acq_rel);
  return freed;
}

size_t scratch_bytes_held(int dev, int* buffers) {
  std::lock_guard<std::mutex> lk(g_mu);
  size_t bytes = 0;
  int n = 0;
  for (int d = 0; d < kPoolMaxDevices; d++) {
    if (dev >= 0 && d != dev) continue;
    for (const Buffer& b : g_buffers[d]) {
      bytes += kCounterBytes + b.partial_bytes;
      ++n;
    }
  }
  if (buffers) *buffers = n;
  return bytes;
}

}  // namespace w4a16
