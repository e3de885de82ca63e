// Library-owned device scratch shared by the W4A16 and the dense GEMM paths:
// fp32 partial sums of output tiles that several workgroups share, and the
// tile counters of the kernels whose tiles outnumber the caller's workspace.
//
// One buffer per (device, stream), so that GEMMs on different streams never see
// each other's partial sums.  Layout: kCounterBytes of int counters (zero
// whenever no launch is in flight: the kernels hand them back zeroed), then the
// partial sums.  A buffer is sized by the plan of the call that needs it and
// grows on demand; nothing is allocated for calls that exchange nothing.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace w4a16 {

constexpr size_t kCounterBytes = 64 * 1024;  // 16384 tile counters
constexpr int kMaxCounters = (int)(kCounterBytes / sizeof(int));
constexpr int kPoolMaxDevices = 16;
// buffers held per device at most (live and outgrown ones together); every
// stream handle that ever shared tiles keeps its buffer until scratch_release
constexpr size_t kPoolMaxBuffers = 256;

struct ScratchView {
  int* counters;    // kMaxCounters ints, zero between launches
  float* partials;  // at least the requested bytes
};

// The scratch of (dev, stream) with room for partial_bytes of partial sums;
// `dev` must be the current device.  Allocates or grows when needed: growing
// waits for the stream's earlier work (which may still use the old buffer).
// Fails -- returns false with a message in err -- when hipMalloc fails, when
// an allocation would be needed while the stream is being captured into a
// graph, or when the device already holds kPoolMaxBuffers buffers.  (While
// another stream is under capture the allocation is made in relaxed capture
// mode, which leaves that capture valid.)
bool scratch_acquire(int dev, hipStream_t stream, size_t partial_bytes, ScratchView* out,
                     char* err, size_t err_len);

// Frees every buffer of device dev (all devices if dev < 0) after waiting for
// the device's work.  Returns the number of bytes freed.
size_t scratch_release(int dev);

// Bytes currently held for device dev (all devices if dev < 0), and the number
// of (device, stream) buffers.  Touches no GPU.
size_t scratch_bytes_held(int dev, int* buffers);

}  // namespace w4a16
