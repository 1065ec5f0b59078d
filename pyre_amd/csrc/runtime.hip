// The library's small host-side state: the per-thread error message.
#include "pyre_api.h"
#include "pyre_common.h"

namespace pyre {
char* error_buffer() {
  static thread_local char buf[512] = "";
  return buf;
}
}  // namespace pyre

extern "C" const char* pyre_last_error() { return pyre::error_buffer(); }
extern "C" int pyre_abi_version() { return 14; }

// ---------------------------------------------------------------------------
// A plain streaming read of `bytes` (a multiple of 16) for measuring what the
// memory system delivers: every lane loads 16 bytes per iteration, the loads of
// one wave are contiguous, and nothing but a checksum is written.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ p, size_t n,
                                                          unsigned* __restrict__ sink) {
  unsigned acc = 0;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n; i += 4 * stride) {
    const uint4 a = p[i], b = p[i + stride], c = p[i + 2 * stride], d = p[i + 3 * stride];
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < n; i += stride) {
    const uint4 a = p[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u) *sink = acc;  // practically never: keeps the loads alive
}

extern "C" int pyre_read_probe(const void* p, size_t bytes, int blocks, unsigned* sink, hipStream_t stream) {
  PYRE_REQUIRE(bytes % 16 == 0 && blocks > 0, "read_probe: bytes must be a multiple of 16");
  hipLaunchKernelGGL(read_probe_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<const uint4*>(p),
                     bytes / 16, sink);
  return pyre::check_launch("read_probe");
}
