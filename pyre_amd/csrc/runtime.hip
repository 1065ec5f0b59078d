// The library's small host-side state: the per-thread error message, the number of compute
// units of each device, the digest of the sources it was built from.
#include <atomic>

#include "pyre_api.h"
#include "pyre_common.h"

#ifndef PYRE_SOURCES_DIGEST
#define PYRE_SOURCES_DIGEST "unknown"
#endif

namespace pyre {
char* error_buffer() {
  static thread_local char buf[512] = "";
  return buf;
}

// Compute units of the current device, asked for once per device; kDefaultUnits where there
// is no device to ask (launch plans made on a machine without one).
int compute_units() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> known[kMaxDevices];
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    (void)hipGetLastError();
    return kDefaultUnits;
  }
  int n = known[device].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return kDefaultUnits;
  }
  known[device].store(n, std::memory_order_relaxed);
  return n;
}
}  // namespace pyre

extern "C" const char* pyre_last_error() { return pyre::error_buffer(); }
extern "C" int pyre_abi_version() { return 19; }
extern "C" int pyre_compute_units() { return pyre::compute_units(); }
extern "C" const char* pyre_sources_digest() { return PYRE_SOURCES_DIGEST; }

// ---------------------------------------------------------------------------
// A plain streaming read of `bytes` (a multiple of 16) for measuring what the
// memory system delivers: every lane loads 16 bytes per iteration, the loads of
// one wave are contiguous, and nothing but a checksum is written. The loads are
// non-temporal, as those of the kernels that stream weights: data that is read once
// goes past the caches (ordinary loads reach about four fifths of this).
// ---------------------------------------------------------------------------
typedef unsigned probe_u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void read_probe_kernel(const probe_u32x4* __restrict__ p, size_t n,
                                                          unsigned* __restrict__ sink) {
  // A block takes spans of 64 KB (4,096 pieces of 16 bytes), span b, b + blocks, ...: 16 loads
  // per thread and span, four in flight.
  constexpr size_t kSpan = 4096;
  unsigned acc = 0;
  for (size_t s0 = static_cast<size_t>(blockIdx.x) * kSpan; s0 < n; s0 += static_cast<size_t>(gridDim.x) * kSpan) {
    const size_t end = s0 + kSpan < n ? s0 + kSpan : n;
    size_t i = s0 + threadIdx.x;
    for (; i + 768 < end; i += 1024) {
      const probe_u32x4 a = __builtin_nontemporal_load(p + i), b = __builtin_nontemporal_load(p + i + 256),
                        c = __builtin_nontemporal_load(p + i + 512), d = __builtin_nontemporal_load(p + i + 768);
      acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; i < end; i += 256) {
      const probe_u32x4 a = __builtin_nontemporal_load(p + i);
      acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
  }
  if (acc == 0x9e3779b9u) *sink = acc;  // practically never: keeps the loads alive
}

extern "C" int pyre_read_probe(const void* p, size_t bytes, int blocks, unsigned* sink, hipStream_t stream) {
  PYRE_REQUIRE(bytes % 16 == 0 && blocks > 0, "read_probe: bytes must be a multiple of 16");
  hipLaunchKernelGGL(read_probe_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<const probe_u32x4*>(p),
                     bytes / 16, sink);
  return pyre::check_launch("read_probe");
}
