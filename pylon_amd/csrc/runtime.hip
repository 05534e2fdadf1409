// Process-wide pieces of the kernel library: the error text of the last refused call
// (per host thread) and a description of the device the kernels were built for.
#include "common.h"

#include <string.h>

thread_local char pylon_error_text[512] = "";

extern "C" const char* pylon_last_error() { return pylon_error_text; }

extern "C" int pylon_abi_version() { return 1; }

// 0 if the current device can run this library's code objects (gfx950), else 1 with
// the device's architecture name in the error text.
extern "C" int pylon_check_device() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) PYLON_REFUSE("no HIP device: %s", hipGetErrorString(e));
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) PYLON_REFUSE("hipGetDeviceProperties failed: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    PYLON_REFUSE("these kernels are built for gfx950; the device is %s", prop.gcnArchName);
  return 0;
}

// Compute units of the current device, kept per device after the first question.
extern "C" int pylon_compute_units() {
  static int known[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return 0;
  }
  if (known[dev] == 0) {
    int units = 0;
    if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    known[dev] = units;
  }
  return known[dev];
}

// ---- a measurement aid: how fast can this device read memory? ---------------------------
// Every thread reads 16 bytes at a time, eight loads in flight, and folds them into a word
// nobody looks at (the store is never taken).  bench.py times it over a buffer larger than
// every cache to report bandwidths against a measured peak beside the published one.
typedef unsigned int probe_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void probe_read_kernel(const probe_u32x4* __restrict__ p, size_t n16,
                                                         unsigned* __restrict__ sink) {
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  unsigned acc = 0;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    probe_u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) {
    const probe_u32x4 v = p[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

extern "C" int pylon_probe_read(const void* data, long long bytes, unsigned* sink, hipStream_t stream) {
  PYLON_REQUIRE(data != nullptr && sink != nullptr && bytes >= 16 && (reinterpret_cast<uintptr_t>(data) & 15) == 0,
                "probe_read: needs a 16-byte aligned buffer of at least 16 bytes and a sink");
  hipLaunchKernelGGL(probe_read_kernel, dim3(8192), dim3(256), 0, stream,
                     static_cast<const probe_u32x4*>(data), static_cast<size_t>(bytes) / 16, sink);
  PYLON_LAUNCHED("probe_read");
}
