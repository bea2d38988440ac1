// Measurement aid of bench.py, not part of the plugin path: reads a buffer once, front to back,
// with 128-bit loads and nothing else, the rate a kernel that only reads contiguous memory gets from
// HBM on this GPU.  The yardstick for the gather of uniform random rows beside the 8 TB/s peak and the
// device copy (which also writes).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {
typedef uint32_t U4 __attribute__((ext_vector_type(4)));
constexpr int kInFlight = 8;

// Every lane xors what it loads; the result is stored only if it equals a value the host chooses so
// that it never does (the loads cannot be dropped, nothing is written).
__global__ __launch_bounds__(256) void stream_read_kernel(const U4* __restrict__ src, size_t n_vec, U4* sink, uint32_t never) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  U4 acc = {0, 0, 0, 0};
  for (; i + (kInFlight - 1) * stride < n_vec; i += kInFlight * stride) {
    U4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) acc ^= v[u];
  }
  for (; i < n_vec; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == never && never != 0) sink[threadIdx.x] = acc;
}
}  // namespace

// Reads `bytes` (a multiple of 16) at `src` with `grid` workgroups of 256 lanes.  Returns the hipError_t (0 = ok).
extern "C" int fwdmi_mb_stream_read(const void* src, size_t bytes, int grid, void* stream) {
  if (!src || bytes < 16 || (bytes & 15) || grid <= 0 || (reinterpret_cast<uintptr_t>(src) & 15)) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const U4*>(src), bytes / 16, nullptr, 0u);
  return (int)hipGetLastError();
}
