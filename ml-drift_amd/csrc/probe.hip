// Measurement aids: the two floors a streaming kernel is judged against on a given box.  An empty
// launch (what a dependent launch costs with nothing to do) and a plain streaming read (every
// work-group reads one contiguous run of the buffer with 16-byte loads and keeps nothing).
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mldhip {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ void probe_empty_kernel(uint32_t* sink) {
  if (sink == nullptr) sink[0] = 1;
}

// 1024 threads x 8 loads of 16 bytes: 128 KB per work-group, contiguous.
__global__ __launch_bounds__(1024) void probe_stream_read_kernel(const u32x4* __restrict__ src, uint32_t* sink) {
  u32x4 v[8];
  const size_t base = (size_t)blockIdx.x * 8 * 1024 + threadIdx.x;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = __builtin_nontemporal_load(src + base + (size_t)j * 1024);
  uint32_t acc = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) acc ^= v[j][0] ^ v[j][1] ^ v[j][2] ^ v[j][3];
  if (acc == 0x12345678u) sink[threadIdx.x] = acc;  // keeps the loads alive; practically never taken
}

}  // namespace

hipError_t LaunchProbe(int kind, const void* src, size_t bytes, void* sink, hipStream_t stream) {
  if (kind == 0) {
    hipLaunchKernelGGL(probe_empty_kernel, dim3(224), dim3(1024), 0, stream, static_cast<uint32_t*>(sink));
    return hipGetLastError();
  }
  const size_t groups = bytes / (128 * 1024);
  if (kind != 1 || groups == 0 || groups > 0x7FFFFFFF) return hipErrorInvalidValue;
  hipLaunchKernelGGL(probe_stream_read_kernel, dim3((unsigned)groups), dim3(1024), 0, stream,
                     static_cast<const u32x4*>(src), static_cast<uint32_t*>(sink));
  return hipGetLastError();
}

}  // namespace mldhip
