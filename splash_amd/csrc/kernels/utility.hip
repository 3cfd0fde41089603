// Utility kernels: copy_bytes moves 16-byte vectors (grid-stride), read_bytes streams a buffer and
// folds it into one word per workgroup. Both are what a plain memory-bound kernel looks like on
// this device: the operators' kernels are measured against them.
#include "abi/Utility.h"
#include "backend/KernelRegistry.hpp"
#include "kernels/device_common.hpp"

namespace splash::kernels {

__global__ __launch_bounds__(256) void copy_bytes(const uint4 *__restrict__ source, uint4 *__restrict__ destination,
                                                  UtilityCopyParams p) {
  const uint64_t stride = uint64_t(gridDim.x) * blockDim.x;
  for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < p.vectors; i += stride)
    destination[i] = load_stream(source + i);
}
SP_REGISTER_KERNEL("copy_bytes", &copy_bytes);

// Each thread keeps four independent 16-byte loads in flight per trip.
__global__ __launch_bounds__(256) void read_bytes(const uint4 *__restrict__ source, uint32_t *__restrict__ folded,
                                                  UtilityCopyParams p) {
  const uint64_t stride = uint64_t(gridDim.x) * blockDim.x;
  uint32_t fold = 0;
  uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < p.vectors; i += 4 * stride) {
    const uint4 a = load_stream(source + i), b = load_stream(source + i + stride), c = load_stream(source + i + 2 * stride),
                d = load_stream(source + i + 3 * stride);
    fold ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < p.vectors; i += stride) {
    const uint4 a = load_stream(source + i);
    fold ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  fold = wave_sum(fold);
  if ((threadIdx.x & 63u) == 0 && fold == 0x9E3779B9u) folded[blockIdx.x] = fold;  // keeps the loads alive
}
SP_REGISTER_KERNEL("read_bytes", &read_bytes);

} // namespace splash::kernels
