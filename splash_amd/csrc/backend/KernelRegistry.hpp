// Kernels are looked up by name, as the reference's MetalBackend looks up its pipelines
// (runtime/metal/MetalBackend.hpp:156-169 ComputeDispatch::pipelineName). Each .hip file registers
// its kernels with SP_REGISTER_KERNEL; the launcher binds the dispatch's buffers, in order, to the
// kernel's pointer parameters and copies the parameter struct by value into its last one.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

namespace splash::hipbackend {

struct LaunchArgs {
  hipStream_t stream;
  dim3 grid, block;
  void *const *buffers;
  uint32_t buffer_count;
  const void *params;
  uint32_t params_bytes;
};
using KernelLauncher = hipError_t (*)(const LaunchArgs &);

struct KernelEntry {
  std::string name;
  KernelLauncher launch = nullptr;
  uint32_t buffers = 0;       // pointer parameters the kernel binds
  uint32_t params_bytes = 0;  // sizeof its parameter struct
};

void registerKernel(KernelEntry entry);
const KernelEntry *findKernel(const char *name);
const std::vector<KernelEntry> &allKernels();

template <class F> struct KernelTraits;
template <class... A> struct KernelTraits<void (*)(A...)> {
  using Args = std::tuple<A...>;
  static constexpr size_t kCount = sizeof...(A);
  using Params = std::tuple_element_t<kCount - 1, Args>;
};

template <auto Kernel, size_t... I> hipError_t launchTyped(const LaunchArgs &a, std::index_sequence<I...>) {
  using Traits = KernelTraits<decltype(Kernel)>;
  typename Traits::Params params;
  std::memcpy(&params, a.params, sizeof(params));
  hipLaunchKernelGGL(Kernel, a.grid, a.block, 0, a.stream,
                     reinterpret_cast<std::tuple_element_t<I, typename Traits::Args>>(a.buffers[I])..., params);
  return hipGetLastError();
}
template <auto Kernel> hipError_t launchKernel(const LaunchArgs &a) {
  return launchTyped<Kernel>(a, std::make_index_sequence<KernelTraits<decltype(Kernel)>::kCount - 1>{});
}
template <auto Kernel> KernelEntry makeEntry(std::string name) {
  using Traits = KernelTraits<decltype(Kernel)>;
  return {std::move(name), &launchKernel<Kernel>, uint32_t(Traits::kCount - 1), uint32_t(sizeof(typename Traits::Params))};
}

struct KernelRegistrar {
  explicit KernelRegistrar(KernelEntry entry) { registerKernel(std::move(entry)); }
};

} // namespace splash::hipbackend

#define SP_CONCAT_(a, b) a##b
#define SP_CONCAT(a, b) SP_CONCAT_(a, b)
// Registers `kernel` (a __global__ function whose last parameter is its POD parameter struct and
// whose other parameters are device pointers) under `name`.
#define SP_REGISTER_KERNEL(name, ...)                                                           \
  static ::splash::hipbackend::KernelRegistrar SP_CONCAT(sp_registrar_, __COUNTER__)(           \
      ::splash::hipbackend::makeEntry<(__VA_ARGS__)>(name))
