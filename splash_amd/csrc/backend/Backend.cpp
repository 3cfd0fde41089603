// The C ABI of include/splash_hip.h over the HIP runtime: one device, one command stream, one
// command in flight, buffers as reference-counted handles, kernels by name.
#include "splash_hip.h"
#include "backend/KernelRegistry.hpp"
#include "backend/Internal.hpp"

#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

namespace splash::hipbackend {

namespace {
std::vector<KernelEntry> &registry() {
  static std::vector<KernelEntry> entries;
  return entries;
}
std::map<std::string, size_t> &registryIndex() {
  static std::map<std::string, size_t> index;
  return index;
}
} // namespace

void registerKernel(KernelEntry entry) {
  auto &index = registryIndex();
  if (index.count(entry.name)) {
    std::fprintf(stderr, "splash_hip: kernel %s registered twice\n", entry.name.c_str());
    std::abort();
  }
  index[entry.name] = registry().size();
  registry().push_back(std::move(entry));
}
const KernelEntry *findKernel(const char *name) {
  if (!name) return nullptr;
  const auto &index = registryIndex();
  const auto it = index.find(name);
  return it == index.end() ? nullptr : &registry()[it->second];
}
const std::vector<KernelEntry> &allKernels() { return registry(); }

} // namespace splash::hipbackend

using namespace splash::hipbackend;
using Clock = std::chrono::steady_clock;

namespace {
thread_local std::string tlsError;
sp_status fail(sp_status status, std::string message) {
  tlsError = std::move(message);
  return status;
}
sp_status hipFail(hipError_t error, const char *what) {
  return fail(error == hipErrorOutOfMemory ? SP_OUT_OF_MEMORY : SP_BACKEND_ERROR,
              std::string(what) + ": " + hipGetErrorString(error));
}
constexpr double kDefaultCommandTimeout = 120.0;  // runtime/Supervision.hpp:41
} // namespace

namespace splash::hipbackend {
void setLastError(const std::string &message) { tlsError = message; }
} // namespace splash::hipbackend

struct sp_backend {
  int device = 0;
  hipStream_t stream = nullptr;
  double timeout = kDefaultCommandTimeout;
  std::atomic<bool> healthy{true};
  std::atomic<bool> stopped{false};
  std::atomic<bool> inFlight{false};
  std::atomic<bool> profiling{false};
  mutable std::mutex mutex;  // reason, stats
  std::string reason;
  uint64_t allocated = 0, peak = 0, deviceCurrent = 0, devicePeak = 0;
  uint64_t deviceBaseline = 0;  // bytes in use on the device before this backend allocated
  std::atomic<int> liveBuffers{0};
  // The backend's memory outlives sp_backend_destroy while buffers, tickets or commands still name it.
  std::atomic<int> refs{1};
  void retain() { ++refs; }
  void release() { if (--refs == 0) delete this; }

  void markUnhealthy(const std::string &why) {
    std::lock_guard<std::mutex> lock(mutex);
    if (healthy.exchange(false)) reason = why;
  }
  void sampleDevice() {
    size_t freeBytes = 0, total = 0;
    if (hipMemGetInfo(&freeBytes, &total) != hipSuccess) return;
    const uint64_t used = total - freeBytes;
    deviceCurrent = used > deviceBaseline ? used - deviceBaseline : 0;
    devicePeak = std::max(devicePeak, deviceCurrent);
  }
};

struct sp_buffer {
  std::atomic<int> refs{1};
  sp_backend *backend = nullptr;
  sp_buffer *base = nullptr;  // retained; null for an allocation
  char *device = nullptr;     // address kernels use
  char *host = nullptr;       // Shared storage only
  uint64_t size = 0, allocated = 0;
  sp_storage storage = SP_STORAGE_PRIVATE;
  std::string label;
  const sp_buffer *root() const { return base ? base : this; }
};

struct RecordedDispatch {
  const KernelEntry *kernel = nullptr;
  std::vector<void *> pointers;
  std::vector<unsigned char> params;
  dim3 grid, block;
};

struct sp_ticket {
  sp_backend *backend = nullptr;
  hipEvent_t start = nullptr, end = nullptr;
  hipEvent_t fence = nullptr;     // after the completion callback, when there is one: what wait() polls
  std::vector<hipEvent_t> marks;  // dispatch profiling: count + 1 events
  std::vector<sp_buffer *> retained;
  Clock::time_point wallStart;
  std::atomic<bool> done{false};
  sp_completion completion = nullptr;
  void *user = nullptr;
};

struct sp_command {
  sp_backend *backend = nullptr;
  std::vector<RecordedDispatch> dispatches;
  std::vector<sp_buffer *> retained;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

namespace {

sp_status validateDispatch(const sp_dispatch &d, uint32_t index, RecordedDispatch &out, std::vector<sp_buffer *> &retained,
                           sp_backend *backend) {
  const std::string at = "dispatch " + std::to_string(index) + " (" + (d.kernel ? d.kernel : "<null>") + ")";
  const KernelEntry *kernel = findKernel(d.kernel);
  if (!kernel) return fail(SP_UNKNOWN_KERNEL, at + ": no kernel of that name");
  if (d.buffer_count != kernel->buffers)
    return fail(SP_INVALID_ARGUMENT, at + ": binds " + std::to_string(d.buffer_count) + " buffers, the kernel takes " +
                                         std::to_string(kernel->buffers));
  if (d.params_bytes != kernel->params_bytes || !d.params)
    return fail(SP_INVALID_ARGUMENT, at + ": parameter struct of " + std::to_string(d.params_bytes) +
                                         " bytes, the kernel takes " + std::to_string(kernel->params_bytes));
  if (d.indirect) return fail(SP_INVALID_ARGUMENT, at + ": indirect grids are not supported by this kernel");
  for (int i = 0; i < 3; ++i)
    if (!d.grid[i] || !d.block[i]) return fail(SP_INVALID_ARGUMENT, at + ": empty grid or workgroup");
  if (uint64_t(d.block[0]) * d.block[1] * d.block[2] > 1024)
    return fail(SP_INVALID_ARGUMENT, at + ": more than 1024 threads per workgroup");
  if (d.grid[1] > 65535 || d.grid[2] > 65535) return fail(SP_INVALID_ARGUMENT, at + ": grid y or z beyond 65535");
  out.kernel = kernel;
  out.grid = dim3(d.grid[0], d.grid[1], d.grid[2]);
  out.block = dim3(d.block[0], d.block[1], d.block[2]);
  out.params.assign(static_cast<const unsigned char *>(d.params), static_cast<const unsigned char *>(d.params) + d.params_bytes);
  out.pointers.resize(d.buffer_count);
  for (uint32_t b = 0; b < d.buffer_count; ++b) {
    sp_buffer *buffer = d.buffers[b];
    if (!buffer) return fail(SP_INVALID_ARGUMENT, at + ": buffer " + std::to_string(b) + " is null");
    if (buffer->backend != backend)
      return fail(SP_INVALID_ARGUMENT, at + ": buffer " + std::to_string(b) + " belongs to another backend");
    out.pointers[b] = buffer->device;
    retained.push_back(buffer);
  }
  return SP_OK;
}

void retainAll(const std::vector<sp_buffer *> &buffers) {
  for (sp_buffer *b : buffers) sp_buffer_retain(b);
}
void releaseAll(std::vector<sp_buffer *> &buffers) {
  for (sp_buffer *b : buffers) sp_buffer_release(b);
  buffers.clear();
}

hipError_t launchRecorded(sp_backend *backend, const RecordedDispatch &d) {
  LaunchArgs args{backend->stream, d.grid, d.block, d.pointers.data(), uint32_t(d.pointers.size()), d.params.data(),
                  uint32_t(d.params.size())};
  return d.kernel->launch(args);
}

void completionTrampoline(void *data) {
  auto *ticket = static_cast<sp_ticket *>(data);
  if (ticket->completion) ticket->completion(ticket->user);
}

sp_status guardSubmit(sp_backend *backend) {
  if (!backend) return fail(SP_INVALID_ARGUMENT, "null backend");
  if (backend->stopped) return fail(SP_BACKEND_ERROR, "the backend is stopped");
  if (!backend->healthy) return fail(SP_UNHEALTHY, "the backend is unhealthy");
  if (backend->inFlight) return fail(SP_BUSY, "a command is already in flight; wait for its ticket first");
  return SP_OK;
}

sp_status beginTicket(sp_backend *backend, sp_completion completion, void *user, size_t marks, sp_ticket **out) {
  auto *ticket = new sp_ticket;
  ticket->backend = backend;
  ticket->completion = completion;
  ticket->user = user;
  hipError_t e = hipEventCreate(&ticket->start);
  if (e == hipSuccess) e = hipEventCreate(&ticket->end);
  if (e == hipSuccess && completion) e = hipEventCreate(&ticket->fence);
  for (size_t i = 0; e == hipSuccess && i < marks; ++i) {
    hipEvent_t mark = nullptr;
    e = hipEventCreate(&mark);
    if (e == hipSuccess) ticket->marks.push_back(mark);
  }
  if (e != hipSuccess) {
    for (hipEvent_t m : ticket->marks) (void)hipEventDestroy(m);
    if (ticket->start) (void)hipEventDestroy(ticket->start);
    if (ticket->end) (void)hipEventDestroy(ticket->end);
    if (ticket->fence) (void)hipEventDestroy(ticket->fence);
    delete ticket;
    return hipFail(e, "hipEventCreate");
  }
  *out = ticket;
  return SP_OK;
}

void destroyTicket(sp_ticket *ticket) {
  for (hipEvent_t m : ticket->marks) (void)hipEventDestroy(m);
  (void)hipEventDestroy(ticket->start);
  (void)hipEventDestroy(ticket->end);
  if (ticket->fence) (void)hipEventDestroy(ticket->fence);
  releaseAll(ticket->retained);
  delete ticket;
}

// Waits for the ticket's end event under the command watchdog (CommandWatchdog.hpp:16-44).
sp_status awaitTicket(sp_ticket *ticket) {
  sp_backend *backend = ticket->backend;
  const auto begin = Clock::now();
  uint32_t spins = 0;
  for (;;) {
    const hipError_t e = hipEventQuery(ticket->fence ? ticket->fence : ticket->end);
    if (e == hipSuccess) return SP_OK;
    if (e != hipErrorNotReady) {
      backend->markUnhealthy(std::string("command failed: ") + hipGetErrorString(e));
      return hipFail(e, "command");
    }
    if (std::chrono::duration<double>(Clock::now() - begin).count() > backend->timeout) {
      backend->markUnhealthy("command watchdog: no completion within the command timeout");
      return fail(SP_TIMEOUT, "command watchdog: no completion within the command timeout");
    }
    if (++spins < 2000) std::this_thread::yield();
    else std::this_thread::sleep_for(std::chrono::microseconds(spins < 20000 ? 20 : 500));
  }
}

sp_status finishSubmit(sp_backend *backend, sp_ticket *ticket, hipError_t launchError, sp_ticket **out) {
  if (launchError != hipSuccess) {
    (void)hipStreamSynchronize(backend->stream);
    destroyTicket(ticket);
    backend->markUnhealthy(std::string("launch failed: ") + hipGetErrorString(launchError));
    return hipFail(launchError, "kernel launch");
  }
  if (ticket->completion) {
    // The callback runs between `end` and `fence`, so the ticket outlives it.
    (void)hipLaunchHostFunc(backend->stream, completionTrampoline, ticket);
    (void)hipEventRecord(ticket->fence, backend->stream);
  }
  backend->inFlight = true;
  *out = ticket;
  return SP_OK;
}

} // namespace

extern "C" {

const char *sp_last_error(void) { return tlsError.c_str(); }

sp_status sp_backend_create(int device, double command_timeout_seconds, sp_backend **out) {
  if (!out) return fail(SP_INVALID_ARGUMENT, "null result pointer");
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0) return fail(SP_BACKEND_ERROR, "no HIP device is visible");
  if (device < 0 || device >= count) return fail(SP_INVALID_ARGUMENT, "no such device");
  if ((e = hipSetDevice(device)) != hipSuccess) return hipFail(e, "hipSetDevice");
  auto *backend = new sp_backend;
  backend->device = device;
  if (command_timeout_seconds > 0) backend->timeout = command_timeout_seconds;
  if ((e = hipStreamCreateWithFlags(&backend->stream, hipStreamNonBlocking)) != hipSuccess) {
    delete backend;
    return hipFail(e, "hipStreamCreate");
  }
  size_t freeBytes = 0, total = 0;
  if (hipMemGetInfo(&freeBytes, &total) == hipSuccess) backend->deviceBaseline = total - freeBytes;
  *out = backend;
  return SP_OK;
}

void sp_backend_destroy(sp_backend *backend) {
  if (!backend) return;
  (void)hipSetDevice(backend->device);
  (void)hipStreamSynchronize(backend->stream);
  (void)hipStreamDestroy(backend->stream);
  backend->stream = nullptr;
  backend->stopped = true;
  // Buffers still alive keep the backend's bookkeeping; their memory is freed as they are released.
  backend->release();
}

void sp_backend_stop(sp_backend *backend) { if (backend) backend->stopped = true; }

sp_status sp_backend_device_info(sp_backend *backend, sp_device_info *out) {
  if (!backend || !out) return fail(SP_INVALID_ARGUMENT, "null argument");
  hipDeviceProp_t prop;
  const hipError_t e = hipGetDeviceProperties(&prop, backend->device);
  if (e != hipSuccess) return hipFail(e, "hipGetDeviceProperties");
  std::memset(out, 0, sizeof(*out));
  std::snprintf(out->name, sizeof(out->name), "%s", prop.name);
  std::snprintf(out->arch, sizeof(out->arch), "%s", prop.gcnArchName);
  out->compute_units = uint32_t(prop.multiProcessorCount);
  out->wavefront_size = uint32_t(prop.warpSize);
  out->lds_bytes_per_cu = uint32_t(prop.maxSharedMemoryPerMultiProcessor);
  out->l2_bytes = uint32_t(prop.l2CacheSize);
  out->hbm_bytes = prop.totalGlobalMem;
  out->clock_khz = uint32_t(prop.clockRate);
  out->memory_clock_khz = uint32_t(prop.memoryClockRate);
  out->memory_bus_bits = uint32_t(prop.memoryBusWidth);
  return SP_OK;
}

sp_status sp_buffer_alloc(sp_backend *backend, uint64_t bytes, sp_storage storage, const char *label, sp_buffer **out) {
  if (!backend || !out) return fail(SP_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  if (!bytes) return fail(SP_INVALID_ARGUMENT, std::string("buffer ") + (label ? label : "") + " has no bytes");
  if (storage != SP_STORAGE_SHARED && storage != SP_STORAGE_PRIVATE) return fail(SP_INVALID_ARGUMENT, "unknown storage");
  if (backend->stopped) return fail(SP_BACKEND_ERROR, "the backend is stopped");
  (void)hipSetDevice(backend->device);
  void *device = nullptr, *host = nullptr;
  hipError_t e;
  if (storage == SP_STORAGE_SHARED) {
    e = hipHostMalloc(&host, bytes, hipHostMallocDefault);
    if (e == hipSuccess) {
      std::memset(host, 0, bytes);
      e = hipHostGetDevicePointer(&device, host, 0);
      if (e != hipSuccess) (void)hipHostFree(host);
    }
  } else {
    e = hipMalloc(&device, bytes);
    if (e == hipSuccess) {
      e = hipMemsetAsync(device, 0, bytes, backend->stream);
      if (e == hipSuccess) e = hipStreamSynchronize(backend->stream);
      if (e != hipSuccess) (void)hipFree(device);
    }
  }
  if (e != hipSuccess) return hipFail(e, (std::string("allocating ") + (label ? label : "buffer")).c_str());
  auto *buffer = new sp_buffer;
  buffer->backend = backend;
  buffer->device = static_cast<char *>(device);
  buffer->host = static_cast<char *>(host);
  buffer->size = buffer->allocated = bytes;
  buffer->storage = storage;
  buffer->label = label ? label : "";
  backend->retain();
  ++backend->liveBuffers;
  {
    std::lock_guard<std::mutex> lock(backend->mutex);
    backend->allocated += bytes;
    backend->peak = std::max(backend->peak, backend->allocated);
    backend->sampleDevice();
  }
  *out = buffer;
  return SP_OK;
}

sp_status sp_buffer_view(sp_buffer *base, uint64_t offset_bytes, uint64_t length_bytes, sp_buffer **out) {
  if (!base || !out) return fail(SP_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  if (!length_bytes || offset_bytes > base->size || length_bytes > base->size - offset_bytes)
    return fail(SP_INVALID_ARGUMENT, "view of " + base->label + " is outside the buffer");
  auto *view = new sp_buffer;
  view->backend = base->backend;
  view->base = const_cast<sp_buffer *>(base->root());
  sp_buffer_retain(view->base);
  view->device = base->device + offset_bytes;
  view->host = base->host ? base->host + offset_bytes : nullptr;
  view->size = length_bytes;
  view->allocated = base->allocated;
  view->storage = base->storage;
  view->label = base->label;
  *out = view;
  return SP_OK;
}

void sp_buffer_retain(sp_buffer *buffer) { if (buffer) ++buffer->refs; }

void sp_buffer_release(sp_buffer *buffer) {
  if (!buffer || --buffer->refs > 0) return;
  if (buffer->base) {
    sp_buffer_release(buffer->base);
    delete buffer;
    return;
  }
  sp_backend *backend = buffer->backend;
  (void)hipSetDevice(backend->device);
  if (buffer->storage == SP_STORAGE_SHARED) (void)hipHostFree(buffer->host);
  else (void)hipFree(buffer->device);
  {
    std::lock_guard<std::mutex> lock(backend->mutex);
    backend->allocated -= buffer->allocated;
  }
  --backend->liveBuffers;
  delete buffer;
  backend->release();
}

uint64_t sp_buffer_size(const sp_buffer *buffer) { return buffer ? buffer->size : 0; }
uint64_t sp_buffer_allocated(const sp_buffer *buffer) { return buffer ? buffer->allocated : 0; }
sp_storage sp_buffer_storage(const sp_buffer *buffer) { return buffer ? buffer->storage : SP_STORAGE_PRIVATE; }
void *sp_buffer_contents(const sp_buffer *buffer) { return buffer ? buffer->host : nullptr; }
uint64_t sp_buffer_gpu_address(const sp_buffer *buffer) { return buffer ? reinterpret_cast<uint64_t>(buffer->device) : 0; }
int sp_buffer_same_view(const sp_buffer *a, const sp_buffer *b) {
  return a && b && a->root() == b->root() && a->device == b->device && a->size == b->size;
}

sp_status sp_buffer_upload(sp_buffer *buffer, uint64_t offset_bytes, const void *source, uint64_t bytes) {
  if (!buffer || (!source && bytes)) return fail(SP_INVALID_ARGUMENT, "null argument");
  if (offset_bytes > buffer->size || bytes > buffer->size - offset_bytes)
    return fail(SP_INVALID_ARGUMENT, "upload outside " + buffer->label);
  if (!bytes) return SP_OK;
  sp_backend *backend = buffer->backend;
  if (!backend->stream) return fail(SP_BACKEND_ERROR, "the backend is destroyed");
  (void)hipSetDevice(backend->device);
  hipError_t e = hipMemcpyAsync(buffer->device + offset_bytes, source, bytes, hipMemcpyHostToDevice, backend->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(backend->stream);
  return e == hipSuccess ? SP_OK : hipFail(e, "upload");
}

sp_status sp_buffer_download(const sp_buffer *buffer, uint64_t offset_bytes, void *destination, uint64_t bytes) {
  if (!buffer || (!destination && bytes)) return fail(SP_INVALID_ARGUMENT, "null argument");
  if (offset_bytes > buffer->size || bytes > buffer->size - offset_bytes)
    return fail(SP_INVALID_ARGUMENT, "download outside " + buffer->label);
  if (!bytes) return SP_OK;
  sp_backend *backend = buffer->backend;
  if (!backend->stream) return fail(SP_BACKEND_ERROR, "the backend is destroyed");
  (void)hipSetDevice(backend->device);
  hipError_t e = hipMemcpyAsync(destination, buffer->device + offset_bytes, bytes, hipMemcpyDeviceToHost, backend->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(backend->stream);
  return e == hipSuccess ? SP_OK : hipFail(e, "download");
}

sp_status sp_buffer_fill(sp_buffer *buffer, uint64_t offset_bytes, int byte_value, uint64_t bytes) {
  if (!buffer) return fail(SP_INVALID_ARGUMENT, "null argument");
  if (offset_bytes > buffer->size || bytes > buffer->size - offset_bytes)
    return fail(SP_INVALID_ARGUMENT, "fill outside " + buffer->label);
  if (!bytes) return SP_OK;
  sp_backend *backend = buffer->backend;
  if (!backend->stream) return fail(SP_BACKEND_ERROR, "the backend is destroyed");
  (void)hipSetDevice(backend->device);
  hipError_t e = hipMemsetAsync(buffer->device + offset_bytes, byte_value, bytes, backend->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(backend->stream);
  return e == hipSuccess ? SP_OK : hipFail(e, "fill");
}

int sp_kernel_exists(const char *name) { return findKernel(name) != nullptr; }

size_t sp_kernel_names(char *out, size_t capacity) {
  std::string all;
  for (const KernelEntry &k : allKernels()) { all += k.name; all += '\n'; }
  if (out && capacity) {
    const size_t n = std::min(capacity - 1, all.size());
    std::memcpy(out, all.data(), n);
    out[n] = 0;
  }
  return all.size() + 1;
}

sp_status sp_submit(sp_backend *backend, const sp_dispatch *dispatches, uint32_t count, sp_completion completion,
                    void *user, sp_ticket **out) {
  if (!out) return fail(SP_INVALID_ARGUMENT, "null result pointer");
  *out = nullptr;
  if (sp_status s = guardSubmit(backend)) return s;
  if (!dispatches && count) return fail(SP_INVALID_ARGUMENT, "null dispatches");
  // Every dispatch is validated before any is launched (the reference's operators and backend
  // throw before anything is encoded).
  std::vector<RecordedDispatch> recorded(count);
  std::vector<sp_buffer *> retained;
  for (uint32_t i = 0; i < count; ++i)
    if (sp_status s = validateDispatch(dispatches[i], i, recorded[i], retained, backend)) return s;
  (void)hipSetDevice(backend->device);
  const bool profile = backend->profiling;
  sp_ticket *ticket = nullptr;
  if (sp_status s = beginTicket(backend, completion, user, profile ? count + 1 : 0, &ticket)) return s;
  ticket->retained = std::move(retained);
  retainAll(ticket->retained);
  ticket->wallStart = Clock::now();
  hipError_t e = hipEventRecord(ticket->start, backend->stream);
  for (uint32_t i = 0; e == hipSuccess && i < count; ++i) {
    if (profile) e = hipEventRecord(ticket->marks[i], backend->stream);
    if (e == hipSuccess) e = launchRecorded(backend, recorded[i]);
  }
  if (e == hipSuccess && profile) e = hipEventRecord(ticket->marks[count], backend->stream);
  if (e == hipSuccess) e = hipEventRecord(ticket->end, backend->stream);
  return finishSubmit(backend, ticket, e, out);
}

int sp_ticket_ready(const sp_ticket *ticket) {
  return !ticket || hipEventQuery(ticket->fence ? ticket->fence : ticket->end) != hipErrorNotReady;
}

sp_status sp_ticket_wait_profiled(sp_ticket *ticket, double *gpu_seconds, double *wall_seconds,
                                  double *dispatch_seconds, uint32_t count) {
  if (!ticket) return fail(SP_INVALID_ARGUMENT, "null ticket");
  sp_backend *backend = ticket->backend;
  (void)hipSetDevice(backend->device);
  sp_status status = awaitTicket(ticket);
  if (status == SP_OK) {
    float ms = 0;
    const hipError_t e = hipEventElapsedTime(&ms, ticket->start, ticket->end);
    if (e != hipSuccess) status = hipFail(e, "hipEventElapsedTime");
    if (gpu_seconds) *gpu_seconds = ms * 1e-3;
    if (wall_seconds) *wall_seconds = std::chrono::duration<double>(Clock::now() - ticket->wallStart).count();
    if (dispatch_seconds)
      for (uint32_t i = 0; i < count; ++i) {
        float dms = 0;
        if (i + 1 < ticket->marks.size() && hipEventElapsedTime(&dms, ticket->marks[i], ticket->marks[i + 1]) == hipSuccess)
          dispatch_seconds[i] = dms * 1e-3;
        else dispatch_seconds[i] = -1.0;
      }
  }
  if (status != SP_TIMEOUT) {
    // A command the watchdog gave up may still run: its buffers stay retained (leaked with the ticket).
    destroyTicket(ticket);
    backend->inFlight = false;
  }
  return status;
}

sp_status sp_ticket_wait(sp_ticket *ticket, double *gpu_seconds, double *wall_seconds) {
  return sp_ticket_wait_profiled(ticket, gpu_seconds, wall_seconds, nullptr, 0);
}

void sp_ticket_release(sp_ticket *ticket) {
  if (ticket) (void)sp_ticket_wait_profiled(ticket, nullptr, nullptr, nullptr, 0);
}

void sp_backend_set_dispatch_profiling(sp_backend *backend, int on) { if (backend) backend->profiling = on != 0; }

sp_status sp_command_create(sp_backend *backend, const sp_dispatch *dispatches, uint32_t count, sp_command **out) {
  if (!out) return fail(SP_INVALID_ARGUMENT, "null result pointer");
  *out = nullptr;
  if (sp_status s = guardSubmit(backend)) return s;
  if (!dispatches || !count) return fail(SP_INVALID_ARGUMENT, "a command needs a dispatch");
  auto *command = new sp_command;
  command->backend = backend;
  command->dispatches.resize(count);
  for (uint32_t i = 0; i < count; ++i)
    if (sp_status s = validateDispatch(dispatches[i], i, command->dispatches[i], command->retained, backend)) {
      delete command;
      return s;
    }
  retainAll(command->retained);
  (void)hipSetDevice(backend->device);
  hipError_t e = hipStreamBeginCapture(backend->stream, hipStreamCaptureModeThreadLocal);
  if (e == hipSuccess) {
    hipError_t launch = hipSuccess;
    for (uint32_t i = 0; launch == hipSuccess && i < count; ++i) launch = launchRecorded(backend, command->dispatches[i]);
    e = hipStreamEndCapture(backend->stream, &command->graph);
    if (launch != hipSuccess) e = launch;
  }
  if (e == hipSuccess) e = hipGraphInstantiate(&command->exec, command->graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    sp_command_release(command);
    return hipFail(e, "recording the command graph");
  }
  *out = command;
  return SP_OK;
}

sp_status sp_command_submit(sp_command *command, sp_completion completion, void *user, sp_ticket **out) {
  if (!command || !out) return fail(SP_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  sp_backend *backend = command->backend;
  if (sp_status s = guardSubmit(backend)) return s;
  (void)hipSetDevice(backend->device);
  sp_ticket *ticket = nullptr;
  if (sp_status s = beginTicket(backend, completion, user, 0, &ticket)) return s;
  ticket->retained = command->retained;
  retainAll(ticket->retained);
  ticket->wallStart = Clock::now();
  hipError_t e = hipEventRecord(ticket->start, backend->stream);
  if (e == hipSuccess) e = hipGraphLaunch(command->exec, backend->stream);
  if (e == hipSuccess) e = hipEventRecord(ticket->end, backend->stream);
  return finishSubmit(backend, ticket, e, out);
}

void sp_command_release(sp_command *command) {
  if (!command) return;
  (void)hipSetDevice(command->backend->device);
  if (command->exec) (void)hipGraphExecDestroy(command->exec);
  if (command->graph) (void)hipGraphDestroy(command->graph);
  releaseAll(command->retained);
  delete command;
}

int sp_command_in_flight(const sp_backend *backend) { return backend && backend->inFlight; }
int sp_backend_healthy(const sp_backend *backend) { return backend && backend->healthy; }

sp_status sp_backend_check_health(sp_backend *backend) {
  if (!backend) return fail(SP_INVALID_ARGUMENT, "null backend");
  if (!backend->healthy) return fail(SP_UNHEALTHY, "the backend is unhealthy");
  return SP_OK;
}

size_t sp_backend_unhealthy_reason(const sp_backend *backend, char *out, size_t capacity) {
  if (!backend) return 0;
  std::lock_guard<std::mutex> lock(backend->mutex);
  if (out && capacity) {
    const size_t n = std::min(capacity - 1, backend->reason.size());
    std::memcpy(out, backend->reason.data(), n);
    out[n] = 0;
  }
  return backend->reason.size() + 1;
}

sp_status sp_memory_stats(const sp_backend *backend, sp_memory_stats_t *out) {
  if (!backend || !out) return fail(SP_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(backend->mutex);
  out->allocated_bytes = backend->allocated;
  out->peak_allocated_bytes = backend->peak;
  out->device_current_allocated_bytes = backend->deviceCurrent;
  out->device_peak_allocated_bytes = backend->devicePeak;
  return SP_OK;
}

void sp_restart_peaks(sp_backend *backend) {
  if (!backend) return;
  std::lock_guard<std::mutex> lock(backend->mutex);
  backend->sampleDevice();
  backend->peak = backend->allocated;
  backend->devicePeak = backend->deviceCurrent;
}

void *sp_backend_stream(sp_backend *backend) { return backend ? backend->stream : nullptr; }

} // extern "C"
