// C++ value types over the C ABI of include/splash_hip.h, with the method shapes of the
// reference's splash::metal::MetalBuffer, CommandGraph, CommandTicket and MetalBackend
// (runtime/metal/MetalBackend.hpp, CommandGraph.hpp), so the operators above them keep the
// reference's signatures with hip:: in place of metal::. Status codes of the C ABI come back as the
// exception types the reference throws: std::invalid_argument from validation, BackendError
// (MetalBackendError) from the device.
#pragma once
#include "splash_hip.h"

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <deque>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <string_view>
#include <type_traits>
#include <utility>
#include <vector>

namespace splash::hip {

class BackendError : public std::runtime_error {
public:
  using std::runtime_error::runtime_error;
};

inline void throwStatus(sp_status status) {
  if (status == SP_OK) return;
  const std::string message = sp_last_error();
  if (status == SP_INVALID_ARGUMENT || status == SP_UNKNOWN_KERNEL) throw std::invalid_argument(message);
  throw BackendError(message);
}

enum class BufferStorage { Shared, Private };

class Backend;

// MetalBuffer (MetalBackend.hpp:42-78): a cheap copyable handle; views keep the base alive.
class Buffer final {
public:
  Buffer() = default;
  [[nodiscard]] explicit operator bool() const noexcept { return static_cast<bool>(handle_); }
  [[nodiscard]] uint64_t sizeBytes() const noexcept { return sp_buffer_size(handle_.get()); }
  [[nodiscard]] uint64_t allocatedBytes() const noexcept { return sp_buffer_allocated(handle_.get()); }
  [[nodiscard]] BufferStorage storage() const noexcept {
    return sp_buffer_storage(handle_.get()) == SP_STORAGE_SHARED ? BufferStorage::Shared : BufferStorage::Private;
  }
  [[nodiscard]] void *contents() const noexcept { return sp_buffer_contents(handle_.get()); }
  [[nodiscard]] uint64_t gpuAddress() const { return sp_buffer_gpu_address(handle_.get()); }
  [[nodiscard]] bool sameView(const Buffer &other) const noexcept {
    return sp_buffer_same_view(handle_.get(), other.handle_.get()) != 0;
  }
  [[nodiscard]] sp_buffer *handle() const noexcept { return handle_.get(); }
  // Host <-> HBM copies (Private storage has no contents()).
  void upload(const void *source, uint64_t bytes, uint64_t offset = 0) const {
    throwStatus(sp_buffer_upload(handle_.get(), offset, source, bytes));
  }
  void download(void *destination, uint64_t bytes, uint64_t offset = 0) const {
    throwStatus(sp_buffer_download(handle_.get(), offset, destination, bytes));
  }
  void fill(int byte, uint64_t bytes, uint64_t offset = 0) const {
    throwStatus(sp_buffer_fill(handle_.get(), offset, byte, bytes));
  }
  // Bytes [offset, offset + length) of this buffer as a buffer of their own; the view keeps the base alive.
  [[nodiscard]] Buffer slice(uint64_t offsetBytes, uint64_t lengthBytes) const {
    sp_buffer *raw = nullptr;
    throwStatus(sp_buffer_view(handle_.get(), offsetBytes, lengthBytes, &raw));
    return adopt(raw);
  }
  // Adopts a handle the caller owns one reference of.
  static Buffer adopt(sp_buffer *raw) {
    Buffer b;
    b.handle_ = std::shared_ptr<sp_buffer>(raw, [](sp_buffer *p) { sp_buffer_release(p); });
    return b;
  }
  // Shares a handle someone else owns (takes its own reference).
  static Buffer share(sp_buffer *raw) {
    if (!raw) return {};
    sp_buffer_retain(raw);
    return adopt(raw);
  }

private:
  std::shared_ptr<sp_buffer> handle_;
};

struct DispatchSize {
  uint64_t x = 1, y = 1, z = 1;
};

// ComputeDispatch (MetalBackend.hpp:156-169).
struct ComputeDispatch {
  std::string pipelineName;
  std::vector<Buffer> buffers;   // bind 0..n-1
  const void *bytes = nullptr;   // the parameter struct, bound after the buffers
  uint32_t bytesSize = 0;
  DispatchSize threadgroups;
  DispatchSize threadsPerThreadgroup;
};

// CommandGraph (CommandGraph.hpp:26-143): an ordered dispatch list; parameter structs are copied
// into graph-owned storage until submission.
class CommandGraph final {
public:
  static constexpr uint32_t kDefaultThreads = 256;
  CommandGraph() = default;
  CommandGraph(const CommandGraph &) = delete;
  CommandGraph &operator=(const CommandGraph &) = delete;
  CommandGraph(CommandGraph &&) noexcept = default;
  CommandGraph &operator=(CommandGraph &&) noexcept = default;

  template <class Params>
  void add(std::string pipeline, std::vector<Buffer> buffers, const Params &params, DispatchSize groups,
           DispatchSize threads = {kDefaultThreads, 1, 1}) {
    static_assert(std::is_trivially_copyable_v<Params>, "dispatch parameters must be plain data");
    payloads_.emplace_back(sizeof(Params));
    std::memcpy(payloads_.back().data(), &params, sizeof(Params));
    ComputeDispatch dispatch;
    dispatch.pipelineName = std::move(pipeline);
    dispatch.buffers = std::move(buffers);
    dispatch.bytes = payloads_.back().data();
    dispatch.bytesSize = sizeof(Params);
    dispatch.threadgroups = groups;
    dispatch.threadsPerThreadgroup = threads;
    dispatches_.push_back(std::move(dispatch));
  }
  [[nodiscard]] bool empty() const noexcept { return dispatches_.empty(); }
  [[nodiscard]] const std::vector<ComputeDispatch> &dispatches() const noexcept { return dispatches_; }
  [[nodiscard]] size_t size() const noexcept { return dispatches_.size(); }

private:
  std::deque<std::vector<std::byte>> payloads_;
  std::vector<ComputeDispatch> dispatches_;
};

struct CommandTiming {
  double gpuSeconds = 0.0;
  double wallSeconds = 0.0;
};

// CommandTicket (MetalBackend.hpp:293-320): move-only; destroying an unfinished ticket waits.
class CommandTicket final {
public:
  CommandTicket() = default;
  explicit CommandTicket(sp_ticket *ticket) : ticket_(ticket) {}
  ~CommandTicket() { if (ticket_) sp_ticket_release(ticket_); }
  CommandTicket(const CommandTicket &) = delete;
  CommandTicket &operator=(const CommandTicket &) = delete;
  CommandTicket(CommandTicket &&other) noexcept : ticket_(std::exchange(other.ticket_, nullptr)) {}
  CommandTicket &operator=(CommandTicket &&other) noexcept {
    if (this != &other) {
      if (ticket_) sp_ticket_release(ticket_);
      ticket_ = std::exchange(other.ticket_, nullptr);
    }
    return *this;
  }
  [[nodiscard]] bool ready() const noexcept { return sp_ticket_ready(ticket_) != 0; }
  [[nodiscard]] CommandTiming wait() {
    if (!ticket_) throw std::logic_error("the ticket holds no command");
    CommandTiming timing;
    sp_ticket *ticket = std::exchange(ticket_, nullptr);
    throwStatus(sp_ticket_wait(ticket, &timing.gpuSeconds, &timing.wallSeconds));
    return timing;
  }
  // wait() with each dispatch's GPU time (dispatch profiling on).
  [[nodiscard]] CommandTiming wait(std::vector<double> &dispatchSeconds) {
    if (!ticket_) throw std::logic_error("the ticket holds no command");
    CommandTiming timing;
    sp_ticket *ticket = std::exchange(ticket_, nullptr);
    throwStatus(sp_ticket_wait_profiled(ticket, &timing.gpuSeconds, &timing.wallSeconds, dispatchSeconds.data(),
                                        uint32_t(dispatchSeconds.size())));
    return timing;
  }

private:
  sp_ticket *ticket_ = nullptr;
};

using CommandCompletion = std::function<void()>;

struct MemoryStats {
  uint64_t allocatedBytes = 0, peakAllocatedBytes = 0, deviceCurrentAllocatedBytes = 0, devicePeakAllocatedBytes = 0;
};

// Lowers a C++ dispatch list to the C ABI's records; keeps the handle arrays alive.
struct LoweredDispatches {
  std::vector<std::vector<sp_buffer *>> handles;
  std::vector<sp_dispatch> records;
  explicit LoweredDispatches(const std::vector<ComputeDispatch> &dispatches) {
    handles.reserve(dispatches.size());
    records.reserve(dispatches.size());
    for (const ComputeDispatch &d : dispatches) {
      handles.emplace_back();
      for (const Buffer &b : d.buffers) handles.back().push_back(b.handle());
      sp_dispatch r{};
      r.kernel = d.pipelineName.c_str();
      r.buffer_count = uint32_t(handles.back().size());
      r.buffers = handles.back().data();
      r.params = d.bytes;
      r.params_bytes = d.bytesSize;
      r.grid[0] = uint32_t(d.threadgroups.x); r.grid[1] = uint32_t(d.threadgroups.y); r.grid[2] = uint32_t(d.threadgroups.z);
      r.block[0] = uint32_t(d.threadsPerThreadgroup.x); r.block[1] = uint32_t(d.threadsPerThreadgroup.y);
      r.block[2] = uint32_t(d.threadsPerThreadgroup.z);
      records.push_back(r);
    }
  }
};

// A command recorded once and replayed (sp_command).
class RecordedCommand final {
public:
  RecordedCommand() = default;
  explicit RecordedCommand(sp_command *command) : command_(command, [](sp_command *c) { sp_command_release(c); }) {}
  [[nodiscard]] explicit operator bool() const noexcept { return static_cast<bool>(command_); }
  [[nodiscard]] CommandTicket submit() const {
    sp_ticket *ticket = nullptr;
    throwStatus(sp_command_submit(command_.get(), nullptr, nullptr, &ticket));
    return CommandTicket(ticket);
  }

private:
  std::shared_ptr<sp_command> command_;
};

// MetalBackend (MetalBackend.hpp:371-547), the part the verify step's operators use.
class Backend final {
public:
  explicit Backend(int device = 0, double commandTimeoutSeconds = 0.0) {
    throwStatus(sp_backend_create(device, commandTimeoutSeconds, &backend_));
  }
  // Wraps a backend the caller owns.
  explicit Backend(sp_backend *borrowed) : backend_(borrowed), owned_(false) {}
  ~Backend() { if (owned_) sp_backend_destroy(backend_); }
  Backend(const Backend &) = delete;
  Backend &operator=(const Backend &) = delete;

  [[nodiscard]] Buffer allocateBuffer(uint64_t bytes, BufferStorage storage, std::string_view label) const {
    sp_buffer *raw = nullptr;
    const std::string name(label);
    throwStatus(sp_buffer_alloc(backend_, bytes, storage == BufferStorage::Shared ? SP_STORAGE_SHARED : SP_STORAGE_PRIVATE,
                                name.c_str(), &raw));
    return Buffer::adopt(raw);
  }
  [[nodiscard]] Buffer view(const Buffer &base, uint64_t offsetBytes, uint64_t lengthBytes) const {
    sp_buffer *raw = nullptr;
    throwStatus(sp_buffer_view(base.handle(), offsetBytes, lengthBytes, &raw));
    return Buffer::adopt(raw);
  }
  [[nodiscard]] CommandTicket submitCommandAsync(const std::vector<ComputeDispatch> &dispatches,
                                                 CommandCompletion completion = {}) {
    LoweredDispatches lowered(dispatches);
    sp_ticket *ticket = nullptr;
    completion_ = std::move(completion);
    throwStatus(sp_submit(backend_, lowered.records.data(), uint32_t(lowered.records.size()),
                          completion_ ? &Backend::notify : nullptr, this, &ticket));
    return CommandTicket(ticket);
  }
  [[nodiscard]] CommandTiming submit(const ComputeDispatch &dispatch) {
    return submitCommandAsync(std::vector<ComputeDispatch>{dispatch}).wait();
  }
  [[nodiscard]] RecordedCommand record(const std::vector<ComputeDispatch> &dispatches) const {
    LoweredDispatches lowered(dispatches);
    sp_command *command = nullptr;
    throwStatus(sp_command_create(backend_, lowered.records.data(), uint32_t(lowered.records.size()), &command));
    return RecordedCommand(command);
  }
  void preparePipelines(const std::vector<ComputeDispatch> &dispatches) const {
    for (const ComputeDispatch &d : dispatches)
      if (!sp_kernel_exists(d.pipelineName.c_str())) throw std::invalid_argument("no kernel named " + d.pipelineName);
  }
  void setDispatchProfiling(bool on) const { sp_backend_set_dispatch_profiling(backend_, on); }
  [[nodiscard]] MemoryStats memoryStats() const {
    sp_memory_stats_t s{};
    throwStatus(sp_memory_stats(backend_, &s));
    return {s.allocated_bytes, s.peak_allocated_bytes, s.device_current_allocated_bytes, s.device_peak_allocated_bytes};
  }
  [[nodiscard]] sp_device_info deviceInfo() const {
    sp_device_info info{};
    throwStatus(sp_backend_device_info(backend_, &info));
    return info;
  }
  [[nodiscard]] bool commandInFlight() const noexcept { return sp_command_in_flight(backend_) != 0; }
  [[nodiscard]] bool healthy() const noexcept { return sp_backend_healthy(backend_) != 0; }
  void checkHealth() const { throwStatus(sp_backend_check_health(backend_)); }
  [[nodiscard]] std::string unhealthyReason() const {
    std::string reason(sp_backend_unhealthy_reason(backend_, nullptr, 0), '\0');
    sp_backend_unhealthy_reason(backend_, reason.data(), reason.size());
    reason.resize(reason.empty() ? 0 : reason.size() - 1);
    return reason;
  }
  [[nodiscard]] sp_backend *handle() const noexcept { return backend_; }

private:
  static void notify(void *self) {
    auto *backend = static_cast<Backend *>(self);
    if (backend->completion_) backend->completion_();
  }
  sp_backend *backend_ = nullptr;
  bool owned_ = true;
  CommandCompletion completion_;
};

} // namespace splash::hip
