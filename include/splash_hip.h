/* splash_hip.h -- C ABI of the MI355X (gfx950) backend for Splash's speculative-decoding verify step.
 *
 * This is the drop-in boundary: it replaces, for the verify-step operators, what the reference's
 * operators get from splash::metal::MetalBackend and metal::CommandGraph
 * (runtime/metal/MetalBackend.hpp:371-547, runtime/metal/CommandGraph.hpp:26-143): buffers and
 * views, an ordered list of dispatches that name their kernels, one asynchronous command in
 * flight, a ticket that reports GPU and wall time, and a sticky health state. Plain pointers and
 * sizes only; no C++ or framework types cross it.
 *
 * Threading follows the reference (MetalBackend.hpp:371-375): one thread allocates and submits;
 * sp_backend_healthy, sp_backend_unhealthy_reason, sp_backend_check_health, sp_memory_stats and
 * sp_command_in_flight may be called from any thread.
 */
#ifndef SPLASH_HIP_H
#define SPLASH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct sp_backend sp_backend;
typedef struct sp_buffer sp_buffer;
typedef struct sp_ticket sp_ticket;
typedef struct sp_command sp_command;

typedef enum sp_status {
  SP_OK = 0,
  SP_INVALID_ARGUMENT = 1, /* std::invalid_argument of the reference's operators and backend */
  SP_BACKEND_ERROR = 2,    /* MetalBackendError: a HIP call or a command failed */
  SP_UNHEALTHY = 3,        /* the backend refused because it is unhealthy (sticky) */
  SP_BUSY = 4,             /* a second command while one is in flight (MetalBackend.hpp:474-476) */
  SP_OUT_OF_MEMORY = 5,
  SP_UNKNOWN_KERNEL = 6,   /* no kernel of that name (a pipeline lookup that fails) */
  SP_TIMEOUT = 7           /* the command watchdog gave the command up (CommandWatchdog.hpp:16-44) */
} sp_status;

/* BufferStorage (MetalBackend.hpp:23-26). Shared: host-visible pinned memory the GPU reads over
 * the bus, for small control data and results. Private: HBM; contents() is NULL. */
typedef enum sp_storage { SP_STORAGE_SHARED = 0, SP_STORAGE_PRIVATE = 1 } sp_storage;

/* The message of the calling thread's last failed call ("" when none). */
const char *sp_last_error(void);

/* MetalBackend::MetalBackend (MetalBackend.hpp:383-385): opens `device`, creates the command stream.
 * command_timeout_seconds <= 0 takes the default of 120 s (runtime/Supervision.hpp:41). */
sp_status sp_backend_create(int device, double command_timeout_seconds, sp_backend **out);
void sp_backend_destroy(sp_backend *backend);
/* MetalBackend::stop (MetalBackend.hpp:395): refuses new submissions. */
void sp_backend_stop(sp_backend *backend);
/* DeviceCapabilities (runtime/metal/DeviceCapabilities.hpp): what plans read of the device. */
typedef struct sp_device_info {
  char name[64];
  char arch[32];
  uint32_t compute_units;
  uint32_t wavefront_size;
  uint32_t lds_bytes_per_cu;
  uint32_t l2_bytes;
  uint64_t hbm_bytes;
  uint32_t clock_khz;
  uint32_t memory_clock_khz;
  uint32_t memory_bus_bits;
} sp_device_info;
sp_status sp_backend_device_info(sp_backend *backend, sp_device_info *out);

/* MetalBackend::allocateBuffer (MetalBackend.hpp:417-420). Memory is zeroed. */
sp_status sp_buffer_alloc(sp_backend *backend, uint64_t bytes, sp_storage storage, const char *label,
                          sp_buffer **out);
/* MetalBackend::view (MetalBackend.hpp:435-436): keeps the base alive, adds no tracked bytes. */
sp_status sp_buffer_view(sp_buffer *base, uint64_t offset_bytes, uint64_t length_bytes, sp_buffer **out);
/* MetalBuffer copies are reference counts across the ABI (MetalBackend.hpp:42-78). */
void sp_buffer_retain(sp_buffer *buffer);
void sp_buffer_release(sp_buffer *buffer);
uint64_t sp_buffer_size(const sp_buffer *buffer);      /* MetalBuffer::sizeBytes */
uint64_t sp_buffer_allocated(const sp_buffer *buffer); /* MetalBuffer::allocatedBytes */
sp_storage sp_buffer_storage(const sp_buffer *buffer); /* MetalBuffer::storage */
void *sp_buffer_contents(const sp_buffer *buffer);     /* MetalBuffer::contents; NULL for Private */
uint64_t sp_buffer_gpu_address(const sp_buffer *buffer); /* MetalBuffer::gpuAddress */
int sp_buffer_same_view(const sp_buffer *a, const sp_buffer *b); /* MetalBuffer::sameView */
/* Host <-> HBM copies for Private buffers, ordered after the command stream's work and complete on
 * return. The reference needs none (unified memory); a discrete GPU's loader and tests do. */
sp_status sp_buffer_upload(sp_buffer *buffer, uint64_t offset_bytes, const void *source, uint64_t bytes);
sp_status sp_buffer_download(const sp_buffer *buffer, uint64_t offset_bytes, void *destination, uint64_t bytes);
sp_status sp_buffer_fill(sp_buffer *buffer, uint64_t offset_bytes, int byte_value, uint64_t bytes);

/* ComputeDispatch (MetalBackend.hpp:156-169) as CommandGraph::add builds it (CommandGraph.hpp:37-54):
 * buffers bind at indices 0..n-1, the parameter struct after them; both are copied by sp_submit and
 * sp_command_create, so they only need to live until the call returns (MetalBackend.hpp:123-128).
 * indirect (optional): three uint32 workgroup counts the GPU reads as the dispatch starts
 * (IndirectGrid, MetalBackend.hpp:131-139); `grid` is then their upper bound and kernels exit early. */
typedef struct sp_dispatch {
  const char *kernel;
  uint32_t buffer_count;
  sp_buffer *const *buffers;
  const void *params;
  uint32_t params_bytes;
  uint32_t grid[3];  /* workgroups */
  uint32_t block[3]; /* threads per workgroup */
  sp_buffer *indirect;
  uint64_t indirect_offset;
} sp_dispatch;

/* 1 when a kernel of that name is registered (MetalBackend::preparePipelines' lookup). */
int sp_kernel_exists(const char *name);
/* Names of every registered kernel, one per line; returns the bytes needed (with the final NUL). */
size_t sp_kernel_names(char *out, size_t capacity);

/* MetalBackend::submitCommandAsync (MetalBackend.hpp:487-491): validates every dispatch before
 * launching any, then launches them in order on the command stream without waiting. `completion`
 * (optional) only notifies, from a runtime thread, once the command has completed.
 * SP_BUSY while an earlier ticket has not been consumed by sp_ticket_wait. */
typedef void (*sp_completion)(void *user);
sp_status sp_submit(sp_backend *backend, const sp_dispatch *dispatches, uint32_t count, sp_completion completion,
                    void *user, sp_ticket **out);
/* CommandTicket::ready / wait (MetalBackend.hpp:293-320). sp_ticket_wait consumes and frees the
 * ticket; its status is the command's. sp_ticket_release waits, then frees (the destructor). */
int sp_ticket_ready(const sp_ticket *ticket);
sp_status sp_ticket_wait(sp_ticket *ticket, double *gpu_seconds, double *wall_seconds);
void sp_ticket_release(sp_ticket *ticket);

/* BackendInstrumentation::setDispatchProfiling (runtime/metal/BackendInstrumentation.hpp:23-37):
 * while on, every dispatch of a submitted command is bracketed by its own event pair and
 * sp_ticket_dispatch_seconds reports each one's GPU time (call it before sp_ticket_wait's free:
 * pass `seconds` of `count` entries to sp_ticket_wait_profiled). */
void sp_backend_set_dispatch_profiling(sp_backend *backend, int on);
sp_status sp_ticket_wait_profiled(sp_ticket *ticket, double *gpu_seconds, double *wall_seconds,
                                  double *dispatch_seconds, uint32_t count);

/* A command recorded once into a HIP graph and replayed: the launch-bound inner loop of a decode
 * cycle (the reference re-encodes its command each cycle, Runtime.cpp:3985-4006; on HIP a replay
 * costs one graph launch). The command keeps its buffers alive. sp_command_submit is
 * sp_submit of the recorded dispatches. */
sp_status sp_command_create(sp_backend *backend, const sp_dispatch *dispatches, uint32_t count, sp_command **out);
sp_status sp_command_submit(sp_command *command, sp_completion completion, void *user, sp_ticket **out);
void sp_command_release(sp_command *command);

/* MetalBackend::commandInFlight / healthy / checkHealth / unhealthyReason (MetalBackend.hpp:531-542). */
int sp_command_in_flight(const sp_backend *backend);
int sp_backend_healthy(const sp_backend *backend);
sp_status sp_backend_check_health(sp_backend *backend);
/* Copies the reason (empty when healthy); returns the bytes needed. */
size_t sp_backend_unhealthy_reason(const sp_backend *backend, char *out, size_t capacity);

/* MetalMemoryStats (MetalBackend.hpp:335-352). */
typedef struct sp_memory_stats_t {
  uint64_t allocated_bytes;
  uint64_t peak_allocated_bytes;
  uint64_t device_current_allocated_bytes;
  uint64_t device_peak_allocated_bytes;
} sp_memory_stats_t;
sp_status sp_memory_stats(const sp_backend *backend, sp_memory_stats_t *out);
void sp_restart_peaks(sp_backend *backend);

/* The raw HIP stream of the backend (hipStream_t), for callers that time with their own events. */
void *sp_backend_stream(sp_backend *backend);

#ifdef __cplusplus
}
#endif
#endif /* SPLASH_HIP_H */
