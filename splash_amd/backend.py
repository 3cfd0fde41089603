"""Backend, Buffer and CommandGraph over the C ABI (include/splash_hip.h), with the method names of
the reference's MetalBackend / MetalBuffer / CommandGraph (runtime/metal/MetalBackend.hpp,
CommandGraph.hpp)."""
import ctypes

import numpy as np

from . import _native as nat
from ._native import lib, check

STORAGE_SHARED, STORAGE_PRIVATE = 0, 1


class Buffer:
    """MetalBuffer: a handle of backend-owned memory; views keep the base alive."""

    def __init__(self, handle):
        self.handle = ctypes.c_void_p(handle)

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                lib.sp_buffer_release(self.handle)
        except Exception:
            pass

    @property
    def size_bytes(self):
        return lib.sp_buffer_size(self.handle)

    @property
    def gpu_address(self):
        return lib.sp_buffer_gpu_address(self.handle)

    @property
    def storage(self):
        return lib.sp_buffer_storage(self.handle)

    def contents(self):
        """Host view (numpy uint8) of a Shared buffer; None for Private."""
        p = lib.sp_buffer_contents(self.handle)
        if not p:
            return None
        return np.ctypeslib.as_array((ctypes.c_uint8 * self.size_bytes).from_address(p))

    def view(self, offset_bytes, length_bytes):
        out = ctypes.c_void_p()
        check(lib.sp_buffer_view(self.handle, offset_bytes, length_bytes, ctypes.byref(out)))
        return Buffer(out.value)

    def same_view(self, other):
        return bool(lib.sp_buffer_same_view(self.handle, other.handle))

    def upload(self, array, offset_bytes=0):
        a = np.ascontiguousarray(array)
        check(lib.sp_buffer_upload(self.handle, offset_bytes, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype=np.uint8, count=None, offset_bytes=0):
        dtype = np.dtype(dtype)
        if count is None:
            count = (self.size_bytes - offset_bytes) // dtype.itemsize
        out = np.empty(count, dtype=dtype)
        check(lib.sp_buffer_download(self.handle, offset_bytes, out.ctypes.data, out.nbytes))
        return out

    def fill(self, byte=0, offset_bytes=0, length_bytes=None):
        n = self.size_bytes - offset_bytes if length_bytes is None else length_bytes
        check(lib.sp_buffer_fill(self.handle, offset_bytes, byte, n))
        return self


class CommandGraph:
    """metal::CommandGraph: an ordered list of named dispatches."""

    def __init__(self):
        h = ctypes.c_void_p()
        check(lib.spo_graph_create(ctypes.byref(h)))
        self.handle = h
        self._keep = []

    def __del__(self):
        try:
            lib.spo_graph_destroy(self.handle)
        except Exception:
            pass

    def __len__(self):
        return lib.spo_graph_size(self.handle)

    def kernels(self):
        names = []
        for i in range(len(self)):
            n = lib.spo_graph_kernel(self.handle, i, None, 0)
            buf = ctypes.create_string_buffer(n)
            lib.spo_graph_kernel(self.handle, i, buf, n)
            names.append(buf.value.decode())
        return names

    def add(self, kernel, buffers, params, groups, threads=(256, 1, 1)):
        """CommandGraph::add(pipeline, buffers, params, groups, threads): params is a ctypes struct."""
        arr = (ctypes.c_void_p * len(buffers))(*[b.handle for b in buffers])
        grid = (ctypes.c_uint32 * 3)(*groups)
        block = (ctypes.c_uint32 * 3)(*threads)
        check(lib.spo_graph_add(self.handle, kernel.encode(), arr, len(buffers), ctypes.byref(params),
                                ctypes.sizeof(params), grid, block))
        self._keep.extend(buffers)


class Ticket:
    def __init__(self, handle, count=0):
        self.handle = ctypes.c_void_p(handle)
        self.count = count

    def ready(self):
        return bool(lib.sp_ticket_ready(self.handle))

    def wait(self, profiled=False):
        """CommandTicket::wait -> (gpu_seconds, wall_seconds[, per-dispatch seconds])."""
        gpu, wall = ctypes.c_double(), ctypes.c_double()
        h, self.handle = self.handle, None
        if profiled:
            per = (ctypes.c_double * max(1, self.count))()
            check(lib.sp_ticket_wait_profiled(h, ctypes.byref(gpu), ctypes.byref(wall), per, self.count))
            return gpu.value, wall.value, list(per)[:self.count]
        check(lib.sp_ticket_wait(h, ctypes.byref(gpu), ctypes.byref(wall)))
        return gpu.value, wall.value

    def __del__(self):
        try:
            if self.handle:
                lib.sp_ticket_release(self.handle)
        except Exception:
            pass


class RecordedCommand:
    """A command graph recorded once into a HIP graph and replayed."""

    def __init__(self, handle, graph):
        self.handle = ctypes.c_void_p(handle)
        self._graph = graph

    def submit(self):
        t = ctypes.c_void_p()
        check(lib.sp_command_submit(self.handle, None, None, ctypes.byref(t)))
        return Ticket(t.value)

    def __del__(self):
        try:
            lib.sp_command_release(self.handle)
        except Exception:
            pass


class Backend:
    """MetalBackend for one HIP device: allocate, view, submit one command at a time."""

    def __init__(self, device=0, command_timeout_seconds=0.0):
        h = ctypes.c_void_p()
        check(lib.sp_backend_create(device, command_timeout_seconds, ctypes.byref(h)))
        self.handle = h

    def close(self):
        if self.handle:
            lib.sp_backend_destroy(self.handle)
            self.handle = None

    def device_info(self):
        info = nat.DeviceInfo()
        check(lib.sp_backend_device_info(self.handle, ctypes.byref(info)))
        return info

    def allocate_buffer(self, nbytes, storage=STORAGE_PRIVATE, label="buffer"):
        out = ctypes.c_void_p()
        check(lib.sp_buffer_alloc(self.handle, int(nbytes), storage, label.encode(), ctypes.byref(out)))
        return Buffer(out.value)

    def from_array(self, array, storage=STORAGE_PRIVATE, label="array"):
        a = np.ascontiguousarray(array)
        b = self.allocate_buffer(max(a.nbytes, 1), storage, label)
        if a.nbytes:
            b.upload(a)
        return b

    def submit_command_async(self, graph):
        t = ctypes.c_void_p()
        check(lib.spo_graph_submit(self.handle, graph.handle, ctypes.byref(t)))
        return Ticket(t.value, len(graph))

    def run(self, graph, profiled=False):
        return self.submit_command_async(graph).wait(profiled=profiled)

    def record(self, graph):
        c = ctypes.c_void_p()
        check(lib.spo_graph_record(self.handle, graph.handle, ctypes.byref(c)))
        return RecordedCommand(c.value, graph)

    def set_dispatch_profiling(self, on):
        lib.sp_backend_set_dispatch_profiling(self.handle, int(bool(on)))

    def memory_stats(self):
        s = nat.MemoryStats()
        check(lib.sp_memory_stats(self.handle, ctypes.byref(s)))
        return s

    def healthy(self):
        return bool(lib.sp_backend_healthy(self.handle))

    def unhealthy_reason(self):
        n = lib.sp_backend_unhealthy_reason(self.handle, None, 0)
        buf = ctypes.create_string_buffer(max(n, 1))
        lib.sp_backend_unhealthy_reason(self.handle, buf, n)
        return buf.value.decode()

    def command_in_flight(self):
        return bool(lib.sp_command_in_flight(self.handle))
