"""Python mirror of the verify step's operators (splash::ops::*), bound through include/splash_ops.h.
Names follow the reference's operators (runtime/ops/Linear.hpp, Weights.hpp)."""
import ctypes

import numpy as np

from . import _native as nat
from ._native import lib, check
from .backend import Buffer, STORAGE_PRIVATE

FMT_Q4K, FMT_Q6K = 0, 4
EPILOGUE_NONE, EPILOGUE_RESIDUAL, EPILOGUE_GATE_UP = 0, 1, 2


def gguf_image_bytes(fmt, rows, input_size):
    return lib.spo_gguf_image_bytes(fmt, rows, input_size)


def gguf_table_bytes(input_size, rows):
    return lib.spo_gguf_table_bytes(input_size, rows)


def pack_gguf_image(fmt, native, rows, input_size):
    """Native GGUF rows (uint8) -> the weight image (load-time repack)."""
    native = np.ascontiguousarray(native, dtype=np.uint8)
    image = np.empty(native.size, dtype=np.uint8)
    check(lib.spo_gguf_pack_image(fmt, native.ctypes.data, rows, input_size, image.ctypes.data))
    return image


def unpack_gguf_image(fmt, image, rows, input_size):
    image = np.ascontiguousarray(image, dtype=np.uint8)
    native = np.empty(image.size, dtype=np.uint8)
    check(lib.spo_gguf_unpack_image(fmt, image.ctypes.data, rows, input_size, native.ctypes.data))
    return native


def add_dequant(graph, fmt, image, out, rows, input_size):
    check(lib.spo_gguf_add_dequant(graph.handle, fmt, image.handle, out.handle, rows, input_size))
    graph._keep.extend([image, out])


class Projection:
    """ops::Projection: column segments (format, output size, image buffer) over one input size."""

    def __init__(self, segments, input_size, float32=False):
        n = len(segments)
        fmts = (ctypes.c_uint32 * n)(*[s[0] for s in segments])
        outs = (ctypes.c_uint32 * n)(*[s[1] for s in segments])
        imgs = (ctypes.c_void_p * n)(*[s[2].handle for s in segments])
        h = ctypes.c_void_p()
        check(lib.spo_projection_create(n, fmts, outs, input_size, imgs, int(float32), ctypes.byref(h)))
        self.handle = h
        self.segments = segments
        self.input_size = input_size
        self.output_size = sum(s[1] for s in segments)
        self.float32 = float32

    @classmethod
    def from_native(cls, backend, segments, input_size, float32=False):
        """segments: [(fmt, rows, native uint8 array)]; packs and uploads each image."""
        built = []
        for fmt, rows, native in segments:
            image = pack_gguf_image(fmt, native, rows, input_size)
            built.append((fmt, rows, backend.from_array(image, STORAGE_PRIVATE, "weight image")))
        return cls(built, input_size, float32)

    @property
    def weight_bytes(self):
        return lib.spo_projection_weight_bytes(self.handle)

    def __del__(self):
        try:
            lib.spo_projection_destroy(self.handle)
        except Exception:
            pass


class LinearScratch:
    """ops::LinearScratch: activation table, split partials and counters (counters zeroed)."""

    def __init__(self, backend, table_bytes, partials_bytes=0, counters_bytes=0):
        self.table = backend.allocate_buffer(max(table_bytes, 16), STORAGE_PRIVATE, "linear table")
        self.partials = backend.allocate_buffer(max(partials_bytes, 16), STORAGE_PRIVATE, "linear partials")
        self.counters = backend.allocate_buffer(max(counters_bytes, 16), STORAGE_PRIVATE, "linear counters")


class Linear:
    """ops::Linear: plans and dispatches quantized projections."""

    def __init__(self, backend=None, calibration=None):
        h = ctypes.c_void_p()
        if calibration is not None:
            check(lib.spo_linear_create_calibrated(*calibration, ctypes.byref(h)))
        else:
            check(lib.spo_linear_create(backend.handle, ctypes.byref(h)))
        self.handle = h

    def __del__(self):
        try:
            lib.spo_linear_destroy(self.handle)
        except Exception:
            pass

    def plan(self, projection, rows, epilogue=EPILOGUE_NONE, splits=None, k_waves=None):
        p = nat.LinearPlan()
        check(lib.spo_linear_plan_for(self.handle, projection.handle, rows, epilogue, ctypes.byref(p)))
        if splits is not None or k_waves is not None:
            if splits is not None:
                p.splits = splits
            if k_waves is not None:
                p.k_waves = k_waves
            check(lib.spo_linear_plan_with(projection.handle, ctypes.byref(p)))
        return p

    def scratch_for(self, backend, plans):
        t = max(p.scratch_input for p in plans)
        s = max(p.scratch_partials for p in plans)
        c = max(p.scratch_counters for p in plans)
        return LinearScratch(backend, t, s, c)

    def add(self, graph, projection, plan, input, output, scratch, residual=None, gate=None, prepared=False):
        check(lib.spo_linear_add(self.handle, graph.handle, projection.handle, gate.handle if gate else None,
                                 ctypes.byref(plan), input.handle if input else None, output.handle if output else None,
                                 residual.handle if residual else None, scratch.table.handle, scratch.partials.handle,
                                 scratch.counters.handle, int(prepared)))
        graph._keep.extend([projection, gate, input, output, residual, scratch])

    def add_swiglu(self, graph, gate, up, down, normalized, intermediate, residual, output, rows, scratch):
        check(lib.spo_linear_add_swiglu(self.handle, graph.handle, gate.handle, up.handle, down.handle, normalized.handle,
                                        intermediate.handle, residual.handle, output.handle, rows, scratch.table.handle,
                                        scratch.partials.handle, scratch.counters.handle))
        graph._keep.extend([gate, up, down, normalized, intermediate, residual, output, scratch])

    def scratch_size(self, output_size, input_size, rows):
        t, s, c = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
        check(lib.spo_linear_scratch_size(self.handle, output_size, input_size, rows, ctypes.byref(t), ctypes.byref(s),
                                          ctypes.byref(c)))
        return t.value, s.value, c.value
