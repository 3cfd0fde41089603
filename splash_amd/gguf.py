"""GGUF files over the C ABI (include/splash_gguf.h): the reference's model::GgufFile (runtime/model/GgufFile.hpp)."""
import ctypes

import numpy as np

from . import _native as nat
from ._native import lib, check
from .backend import Buffer

NO_FORMAT = 0xFFFFFFFF


class Tensor:
    def __init__(self, index, name, info):
        self.index, self.name = index, name
        self.ggml_type = info.ggml_type
        self.dims = [int(info.dims[d]) for d in range(info.dimensions)]
        self.bytes = int(info.bytes)
        self.format = None if info.format == NO_FORMAT else int(info.format)

    def __repr__(self):
        return f"Tensor({self.name!r}, type {self.ggml_type}, dims {self.dims})"


class GgufFile:
    """model::GgufFile: a mapped GGUF (version 3) file, its scalar metadata and its tensor table. `path` may be the
    list of a split GGUF's parts in split order."""

    def __init__(self, path):
        handle = ctypes.c_void_p()
        if isinstance(path, (list, tuple)):
            parts = (ctypes.c_char_p * len(path))(*[str(p).encode() for p in path])
            check(lib.spg_open_parts(parts, len(path), ctypes.byref(handle)))
        else:
            check(lib.spg_open(str(path).encode(), ctypes.byref(handle)))
        self.handle = handle
        self.tensors = []
        for i in range(lib.spg_tensor_count(handle)):
            size = lib.spg_tensor_name(handle, i, None, 0)
            name = ctypes.create_string_buffer(size)
            lib.spg_tensor_name(handle, i, name, size)
            info = nat.GgufTensor()
            check(lib.spg_tensor_info(handle, i, ctypes.byref(info)))
            self.tensors.append(Tensor(i, name.value.decode(), info))

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                lib.spg_close(self.handle)
        except Exception:
            pass

    def unsigned(self, key):
        v = ctypes.c_uint64()
        return int(v.value) if lib.spg_metadata_unsigned(self.handle, key.encode(), ctypes.byref(v)) else None

    def float(self, key):
        v = ctypes.c_double()
        return float(v.value) if lib.spg_metadata_float(self.handle, key.encode(), ctypes.byref(v)) else None

    def string(self, key):
        size = lib.spg_metadata_string(self.handle, key.encode(), None, 0)
        if not size:
            return None
        out = ctypes.create_string_buffer(size)
        lib.spg_metadata_string(self.handle, key.encode(), out, size)
        return out.value.decode()

    def find(self, name):
        index = lib.spg_find(self.handle, name.encode())
        return self.tensors[index] if index >= 0 else None

    def data(self, tensor):
        """The tensor's bytes in the mapped file (a copy)."""
        p = lib.spg_tensor_data(self.handle, tensor.index)
        return np.ctypeslib.as_array((ctypes.c_uint8 * tensor.bytes).from_address(p)).copy()

    def load_image(self, backend, tensor, first_row=0, rows=0):
        """(format, rows, input size, image buffer) of a projection tensor's rows: what ops.Projection takes."""
        image, fmt, n, k = ctypes.c_void_p(), ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
        check(lib.spg_load_image(backend.handle, self.handle, tensor.index, first_row, rows, ctypes.byref(image), ctypes.byref(fmt),
                                 ctypes.byref(n), ctypes.byref(k)))
        return int(fmt.value), int(n.value), int(k.value), Buffer(image.value)

    def load_bf16(self, backend, tensor):
        out = ctypes.c_void_p()
        check(lib.spg_load_bf16(backend.handle, self.handle, tensor.index, ctypes.byref(out), None))
        return Buffer(out.value)
