"""The dense verify step (model::DenseVerify), bound through include/splash_ops.h: the target part of
one speculative-decoding cycle, as the reference's Runtime::decodeAsync encodes it
(runtime/model/Runtime.cpp:3985-3993)."""
import ctypes

import numpy as np

from . import _native as nat
from ._native import lib, check
from .backend import Buffer, CommandGraph, STORAGE_PRIVATE
from . import ops

(INPUT_TOKENS, TREE_ROWS, DEPTHS, UNIFORMS, TOKENS, RETAINED, ACCEPTED, RETAINED_ROWS, PAGE_TABLE, KV_POOL, LOGITS,
 DRAFT_PROBABILITIES, HIDDEN) = range(13)


class Lane:
    def __init__(self, rows, committed, table_first=0, temperature=0.0, remaining=0xFFFFFFFF):
        self.rows, self.committed, self.table_first, self.temperature, self.remaining = rows, committed, table_first, temperature, remaining

    def struct(self):
        return nat.VerifyLane(self.rows, self.committed, self.table_first, self.temperature, self.remaining)


class DenseVerify:
    def __init__(self, backend, hidden, q_heads, kv_heads, head_dim, ffn, vocabulary, layers, rotary_pairs=None,
                 normalize_heads=True, rope_theta=1e6, max_lanes=1, physical_pages=2, page_table_entries=None):
        self.backend = backend
        pairs = head_dim // 2 if rotary_pairs is None else rotary_pairs
        self.dims = nat.DenseDimensions(hidden, q_heads, kv_heads, head_dim, ffn, vocabulary, layers, pairs, int(normalize_heads),
                                        rope_theta)
        h = ctypes.c_void_p()
        entries = page_table_entries if page_table_entries is not None else physical_pages
        check(lib.spo_dense_verify_create(backend.handle, ctypes.byref(self.dims), max_lanes, physical_pages, entries, ctypes.byref(h)))
        self.handle = h
        self.physical_pages = physical_pages
        self._keep = []

    def __del__(self):
        try:
            lib.spo_dense_verify_destroy(self.handle)
        except Exception:
            pass

    def buffer(self, which, index=0):
        out = ctypes.c_void_p()
        check(lib.spo_dense_verify_buffer(self.handle, which, index, ctypes.byref(out)))
        return Buffer(out.value)

    @property
    def page_bytes(self):
        return lib.spo_dense_verify_page_bytes(self.handle)

    def set_layer(self, layer, qkv, output, gate, up, down, input_norm, post_norm, query_norm, key_norm):
        check(lib.spo_dense_verify_set_layer(self.handle, layer, qkv.handle, output.handle, gate.handle, up.handle, down.handle,
                                             input_norm.handle, post_norm.handle, query_norm.handle, key_norm.handle))
        self._keep.extend([qkv, output, gate, up, down, input_norm, post_norm, query_norm, key_norm])

    def set_head(self, embedding_format, embedding_rows, final_norm, head):
        check(lib.spo_dense_verify_set_head(self.handle, embedding_format, embedding_rows.handle, final_norm.handle, head.handle))
        self._keep.extend([embedding_rows, final_norm, head])

    def _lanes(self, lanes):
        return (nat.VerifyLane * len(lanes))(*[l.struct() for l in lanes])

    def step_bytes(self, lanes):
        return lib.spo_dense_verify_step_bytes(self.handle, self._lanes(lanes), len(lanes))

    def encode(self, lanes, commit=True, graph=None):
        graph = graph or CommandGraph()
        check(lib.spo_dense_verify_encode(self.handle, graph.handle, self._lanes(lanes), len(lanes), int(commit)))
        graph._keep.append(self)
        return graph

    def encode_part(self, part, index, lanes, graph=None):
        graph = graph or CommandGraph()
        check(lib.spo_dense_verify_encode_part(self.handle, graph.handle, part, index, self._lanes(lanes), len(lanes)))
        graph._keep.append(self)
        return graph

    def set_block(self, lanes, tokens, tree_rows=None, uniforms=None):
        """Writes the step's host-visible inputs: packed input tokens, tree rows (chains by default), depths."""
        rows = sum(l.rows for l in lanes)
        tokens = np.asarray(tokens, dtype=np.uint32)
        assert tokens.size == rows
        tree = tree_rows if tree_rows is not None else ops.chain_tree_rows([l.rows for l in lanes])
        self.buffer(INPUT_TOKENS).contents()[:rows * 4] = tokens.view(np.uint8)
        self.buffer(TREE_ROWS).contents()[:rows * 8] = tree.view(np.uint8)
        self.buffer(DEPTHS).contents()[:rows * 4] = tree["depth"].astype(np.uint32).view(np.uint8)
        if uniforms is not None:
            self.buffer(UNIFORMS).contents()[:rows * 8] = np.asarray(uniforms, dtype=np.float32).reshape(rows, 2).view(np.uint8).ravel()

    def results(self, lanes):
        """(selected/retained tokens per packed row, retained count, accepted count, retained-row mask) per lane."""
        rows = sum(l.rows for l in lanes)
        n = len(lanes)
        rd = lambda which, count: self.buffer(which).contents()[:count * 4].view(np.uint32).copy()
        return rd(TOKENS, rows), rd(RETAINED, n), rd(ACCEPTED, n), rd(RETAINED_ROWS, n)
