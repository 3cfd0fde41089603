"""Python mirror of the verify step's operators (splash::ops::*), bound through include/splash_ops.h.
Names follow the reference's operators (runtime/ops/Linear.hpp, Weights.hpp)."""
import ctypes

import numpy as np

from . import _native as nat
from ._native import lib, check
from .backend import Buffer, STORAGE_PRIVATE

FMT_Q4K, FMT_IQ4XS, FMT_IQ4NL, FMT_Q5K, FMT_Q6K, FMT_Q80 = 0, 1, 2, 3, 4, 6
FORMATS = (FMT_Q4K, FMT_Q6K, FMT_Q5K, FMT_Q80, FMT_IQ4XS, FMT_IQ4NL)   # the formats with a weight image
EPILOGUE_NONE, EPILOGUE_RESIDUAL, EPILOGUE_GATE_UP, EPILOGUE_RESIDUAL_NORM = 0, 1, 2, 3
# `prepared` of Linear.add: the table holds the input rows; or the table a residual + norm plan wrote, whose rows lack
# their inverse RMS
PREPARED_TABLE, PREPARED_UNSCALED = 1, 2


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


GGML_Q4_0, GGML_Q5_0, GGML_Q3_K = 2, 6, 11
_REWRITE_BYTES = {GGML_Q3_K: (110, 210), GGML_Q4_0: (8 * 18, 8 * 34), GGML_Q5_0: (8 * 22, 8 * 34)}   # of 256 values: source, written


def rewrite_native(ggml_type, native):
    """Rows of a ggml type with no kernels of its own as the blocks of the format that reads them, with the same values:
    Q3_K as Q6_K, Q4_0 and Q5_0 as Q8_0. Returns (format, native rows of that format)."""
    native = np.ascontiguousarray(native, dtype=np.uint8)
    if ggml_type not in _REWRITE_BYTES or native.size % _REWRITE_BYTES[ggml_type][0]:
        raise nat.InvalidArgument(1, "rows of whole 256-value blocks of Q3_K, Q4_0 or Q5_0")
    source, written = _REWRITE_BYTES[ggml_type]
    out = np.empty(native.size // source * written, dtype=np.uint8)
    check(lib.spo_gguf_rewrite(ggml_type, native.ctypes.data, native.size // source, out.ctypes.data))
    return lib.spo_gguf_rewrite_format(ggml_type), out


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

    def rows(self, ranges):
        """ops::Projection::rows: a view over one or two (first, count) ranges of this projection's rows, whole 16-row
        tiles, which become its output columns in order; slices of the same image."""
        firsts = (ctypes.c_uint32 * len(ranges))(*[r[0] for r in ranges])
        counts = (ctypes.c_uint32 * len(ranges))(*[r[1] for r in ranges])
        h = ctypes.c_void_p()
        check(lib.spo_projection_rows(self.handle, firsts, counts, len(ranges), ctypes.byref(h)))
        view = Projection.__new__(Projection)
        view.handle, view.segments, view.input_size = h, self.segments, self.input_size    # the segments keep the image alive
        view.output_size, view.float32 = sum(r[1] for r in ranges), self.float32
        return view

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

    def plan(self, projection, rows, epilogue=EPILOGUE_NONE, splits=None, whole_groups=None, staged=False, column=False):
        """staged: the plan runs the staged rule (weights rounded once to half, products accumulated in fp32) instead of
        the register rule. column: the plan (one or two rows) runs the column rule, every addition in a fixed order."""
        p = nat.LinearPlan()
        if column:
            p.rows, p.epilogue, p.float32 = rows, epilogue, int(projection.float32 and epilogue == EPILOGUE_NONE)
            p.splits, p.whole_groups, p.tile = 1, 0, 2
            check(lib.spo_linear_plan_with(projection.handle, ctypes.byref(p)))
            return p
        check(lib.spo_linear_plan_for(self.handle, projection.handle, rows, epilogue, ctypes.byref(p)))
        if splits is not None or whole_groups is not None or staged:
            if splits is not None:
                p.splits = splits
            if whole_groups is not None:
                p.whole_groups = whole_groups
            p.tile = 1 if staged else 0
            check(lib.spo_linear_plan_with(projection.handle, ctypes.byref(p)))
        return p

    def scratch_for(self, backend, plans):
        t = max(p.scratch_input for p in plans)
        s = max(p.scratch_partials for p in plans)
        c = max(p.scratch_counters for p in plans)
        return LinearScratch(backend, t, s, c)

    def add(self, graph, projection, plan, input, output, scratch, residual=None, gate=None, prepared=False, norm_weight=None,
            next_table=None):
        """norm_weight, next_table: of a plan with EPILOGUE_RESIDUAL_NORM, which also writes its output rows times the
        norm's weights as the next projection's activation table; that projection passes prepared=PREPARED_UNSCALED."""
        if plan.epilogue == EPILOGUE_RESIDUAL_NORM:
            check(lib.spo_linear_add_residual_norm(self.handle, graph.handle, projection.handle, ctypes.byref(plan),
                                                   input.handle if input else None, output.handle if output else None,
                                                   residual.handle if residual else None,
                                                   norm_weight.handle if norm_weight else None,
                                                   next_table.handle if next_table else None, scratch.table.handle,
                                                   scratch.partials.handle, scratch.counters.handle, int(prepared)))
            graph._keep.extend([projection, input, output, residual, scratch, norm_weight, next_table])
            return
        check(lib.spo_linear_add(self.handle, graph.handle, projection.handle, gate.handle if gate else None,
                                 ctypes.byref(plan), input.handle if input else None, output.handle if output else None,
                                 residual.handle if residual else None, scratch.table.handle, scratch.partials.handle,
                                 scratch.counters.handle, int(prepared)))
        graph._keep.extend([projection, gate, input, output, residual, scratch])

    CHAIN_PROGRESS_BYTES = 65792

    def set_chain_spin_limit(self, polls):
        check(lib.spo_linear_set_chain_spin_limit(self.handle, polls))
    CHAIN_STATUS_OFFSET = 16

    @staticmethod
    def _fill_link(slot, link):
        handle = lambda b: b.handle if b is not None else None
        scratch = link["scratch"]
        slot.projection, slot.gate = link["projection"].handle, handle(link.get("gate"))
        slot.plan = link["plan"]
        slot.input, slot.output, slot.residual = handle(link.get("input")), handle(link.get("output")), handle(link.get("residual"))
        slot.norm_weight, slot.next_table = handle(link.get("norm_weight")), handle(link.get("next_table"))
        slot.table, slot.partials, slot.counters = scratch.table.handle, scratch.partials.handle, scratch.counters.handle
        slot.prepared = int(link.get("prepared", 0))

    def add_chain(self, graph, links, progress):
        """Up to four projections as one dispatch, each reading what the one before it wrote. links: dicts of add()'s
        arguments (projection, plan, input, output, scratch, and residual, gate, prepared, norm_weight, next_table as
        that link takes them); progress: CHAIN_PROGRESS_BYTES bytes the chain owns, zero before its first dispatch."""
        array = (nat.ChainLink * len(links))()
        for slot, link in zip(array, links):
            self._fill_link(slot, link)
            graph._keep.extend(link.values())
        check(lib.spo_linear_add_chain(self.handle, graph.handle, array, len(links), progress.handle))
        graph._keep.append(progress)

    def add_link(self, graph, **link):
        """One link as a dispatch of its own (Linear::add of all its buffers)."""
        slot = nat.ChainLink()
        self._fill_link(slot, link)
        check(lib.spo_linear_add_link(self.handle, graph.handle, ctypes.byref(slot)))
        graph._keep.extend(link.values())

    def add_swiglu(self, graph, gate, up, down, normalized, intermediate, residual, output, rows, scratch, next_table=None):
        """next_table: a second activation table (gguf_table_bytes(ffn, rows)); the gate/up pass then writes
        the down projection's table itself."""
        check(lib.spo_linear_add_swiglu(self.handle, graph.handle, gate.handle, up.handle, down.handle, normalized.handle,
                                        intermediate.handle, residual.handle, output.handle, rows, scratch.table.handle,
                                        scratch.partials.handle, scratch.counters.handle,
                                        next_table.handle if next_table is not None else None))
        graph._keep.extend([gate, up, down, normalized, intermediate, residual, output, scratch, next_table])

    @staticmethod
    def prefill_table_bytes(input_size, rows):
        return lib.spo_linear_prefill_table_bytes(input_size, rows)

    @staticmethod
    def add_prefill(graph, projection, input, output, table, rows, residual=None):
        """A chunk of up to 16384 rows through the projection under the staged rule (Linear::addPrefill). table:
        prefill_table_bytes(input size, rows) bytes."""
        check(lib.spo_linear_add_prefill(graph.handle, projection.handle, input.handle, output.handle,
                                         residual.handle if residual is not None else None, table.handle, rows))
        graph._keep.extend([projection, input, output, table, residual])

    def scratch_size(self, output_size, input_size, rows):
        t, s, c = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
        check(lib.spo_linear_scratch_size(self.handle, output_size, input_size, rows, ctypes.byref(t), ctypes.byref(s),
                                          ctypes.byref(c)))
        return t.value, s.value, c.value


# ---------------------------------------------------------------------------------------------
# PagedAttention (runtime/ops/PagedAttention.hpp in the reference)
# ---------------------------------------------------------------------------------------------
PAGE_TOKENS = 256
VALUE_BLOCK = 64


def kv_page_bytes(kv_heads, head_dim):
    return lib.spo_kv_page_bytes(kv_heads, head_dim)


class KvPages:
    """One layer's KV pool: physical pages, and the page table (uint64 physical page per logical page)."""

    def __init__(self, backend, kv_heads, head_dim, physical_pages, page_table):
        self.kv_heads, self.head_dim = kv_heads, head_dim
        self.page_bytes = kv_page_bytes(kv_heads, head_dim)
        self.physical_pages = physical_pages
        self.pool = backend.allocate_buffer(self.page_bytes * physical_pages, STORAGE_PRIVATE, "kv pool")
        self.table = backend.from_array(np.asarray(page_table, dtype=np.uint64), STORAGE_PRIVATE, "page table")

    # Host-side (de)serialisation of pages from logical arrays, for tests and synthetic contexts.
    def pack_pages(self, kcodes, kscales, vcodes, vscales):
        """Logical arrays [pages][kv_heads][256][D] int8 and [pages][kv_heads][256] float -> page bytes."""
        pages, H, T, D = kcodes.shape
        out = np.zeros((pages, self.page_bytes), dtype=np.uint8)
        kb = H * T * D
        out[:, :kb] = kcodes.reshape(pages, kb).view(np.uint8)
        # values: [H][T/64][D][64]
        v = vcodes.reshape(pages, H, T // VALUE_BLOCK, VALUE_BLOCK, D).transpose(0, 1, 2, 4, 3)
        out[:, kb:2 * kb] = np.ascontiguousarray(v).reshape(pages, kb).view(np.uint8)
        sb = H * T * 2
        out[:, 2 * kb:2 * kb + sb] = kscales.astype(np.float16).reshape(pages, H * T).view(np.uint8)
        out[:, 2 * kb + sb:2 * kb + 2 * sb] = vscales.astype(np.float16).reshape(pages, H * T).view(np.uint8)
        return out

    def unpack_pages(self, raw):
        pages = raw.shape[0]
        H, T, D = self.kv_heads, PAGE_TOKENS, self.head_dim
        kb, sb = H * T * D, H * T * 2
        kcodes = raw[:, :kb].view(np.int8).reshape(pages, H, T, D)
        v = raw[:, kb:2 * kb].view(np.int8).reshape(pages, H, T // VALUE_BLOCK, D, VALUE_BLOCK).transpose(0, 1, 2, 4, 3)
        vcodes = np.ascontiguousarray(v).reshape(pages, H, T, D)
        kscales = raw[:, 2 * kb:2 * kb + sb].copy().view(np.float16).reshape(pages, H, T).astype(np.float32)
        vscales = raw[:, 2 * kb + sb:2 * kb + 2 * sb].copy().view(np.float16).reshape(pages, H, T).astype(np.float32)
        return kcodes, kscales, vcodes, vscales

    def upload(self, page_bytes_array, first_page=0):
        self.pool.upload(page_bytes_array, first_page * self.page_bytes)

    def download(self):
        return self.pool.download(np.uint8).reshape(self.physical_pages, self.page_bytes)


class AttentionPlan:
    """ops::AttentionPlan: geometry + sequences + history splits."""

    def __init__(self, q_heads, kv_heads, head_dim, sequences, rotary_pairs=0, normalize=False, gated=False, int8_queries=False):
        """sequences: [(first_row, rows, committed, table_first)]; gated: a projection row holds each query head's
        queries, then its gate, and the output rows are multiplied by the gates' sigmoids."""
        g = nat.AttentionGeometry(q_heads, kv_heads, head_dim, rotary_pairs, int(normalize), int(gated), int(int8_queries))
        rows = (nat.AttentionRows * len(sequences))(*[nat.AttentionRows(*s) for s in sequences])
        h = ctypes.c_void_p()
        check(lib.spo_attention_plan_create(ctypes.byref(g), rows, len(sequences), ctypes.byref(h)))
        self.handle = h
        self.geometry = g
        self.sequences = sequences

    @property
    def splits(self):
        return lib.spo_attention_plan_splits(self.handle)

    def workspace_sizes(self):
        sizes = (ctypes.c_uint64 * 4)()
        check(lib.spo_attention_workspace(self.handle, sizes))
        return list(sizes)

    def __del__(self):
        try:
            lib.spo_attention_plan_destroy(self.handle)
        except Exception:
            pass


class AttentionChunkPlan:
    """ops::AttentionChunkPlan: prompt chunks [(first_row, tokens, committed, table_first)] as dispatches of eight 16-row tiles."""

    def __init__(self, q_heads, kv_heads, head_dim, chunks, rotary_pairs=0, normalize=False, gated=False, int8_queries=False):
        g = nat.AttentionGeometry(q_heads, kv_heads, head_dim, rotary_pairs, int(normalize), int(gated), int(int8_queries))
        rows = (nat.AttentionRows * len(chunks))(*[nat.AttentionRows(*c) for c in chunks])   # a chunk has a sequence's four fields
        h = ctypes.c_void_p()
        check(lib.spo_attention_chunk_plan_create(ctypes.byref(g), rows, len(chunks), ctypes.byref(h)))
        self.handle = h
        self.geometry = g
        self.chunks = chunks

    @property
    def dispatches(self):
        return lib.spo_attention_chunk_plan_dispatches(self.handle)

    def workspace_sizes(self):
        sizes = (ctypes.c_uint64 * 4)()
        check(lib.spo_attention_chunk_workspace(self.handle, sizes))
        return list(sizes)

    def __del__(self):
        try:
            lib.spo_attention_chunk_plan_destroy(self.handle)
        except Exception:
            pass


class AttentionWorkspace:
    def __init__(self, backend, plan):
        q, qs, po, ps = plan.workspace_sizes()
        self.queries = backend.allocate_buffer(q, STORAGE_PRIVATE, "staged queries")
        self.query_sums = backend.allocate_buffer(qs, STORAGE_PRIVATE, "query sums")
        self.partials = backend.allocate_buffer(po, STORAGE_PRIVATE, "attention partials")
        self.partial_sums = backend.allocate_buffer(ps, STORAGE_PRIVATE, "attention partial sums")


class PagedAttention:
    """ops::PagedAttention: addProjection, addAttention, addPathCommit."""

    @staticmethod
    def add_projection(graph, plan, qkv, workspace, pages, query_norm=None, key_norm=None, rope_cos=None, rope_sin=None):
        h = lambda b: b.handle if b is not None else None
        check(lib.spo_attention_add_projection(graph.handle, plan.handle, qkv.handle, h(query_norm), h(key_norm), h(rope_cos),
                                               h(rope_sin), workspace.queries.handle, workspace.query_sums.handle,
                                               pages.table.handle, pages.pool.handle, pages.page_bytes))
        graph._keep.extend([plan, qkv, workspace, pages, query_norm, key_norm, rope_cos, rope_sin])

    @staticmethod
    def fuses_projection(plan, projection, linear_plan):
        """Whether the q|k|v projection of this plan can prepare the attention block from its epilogue."""
        return bool(lib.spo_attention_fuses_projection(plan.handle, projection.handle, ctypes.byref(linear_plan)))

    @staticmethod
    def add_fused_projection(graph, linear, attention, workspace, pages, query_norm=None, key_norm=None, rope_cos=None, rope_sin=None,
                             **qkv):
        """The q|k|v projection (`qkv`: a link as Linear.add_link takes it, whose output is the block's packed rows) and
        add_projection's work for the block of the plan `attention` in one dispatch."""
        h = lambda b: b.handle if b is not None else None
        slot = nat.ChainLink()
        linear._fill_link(slot, qkv)
        check(lib.spo_attention_add_fused_projection(linear.handle, graph.handle, ctypes.byref(slot), attention.handle, h(query_norm),
                                                     h(key_norm), h(rope_cos), h(rope_sin), workspace.queries.handle,
                                                     workspace.query_sums.handle, pages.table.handle, pages.pool.handle,
                                                     pages.page_bytes))
        graph._keep.extend([attention, workspace, pages, query_norm, key_norm, rope_cos, rope_sin, *qkv.values()])

    @staticmethod
    def add_attention(graph, plan, workspace, tree_rows, pages, output, output_table=None, packed_qkv=None):
        check(lib.spo_attention_add_attention(graph.handle, plan.handle, workspace.queries.handle, workspace.query_sums.handle,
                                              workspace.partials.handle, workspace.partial_sums.handle, tree_rows.handle,
                                              pages.table.handle, pages.pool.handle, pages.page_bytes, output.handle,
                                              output_table.handle if output_table is not None else None,
                                              packed_qkv.handle if packed_qkv is not None else None))
        graph._keep.extend([plan, workspace, tree_rows, pages, output, output_table, packed_qkv])

    @staticmethod
    def add_chunk_projection(graph, plan, qkv, workspace, pages, query_norm=None, key_norm=None, rope_cos=None, rope_sin=None):
        h = lambda b: b.handle if b is not None else None
        check(lib.spo_attention_add_chunk_projection(graph.handle, plan.handle, qkv.handle, h(query_norm), h(key_norm), h(rope_cos),
                                                     h(rope_sin), workspace.queries.handle, workspace.query_sums.handle,
                                                     pages.table.handle, pages.pool.handle, pages.page_bytes))
        graph._keep.extend([plan, qkv, workspace, pages, query_norm, key_norm, rope_cos, rope_sin])

    @staticmethod
    def add_chunk_attention(graph, plan, workspace, tree_rows, pages, output, output_table=None, packed_qkv=None):
        check(lib.spo_attention_add_chunk_attention(graph.handle, plan.handle, workspace.queries.handle, workspace.query_sums.handle,
                                                    workspace.partials.handle, workspace.partial_sums.handle, tree_rows.handle,
                                                    pages.table.handle, pages.pool.handle, pages.page_bytes, output.handle,
                                                    output_table.handle if output_table is not None else None,
                                                    packed_qkv.handle if packed_qkv is not None else None))
        graph._keep.extend([plan, workspace, tree_rows, pages, output, output_table, packed_qkv])

    @staticmethod
    def add_path_commit(graph, plan, retained, pages):
        check(lib.spo_attention_add_path_commit(graph.handle, plan.handle, retained.handle, pages.table.handle,
                                                pages.pool.handle, pages.page_bytes))
        graph._keep.extend([plan, retained, pages])


class FloatProjection:
    """ops::FloatProjection: the fp32 projection of weights kept as F32 or BF16 rows."""

    @staticmethod
    def add(graph, input, weight_rows, output_size, input_size, output, rows, out_stride=None, out_offset=0, bf16_weights=False,
            float32_output=True):
        check(lib.spo_float_projection_add(graph.handle, input.handle, weight_rows.handle, output_size, input_size, int(bf16_weights),
                                           output.handle, rows, out_stride or output_size, out_offset, int(float32_output)))
        graph._keep.extend([input, weight_rows, output])


class StateCodec:
    """ops::StateCodec: a running state's recurrent layers as int8 codes with a bf16 scale per block of 32 values."""

    @staticmethod
    def layer_bytes(rows, columns):
        return lib.spo_state_codec_layer_bytes(rows, columns)

    @staticmethod
    def shape(layers, rows, columns, state_layer_bytes=None, codes_layer_bytes=None, bf16_state=False):
        state = rows * columns * (2 if bf16_state else 4)
        return nat.StateCodecShape(layers, rows, columns, int(bf16_state), state if state_layer_bytes is None else state_layer_bytes,
                                   StateCodec.layer_bytes(rows, columns) if codes_layer_bytes is None else codes_layer_bytes)

    @staticmethod
    def add_quantize(graph, state, codes, shape):
        check(lib.spo_state_codec_add_quantize(graph.handle, state.handle, codes.handle, ctypes.byref(shape)))
        graph._keep.extend([state, codes])

    @staticmethod
    def add_dequantize(graph, codes, state, shape):
        check(lib.spo_state_codec_add_dequantize(graph.handle, codes.handle, state.handle, ctypes.byref(shape)))
        graph._keep.extend([state, codes])

    @staticmethod
    def add_copy(graph, source, destination, shape):
        check(lib.spo_state_codec_add_copy(graph.handle, source.handle, destination.handle, ctypes.byref(shape)))
        graph._keep.extend([source, destination])


class DraftSelector:
    """ops::DraftSelector: every proposal position's candidates and edge scores, and a decode step's rows from the trees
    a draft selector grew."""

    @staticmethod
    def candidate_scratch_bytes(lanes, columns):
        out = ctypes.c_uint64()
        check(lib.spo_draft_candidate_scratch_bytes(lanes, columns, ctypes.byref(out)))
        return out.value

    @staticmethod
    def add_candidates(graph, logits, selector_hidden, scratch, candidates, unary, edges, predecessor_codebook, successor_codebook,
                       leading, trailing, vocabulary, anchors):
        buffers = [logits, selector_hidden, scratch, candidates, unary, edges, predecessor_codebook, successor_codebook]
        array = (ctypes.c_uint32 * max(len(anchors), 1))(*anchors)
        check(lib.spo_draft_add_candidates(graph.handle, *[b.handle for b in buffers], leading, trailing, vocabulary, array, len(anchors)))
        graph._keep.extend(buffers)

    @staticmethod
    def add_tree(graph, candidates, unary, edges, chain_tokens, chain_rates, tree_tokens, trees, tree_scores, tree_sizes, tree_draws,
                 tree_next, tree_caps, lanes):
        """lanes: dicts of anchor, depth, children and, as the lane has them, chain, slope, intercept (7), temperature, noise."""
        array = (nat.DraftTreeLane * len(lanes))()
        for slot, lane in zip(array, lanes):
            slot.anchor, slot.depth, slot.children, slot.chain = lane["anchor"], lane["depth"], lane["children"], lane.get("chain", 0)
            slot.slope, slot.temperature = lane.get("slope", 1.0), lane.get("temperature", 0.0)
            slot.intercept = (ctypes.c_float * 7)(*lane.get("intercept", [0.0] * 7))
            noise = lane.get("noise", 0)
            slot.noise = (ctypes.c_uint32 * 2)(noise & 0xFFFFFFFF, noise >> 32)
        buffers = [candidates, unary, edges, chain_tokens, chain_rates, tree_tokens, trees, tree_scores, tree_sizes, tree_draws, tree_next,
                   tree_caps]
        check(lib.spo_draft_add_tree(graph.handle, *[b.handle for b in buffers], array, len(lanes)))
        graph._keep.extend(buffers)

    @staticmethod
    def add_verify_children(graph, verify_sources, lane_rows, tree_rows, candidates, tree_next, tree_draws, candidate_ids,
                            candidate_probabilities, candidate_draws, depths, lanes, rows):
        buffers = [verify_sources, lane_rows, tree_rows, candidates, tree_next, tree_draws, candidate_ids, candidate_probabilities,
                   candidate_draws, depths]
        check(lib.spo_draft_add_verify_children(graph.handle, *[b.handle for b in buffers], lanes, rows))
        graph._keep.extend(buffers)

    @staticmethod
    def add_verify_rows(graph, tree_tokens, trees, tree_scores, tree_sizes, input_tokens, tree_rows, lane_rows, verify_sources, lanes,
                        rows, lane_cap, floor=0.0):
        buffers = [tree_tokens, trees, tree_scores, tree_sizes, input_tokens, tree_rows, lane_rows, verify_sources]
        check(lib.spo_draft_add_verify_rows(graph.handle, *[b.handle for b in buffers], lanes, rows, lane_cap, floor))
        graph._keep.extend(buffers)


    @staticmethod
    def add_verify_row_slots(graph, tree_tokens, trees, tree_scores, tree_sizes, input_tokens, tree_rows, lane_rows, verify_sources, lanes,
                             lane_cap, floor=0.0):
        """The verify rows in slots: lane l's rows from row l * lane_cap on, the rest of its slot inert."""
        buffers = [tree_tokens, trees, tree_scores, tree_sizes, input_tokens, tree_rows, lane_rows, verify_sources]
        check(lib.spo_draft_add_verify_row_slots(graph.handle, *[b.handle for b in buffers], lanes, lane_cap, floor))
        graph._keep.extend(buffers)


DRAFT_QUERY_ROWS, DRAFT_WINDOW, DRAFT_QKV_WIDTH, DRAFT_ATTENTION_WIDTH, DRAFT_KV_WIDTH = 8, 2048, 6144, 4096, 1024
DRAFT_RING_BYTES = 8 * DRAFT_WINDOW * 128 * 2


class DraftAttention:
    """ops::DraftAttention: the attention block of the draft model (32 query heads over 8 KV heads of 128, eight query rows
    a lane, rings of 2048 slots) over a hidden state of `hidden` values, for `lanes` lanes."""

    def __init__(self, hidden, lanes):
        self.hidden, self.lanes = hidden, lanes
        sizes = (ctypes.c_uint64 * 5)()
        check(lib.spo_draft_attention_workspace(hidden, lanes, sizes))
        self.convolution_bytes, self.qkv_bytes, self.grouped_queries_bytes, self.query_keys_bytes, self.query_values_bytes = list(sizes)

    @staticmethod
    def window_bytes(width):
        out = ctypes.c_uint64()
        check(lib.spo_draft_context_window_bytes(width, ctypes.byref(out)))
        return out.value

    def add_convolution(self, graph, input, dynamic, weights, residual, output, finish):
        buffers = [input, dynamic, weights, residual if residual is not None else input, output]
        check(lib.spo_draft_attention_add_convolution(graph.handle, *[b.handle for b in buffers], self.hidden, self.lanes, int(finish)))
        graph._keep.extend(buffers)

    def add_prepare(self, graph, qkv, grouped_queries, query_norm, key_norm, rope_cos, rope_sin, query_keys, query_values):
        buffers = [qkv, grouped_queries, query_norm, key_norm, rope_cos, rope_sin, query_keys, query_values]
        check(lib.spo_draft_attention_add_prepare(graph.handle, *[b.handle for b in buffers], self.hidden, self.lanes))
        graph._keep.extend(buffers)

    @staticmethod
    def _offsets(values):
        return (ctypes.c_uint64 * len(values))(*values)

    def add_decode(self, graph, grouped_queries, rings, keys, values, query_keys, query_values, cache_lengths):
        """rings: the buffer lane l's key ring starts keys[l] bytes into and its value ring values[l] bytes."""
        if not len(keys) == len(values) == len(cache_lengths) == self.lanes:
            raise nat.InvalidArgument(1, "a draft step binds a key ring, a value ring and a cache length a lane")
        check(lib.spo_draft_attention_add_decode(graph.handle, grouped_queries.handle, rings.handle, self._offsets(keys), self._offsets(values),
                                                 query_keys.handle, query_values.handle, (ctypes.c_uint32 * len(cache_lengths))(*cache_lengths),
                                                 self.hidden, len(cache_lengths)))
        graph._keep.extend([grouped_queries, rings, query_keys, query_values])

    def add_context_prefill(self, graph, context_kv, key_norm, rope_cos, rope_sin, rings, keys, values, tokens, start_position):
        check(lib.spo_draft_attention_add_context_prefill(graph.handle, context_kv.handle, key_norm.handle, rope_cos.handle, rope_sin.handle,
                                                          rings.handle, keys, values, tokens, start_position, self.hidden))
        graph._keep.extend([context_kv, key_norm, rope_cos, rope_sin, rings])

    def add_context_commit(self, graph, context_kv, key_norm, rope_cos, rope_sin, rings, keys, values, retained_rows, lane_rows,
                           start_positions, rows, lane_cap):
        if not len(keys) == len(values) == len(start_positions):
            raise nat.InvalidArgument(1, "a draft context commit binds a key ring, a value ring and a start position a lane")
        check(lib.spo_draft_attention_add_context_commit(graph.handle, context_kv.handle, key_norm.handle, rope_cos.handle, rope_sin.handle,
                                                         rings.handle, self._offsets(keys), self._offsets(values), retained_rows.handle,
                                                         lane_rows.handle, (ctypes.c_uint32 * len(start_positions))(*start_positions),
                                                         len(start_positions), rows, lane_cap, self.hidden))
        graph._keep.extend([context_kv, key_norm, rope_cos, rope_sin, rings, retained_rows, lane_rows])

    @staticmethod
    def add_window_store(graph, context, window, rows, start_position, width):
        check(lib.spo_draft_attention_add_window_store(graph.handle, context.handle, window.handle, rows, start_position, width))
        graph._keep.extend([context, window])

    @staticmethod
    def add_window_commit(graph, context, window, retained, lane_rows, context_rows, rows, start_position, width):
        check(lib.spo_draft_attention_add_window_commit(graph.handle, context.handle, window.handle, retained.handle, lane_rows.handle,
                                                        context_rows, rows, start_position, width))
        graph._keep.extend([context, window, retained, lane_rows])

    @staticmethod
    def add_window_load(graph, window, context, rows, start_position, width):
        check(lib.spo_draft_attention_add_window_load(graph.handle, window.handle, context.handle, rows, start_position, width))
        graph._keep.extend([window, context])

    @staticmethod
    def add_mask_rows(graph, mask, rows, width, lanes):
        check(lib.spo_draft_attention_add_mask_rows(graph.handle, mask.handle, rows.handle, width, lanes))
        graph._keep.extend([mask, rows])


def chain_tree_rows(rows_per_sequence):
    """SplashTreeRow of chains: ancestors (2 << r) - 1, parent r - 1, depth r, packed per sequence."""
    out = []
    for rows in rows_per_sequence:
        for r in range(rows):
            out.append(((2 << r) - 1, max(r - 1, 0) if r else 0xFFFF, r))
    arr = np.zeros(len(out), dtype=np.dtype([("ancestors", "<u4"), ("parent", "<u2"), ("depth", "<u2")]))
    for i, (a, p, d) in enumerate(out):
        arr[i] = (a, p, d)
    return arr


# ---------------------------------------------------------------------------------------------
# Normalization, Embedding, RoPE, Sampling
# ---------------------------------------------------------------------------------------------
class Normalization:
    @staticmethod
    def add_rms(graph, input, weight, output, width, rows):
        check(lib.spo_norm_add_rms(graph.handle, input.handle, weight.handle, output.handle, width, rows))
        graph._keep.extend([input, weight, output])

    @staticmethod
    def add_rms_table(graph, input, weight, output, table, width, rows):
        check(lib.spo_norm_add_rms_table(graph.handle, input.handle, weight.handle, output.handle, table.handle, width, rows))
        graph._keep.extend([input, weight, output, table])


class Embedding:
    @staticmethod
    def add(graph, fmt, native_rows, vocabulary, hidden, tokens, output, rows):
        check(lib.spo_embedding_add(graph.handle, fmt, native_rows.handle, vocabulary, hidden, tokens.handle, output.handle, rows))
        graph._keep.extend([native_rows, tokens, output])


class RoPE:
    @staticmethod
    def add_tree_tables(graph, inverse_frequency, depth, cosines, sines, pairs, sequences):
        """sequences: [(first_row, rows, anchor)]"""
        arr = (nat.RopeSequence * len(sequences))(*[nat.RopeSequence(*s) for s in sequences])
        check(lib.spo_rope_add_tree_tables(graph.handle, inverse_frequency.handle, depth.handle, cosines.handle, sines.handle,
                                           pairs, arr, len(sequences)))
        graph._keep.extend([inverse_frequency, depth, cosines, sines])


class GDN:
    """ops::GDN: the verify step of Gated DeltaNet layers (addDecode), the fold of a step's accepted rows (addFold) and the
    prompt chunk that builds a lane's state (addPrefill)."""

    def __init__(self, key_heads, value_heads, packed_width=None, sigmoid_gate=False, layers=1):
        conv = (2 * key_heads + value_heads) * 128
        packed_width = packed_width or conv + value_heads * 128 + 2 * value_heads
        self.shape = nat.GdnShape(key_heads, value_heads, conv, packed_width, int(sigmoid_gate))
        self.layers = layers
        self.strides = nat.GdnStateStrides()
        cell, tape = ctypes.c_uint64(), ctypes.c_uint64()
        check(lib.spo_gdn_layout(ctypes.byref(self.shape), layers, ctypes.byref(self.strides), ctypes.byref(cell), ctypes.byref(tape)))
        self.cell_bytes, self.tape_layer_bytes = cell.value, tape.value

    def add_decode(self, graph, buffers, layer, lanes, tiled_heads=False, float_norm=False):
        """buffers: dict of Buffer by the names of spo_gdn_decode_buffers (tree_rows among them: 8 bytes a row, uint32
        ancestors, uint16 parent, uint16 depth); lanes: [dict(first_row, rows, pending_path, pending_tape, step_tape,
        current_cell, next_cell)]."""
        b = nat.GdnDecodeBuffers(**{k: v.handle for k, v in buffers.items()}, float_norm=int(float_norm))
        arr = (nat.GdnLane * len(lanes))(*[nat.GdnLane(l["first_row"], l["rows"], l.get("pending_path", 0), 0, l.get("pending_tape", 0),
                                                       l["step_tape"], l["current_cell"], l["next_cell"]) for l in lanes])
        check(lib.spo_gdn_add_decode(graph.handle, ctypes.byref(b), ctypes.byref(self.shape), layer, ctypes.byref(self.strides),
                                     int(tiled_heads), arr, len(lanes)))
        graph._keep.extend(list(buffers.values()))

    def prefill_workspace(self, backend, tokens):
        """The buffers of rows a chunk of `tokens` rows hands from pass to pass (and its hidden rows)."""
        kw, vw, vh = self.shape.key_heads * 128, self.shape.value_heads * 128, self.shape.value_heads
        sizes = dict(queries=tokens * kw * 2, keys=tokens * kw * 2, values=tokens * vw * 2, decay=tokens * vh * 4, beta=tokens * vh * 2,
                     recurrent_rows=tokens * vw * 2, hidden=tokens * vw * 2)
        return {n: backend.allocate_buffer(max(b, 16), STORAGE_PRIVATE, "gdn prefill " + n) for n, b in sizes.items()}

    def add_prefill(self, graph, buffers, layer, tokens, current_cell, next_cell, captures=(), tiled_heads=False, float_norm=False):
        """GDN::addPrefill: a prompt chunk of one lane and layer. buffers: dict of Buffer by the names of
        spo_gdn_prefill_buffers; captures: [(tokens, cell)], ascending inside the rows."""
        b = nat.GdnPrefillBuffers(**{k: v.handle for k, v in buffers.items()}, float_norm=int(float_norm), current_cell=current_cell,
                                  next_cell=next_cell)
        arr = (nat.GdnPrefillCapture * max(1, len(captures)))(*[nat.GdnPrefillCapture(t, 0, c) for t, c in captures])
        check(lib.spo_gdn_add_prefill(graph.handle, ctypes.byref(b), ctypes.byref(self.shape), layer, tokens, ctypes.byref(self.strides),
                                      int(tiled_heads), arr, len(captures)))
        graph._keep.extend(list(buffers.values()))

    def add_fold(self, graph, states, tape, retained_rows, step_tape, state_cell, fold_cell, rows):
        check(lib.spo_gdn_add_fold(graph.handle, states.handle, tape.handle, retained_rows.handle, step_tape, state_cell, fold_cell,
                                   ctypes.byref(self.shape), self.layers, rows, ctypes.byref(self.strides)))
        graph._keep.extend([states, tape, retained_rows])


class MoE:
    """ops::MoE: routing (addRouting) and the routed experts with their weighted sum (addRouted)."""

    def __init__(self, backend, hidden, ffn, experts, top_k, rows, shared_slices=0, shared_gate=False, sigmoid_router=False):
        self.shape = nat.MoeShape(hidden, ffn, experts, top_k, shared_slices, int(shared_gate), int(sigmoid_router), 0)
        self.rows = rows
        sizes = (ctypes.c_uint64 * 11)()
        check(lib.spo_moe_workspace_sizes(ctypes.byref(self.shape), rows, sizes))
        self.buffers = {n: backend.allocate_buffer(max(int(b), 16), STORAGE_PRIVATE, "moe " + n) for n, b in zip(nat.MOE_WORKSPACE_FIELDS, sizes)}
        self.workspace = nat.MoeWorkspace(**{n: b.handle for n, b in self.buffers.items()})

    def add_routing(self, graph, scores, rows=None, score_stride=None, input=None, shared_scalar_gate=None):
        """input (the normalized rows) and shared_scalar_gate (fp32 [hidden]): of a shape with a gated shared expert."""
        check(lib.spo_moe_add_routing(graph.handle, scores.handle, score_stride or self.shape.experts, ctypes.byref(self.workspace),
                                      ctypes.byref(self.shape), rows or self.rows, input.handle if input is not None else None,
                                      shared_scalar_gate.handle if shared_scalar_gate is not None else None))
        graph._keep.extend([scores, self, input, shared_scalar_gate])

    def add_routed(self, graph, normalized, residual, output, gate_images, up_images, down_images, rows=None, fmt=FMT_Q4K,
                   down_fmt=FMT_Q4K, norm_weight=None, next_table=None):
        """norm_weight, next_table: the output rows also leave as the table of the projection after their RMS norm (that
        projection passes prepared=PREPARED_UNSCALED)."""
        if next_table is not None:
            check(lib.spo_moe_add_routed_norm(graph.handle, normalized.handle, residual.handle, output.handle, gate_images.handle,
                                              up_images.handle, down_images.handle, fmt, down_fmt, ctypes.byref(self.workspace),
                                              ctypes.byref(self.shape), rows or self.rows, norm_weight.handle, next_table.handle))
        else:
            check(lib.spo_moe_add_routed(graph.handle, normalized.handle, residual.handle, output.handle, gate_images.handle, up_images.handle,
                                         down_images.handle, fmt, down_fmt, ctypes.byref(self.workspace), ctypes.byref(self.shape),
                                         rows or self.rows))
        graph._keep.extend([normalized, residual, output, gate_images, up_images, down_images, self, norm_weight, next_table])


NO_TOKEN = 0xFFFFFFFF


class RowCopy:
    """ops::RowCopy: rows of bf16 values between two row regions (row, stride, column)."""

    @staticmethod
    def add(graph, source, from_region, destination, to_region, rows, width):
        check(lib.spo_row_copy_add(graph.handle, source.handle, *from_region, destination.handle, *to_region, rows, width))
        graph._keep.extend([source, destination])


class Sampling:
    """ops::Sampling: addVerify (argmax or rejection sampling per row), addAcceptance (tree walk)."""

    @staticmethod
    def workspace(rows):
        sizes = (ctypes.c_uint64 * 5)()
        check(lib.spo_sampling_workspace(rows, sizes))
        return list(sizes)

    @staticmethod
    def add_verify(graph, buffers, vocabulary, stride, lanes, policies, stop_tokens=None):
        """buffers: dict of Buffer by the names of spo_sampling_buffers (token_mask with mask_words for constrained
        lanes); lanes: [(first, rows)]; policies: a lane's temperature, or (temperature, min_p, top_k, top_p[,
        constrained, excludes_stop_tokens]); stop_tokens: up to four ids."""
        words = buffers.get("mask_words", 0)
        b = nat.SamplingBuffers(**{k: (v.handle if v is not None else None) for k, v in buffers.items() if k != "mask_words"},
                                mask_words=words)
        arr = (nat.LaneRows * len(lanes))(*[nat.LaneRows(*l) for l in lanes])
        full = [tuple(p) if isinstance(p, (tuple, list)) else (p, 0.0, 0, 1.0) for p in policies]
        structs = (nat.SamplingPolicy * len(lanes))(*[nat.SamplingPolicy(*p) for p in full])
        stops = None
        if stop_tokens is not None:
            stops = (ctypes.c_uint32 * 4)(*(list(stop_tokens) + [NO_TOKEN] * 4)[:4])
        check(lib.spo_sampling_add_verify(graph.handle, ctypes.byref(b), vocabulary, stride, arr, structs, len(lanes), stops))
        graph._keep.extend([v for k, v in buffers.items() if k != "mask_words"])

    PENALTY_PROMPT = 0x80000000

    @staticmethod
    def rebuild_penalty_words(vocabulary, history, generated_tokens, pending_token=None, mark_prompt=True):
        """Sampling::rebuildPenaltyWords: a request's row of the penalty table (uint32 [vocabulary], host memory) from its
        history (the prompt, then `generated_tokens` outputs) and the pending anchor."""
        history = np.ascontiguousarray(history, dtype=np.uint32)
        words = np.empty(vocabulary, dtype=np.uint32)
        check(lib.spo_sampling_rebuild_penalty_words(words.ctypes.data, vocabulary, history.ctypes.data, history.size, generated_tokens,
                                                     NO_TOKEN if pending_token is None else int(pending_token), int(mark_prompt)))
        return words

    @staticmethod
    def _penalized(lanes, penalties):
        if len(penalties) != len(lanes):
            raise nat.InvalidArgument(1, "one (repetition, presence, frequency, table row) per lane")
        return ((nat.LaneRows * len(lanes))(*[nat.LaneRows(*l) for l in lanes]),
                (nat.SamplingPenalties * len(lanes))(*[nat.SamplingPenalties(*p) for p in penalties]))

    @staticmethod
    def add_penalties(graph, logits, words, input_tokens, tree_rows, vocabulary, stride, lanes, penalties):
        """Sampling::addPenalties: penalties: a lane's (repetition, presence, frequency, table row); (1, 0, 0, *) leaves
        the lane alone. Runs before add_verify."""
        rows, structs = Sampling._penalized(lanes, penalties)
        check(lib.spo_sampling_add_penalties(graph.handle, logits.handle, words.handle, input_tokens.handle, tree_rows.handle, vocabulary,
                                             stride, rows, structs, len(lanes)))
        graph._keep.extend([logits, words, input_tokens, tree_rows])

    @staticmethod
    def add_penalty_count(graph, words, tokens, retained, vocabulary, lanes, penalties):
        """The tokens each penalized lane retained of the step (add_acceptance's) counted into its row of the table."""
        rows, structs = Sampling._penalized(lanes, penalties)
        check(lib.spo_sampling_add_penalty_count(graph.handle, words.handle, tokens.handle, retained.handle, vocabulary, rows, structs,
                                                 len(lanes)))
        graph._keep.extend([words, tokens, retained])

    @staticmethod
    def thinking_cutoff(row, end, also_ends=NO_TOKEN, waits_for_mask=False):
        """A lane's ops::ThinkingCutoff as the C struct; None stands for a lane without one."""
        end = list(end)
        return nat.ThinkingCutoff(1, row, len(end), (ctypes.c_uint32 * 16)(*end[:16]), also_ends, int(waits_for_mask))

    @staticmethod
    def add_thinking_cutoff(graph, input_tokens, tree_rows, tokens, vocabulary, lanes, cutoffs, token_mask=None, mask_words=0):
        """The thinking cutoffs over add_verify's selections, before add_acceptance: cutoffs: one thinking_cutoff(...) or
        None a lane."""
        arr = (nat.LaneRows * len(lanes))(*[nat.LaneRows(*l) for l in lanes])
        structs = (nat.ThinkingCutoff * len(lanes))(*[c if c is not None else nat.ThinkingCutoff() for c in cutoffs])
        check(lib.spo_sampling_add_thinking_cutoff(graph.handle, input_tokens.handle, tree_rows.handle, tokens.handle,
                                                   token_mask.handle if token_mask is not None else None, mask_words, vocabulary, arr,
                                                   structs, len(lanes)))
        graph._keep.extend([b for b in (input_tokens, tree_rows, tokens, token_mask) if b is not None])

    STATIC_MAXIMUM_ROWS = 256

    @staticmethod
    def greedy_rows_static(logits, rows, vocabulary, stride, tokens, stream=None):
        """spo_sampling_greedy_rows_static: every row's greedy selection, launched on `stream` (a hipStream_t as an
        integer; None is the null stream) with no allocation; logits and tokens are device Buffers. Returns once
        the kernels are launched: the caller synchronizes the stream."""
        check(lib.spo_sampling_greedy_rows_static(logits.gpu_address, rows, vocabulary, stride, tokens.gpu_address, stream))

    @staticmethod
    def add_acceptance(graph, input_tokens, tree_rows, tokens, retained, accepted, retained_rows, lanes, remaining,
                       stop_tokens=(NO_TOKEN,) * 4):
        arr = (nat.LaneRows * len(lanes))(*[nat.LaneRows(*l) for l in lanes])
        rem = (ctypes.c_uint32 * len(lanes))(*remaining)
        stops = (ctypes.c_uint32 * 4)(*stop_tokens)
        check(lib.spo_sampling_add_acceptance(graph.handle, input_tokens.handle, tree_rows.handle, tokens.handle, retained.handle,
                                              accepted.handle, retained_rows.handle, arr, rem, len(lanes), stops))
        graph._keep.extend([input_tokens, tree_rows, tokens, retained, accepted, retained_rows])
