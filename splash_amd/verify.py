"""The verify step's drivers (model::DenseVerify, model::HybridVerify), bound through include/splash_ops.h: the
target part of one speculative-decoding cycle, as the reference's Runtime::decodeAsync encodes it
(runtime/model/Runtime.cpp:3985-3993)."""
import ctypes

import numpy as np

from . import _native as nat
from ._native import lib, check
from .backend import Buffer, CommandGraph, STORAGE_PRIVATE
from . import ops

(INPUT_TOKENS, TREE_ROWS, DEPTHS, UNIFORMS, TOKENS, RETAINED, ACCEPTED, RETAINED_ROWS, PAGE_TABLE, KV_POOL, LOGITS,
 DRAFT_PROBABILITIES, HIDDEN, GDN_STATES, GDN_TAPE, QKV_ROWS, ATTENTION_ROWS, FFN_ROWS, CANDIDATE_CHILDREN, PENALTY_WORDS, TOKEN_MASK) = range(21)


class Lane:
    def __init__(self, rows, committed, table_first=0, temperature=0.0, remaining=0xFFFFFFFF, min_p=0.0, top_k=0, top_p=1.0):
        self.rows, self.committed, self.table_first, self.temperature, self.remaining = rows, committed, table_first, temperature, remaining
        self.min_p, self.top_k, self.top_p = min_p, top_k, top_p

    def struct(self):
        return nat.VerifyLane(self.rows, self.committed, self.table_first, self.temperature, self.remaining, self.min_p, self.top_k,
                              self.top_p)


class DenseVerify:
    def __init__(self, backend, hidden, q_heads, kv_heads, head_dim, ffn, vocabulary, layers, rotary_pairs=None,
                 normalize_heads=True, rope_theta=1e6, max_lanes=1, physical_pages=2, page_table_entries=None, prefill_rows=0):
        """prefill_rows: the most rows of a prompt chunk (encode_prefill); 0: a step's most, 16 x max_lanes."""
        self.backend = backend
        pairs = head_dim // 2 if rotary_pairs is None else rotary_pairs
        self.dims = nat.DenseDimensions(hidden, q_heads, kv_heads, head_dim, ffn, vocabulary, layers, pairs, int(normalize_heads),
                                        rope_theta)
        h = ctypes.c_void_p()
        entries = page_table_entries if page_table_entries is not None else physical_pages
        check(lib.spo_dense_verify_create_chunked(backend.handle, ctypes.byref(self.dims), max_lanes, physical_pages, entries, prefill_rows,
                                                  ctypes.byref(h)))
        self.handle = h
        self.physical_pages = physical_pages
        self._keep = []

    @classmethod
    def from_gguf(cls, backend, gguf_file, max_lanes=1, physical_pages=2, page_table_entries=None):
        """A driver of the geometry the file's metadata names, with every weight loaded from the file
        (spg_dense_dimensions, spo_dense_verify_load_gguf)."""
        d = nat.DenseDimensions()
        check(lib.spg_dense_dimensions(gguf_file.handle, ctypes.byref(d)))
        self = cls(backend, d.hidden, d.q_heads, d.kv_heads, d.head_dim, d.ffn, d.vocabulary, d.layers, d.rotary_pairs,
                   bool(d.normalize_heads), d.rope_theta, max_lanes, physical_pages, page_table_entries)
        check(lib.spo_dense_verify_load_gguf(self.handle, gguf_file.handle))
        self._keep.append(gguf_file)
        return self

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

    def set_staged_prefill(self, on):
        """Long prompt chunks through the prefill tile (the staged rule) instead of the step's kernels; off by default."""
        check(lib.spo_dense_verify_set_staged_prefill(self.handle, int(on)))

    def set_penalties(self, lane, repetition=1.0, presence=0.0, frequency=0.0):
        """The sampling penalties of dispatch lane `lane` for the steps encoded after; its row of the PENALTY_WORDS buffer
        (uint32 [lanes][vocabulary]; ops.Sampling.rebuild_penalty_words makes a row) holds what they read."""
        check(lib.spo_dense_verify_set_penalties(self.handle, lane, repetition, presence, frequency))

    def set_admission(self, lane, constrained=False, excludes_stop_tokens=False):
        """Dispatch lane `lane` of the steps encoded after admits only the tokens of its rows of the TOKEN_MASK buffer
        (uint32 [rows][ceil(vocabulary / 32)]) and / or never selects a stop token."""
        check(lib.spo_dense_verify_set_admission(self.handle, lane, int(constrained), int(excludes_stop_tokens)))

    def set_stop_tokens(self, stop_tokens=()):
        """Up to four tokens that end a sequence, for the steps encoded after."""
        stops = (ctypes.c_uint32 * 4)(*(list(stop_tokens) + [0xFFFFFFFF] * 4)[:4])
        check(lib.spo_dense_verify_set_stop_tokens(self.handle, stops))

    def set_thinking_cutoff(self, lane, row=None, end=(), also_ends=0xFFFFFFFF, waits_for_mask=False):
        """The thinking cutoff of dispatch lane `lane` for the steps encoded after: its rows of depth `row` on select the
        tokens of `end` in order; row None clears it."""
        cutoff = None if row is None else ctypes.byref(ops.Sampling.thinking_cutoff(row, end, also_ends, waits_for_mask))
        check(lib.spo_dense_verify_set_thinking_cutoff(self.handle, lane, cutoff))

    def set_capture(self, layers, destination):
        """After each of `layers` (ascending) every row's output goes to its slot of `destination`, bf16 [rows][len(layers) x hidden]."""
        check(lib.spo_dense_verify_set_capture(self.handle, (ctypes.c_uint32 * max(len(layers), 1))(*layers), len(layers),
                                               destination.handle if destination is not None else None))
        self._keep.append(destination)

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

    def encode_prefill(self, table_first, committed, tokens, graph=None):
        """A chunk of `tokens` prompt tokens of one sequence in one pass over the weights (every layer, no head): see
        set_prefill_block for its inputs."""
        graph = graph or CommandGraph()
        check(lib.spo_dense_verify_encode_prefill(self.handle, graph.handle, table_first, committed, tokens))
        graph._keep.append(self)
        return graph

    def set_prefill_block(self, tokens):
        """A prompt chunk's inputs: its tokens, a chain of tree rows a block of sixteen, each row's depth in its block."""
        tokens = np.asarray(tokens, dtype=np.uint32)
        blocks = [min(16, tokens.size - at) for at in range(0, tokens.size, 16)]
        self.set_block([Lane(rows, 0) for rows in blocks], tokens)

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

    _results_call = "spo_dense_verify_results"

    def set_chained(self, chained):
        """Whether steps encoded from now on chain a layer's projections after its attention into one dispatch (off by
        default): the results are the same bit for bit."""
        check(lib.spo_dense_verify_set_chained(self.handle, int(bool(chained))))

    def chain_status(self):
        """0 when every chained projection of the last completed step met its wait, nonzero when one gave up (the step's
        logits, hidden rows and results are void then); reading it clears it."""
        status = ctypes.c_uint32()
        check(lib.spo_dense_verify_chain_status(self.handle, ctypes.byref(status)))
        return status.value

    def set_fused_prepare(self, fused):
        """Whether a layer's q|k|v projection also prepares its attention block where the kernels take the pair (off by
        default): the results are the same bit for bit."""
        check(lib.spo_dense_verify_set_fused_prepare(self.handle, int(bool(fused))))

    def test_children(self, on=True):
        """Whether the sampled lanes of steps encoded from now on test their draft's drawn children among sixteen
        candidates, or (the default) one child against the full-vocabulary draft probabilities."""
        check(lib.spo_dense_verify_set_test_children(self.handle, int(bool(on))))

    def set_candidate_children(self, ids, probabilities, draws, child_uniforms):
        """The sampled rows' candidate children, by packed row: ids uint32 [rows][16], probabilities fp32 [rows][16], draws
        bytes [rows][4] (0xFF past a row's drawn children), child_uniforms fp32 [rows][4]; later steps test them."""
        self.test_children(True)
        for which, array, dtype in ((0, ids, np.uint32), (1, probabilities, np.float32), (2, draws, np.uint8), (3, child_uniforms, np.float32)):
            raw = np.ascontiguousarray(array, dtype).view(np.uint8).ravel()
            self.buffer(CANDIDATE_CHILDREN, which).contents()[:raw.size] = raw

    def results(self, lanes):
        """(selected/retained tokens per packed row, retained count, accepted count, retained-row mask) per lane, read
        from the driver's buffers after the step's command completed and checked as Runtime::finalizeDecode checks them
        (a SplashError names the lane and the rule a result breaks)."""
        rows, n = sum(l.rows for l in lanes), len(lanes)
        tokens = np.zeros(rows, np.uint32)
        retained, accepted, mask = (np.zeros(n, np.uint32) for _ in range(3))
        p = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))
        check(getattr(lib, self._results_call)(self.handle, self._lanes(lanes), n, p(tokens), p(retained), p(accepted), p(mask)))
        return tokens, retained, accepted, mask


class HybridLane(Lane):
    """A lane of a hybrid step: its block, the rows of its previous step it accepted, and the step's parity (a step
    reads the lane's state cell `parity` and writes the other; the lane's next step flips it)."""

    def __init__(self, rows, committed, table_first=0, temperature=0.0, remaining=0xFFFFFFFF, pending_path=0, parity=0):
        super().__init__(rows, committed, table_first, temperature, remaining)
        self.pending_path, self.parity = pending_path, parity

    def struct(self):
        return nat.HybridLane(super().struct(), self.pending_path, self.parity)


class HybridVerify:
    """model::HybridVerify: Gated DeltaNet and attention mixers (every `attention_interval`-th layer attends) over a
    mixture-of-experts FFN."""

    def __init__(self, backend, hidden, vocabulary, layers, q_heads, kv_heads, head_dim, gdn_key_heads, gdn_value_heads, experts, top_k,
                 expert_ffn, attention_interval=4, rotary_pairs=None, normalize_heads=True, rope_theta=1e6, gdn_packed_width=None,
                 max_lanes=1, physical_pages=2, page_table_entries=None, gated_attention=False, shared_slices=0, shared_gate=False, dense_ffn=0,
                 prefill_rows=0):
        """experts 0 and dense_ffn: every layer's FFN is a dense SwiGLU of that width instead of a mixture of experts.
        prefill_rows: the most rows of a prompt chunk (encode_prefill); 0: a step's most."""
        self.backend = backend
        pairs = head_dim // 2 if rotary_pairs is None else rotary_pairs
        conv = (2 * gdn_key_heads + gdn_value_heads) * 128
        packed = gdn_packed_width or (conv + gdn_value_heads * 128 + 2 * gdn_value_heads + 15) // 16 * 16
        self.dims = nat.HybridDimensions(hidden, vocabulary, layers, attention_interval, q_heads, kv_heads, head_dim, pairs,
                                         int(normalize_heads), int(gated_attention), rope_theta, gdn_key_heads, gdn_value_heads, packed, experts, top_k, expert_ffn,
                                         shared_slices, int(shared_gate), dense_ffn)
        h = ctypes.c_void_p()
        entries = page_table_entries if page_table_entries is not None else physical_pages
        check(lib.spo_hybrid_verify_create_chunked(backend.handle, ctypes.byref(self.dims), max_lanes, physical_pages, entries, prefill_rows,
                                                   ctypes.byref(h)))
        self.handle = h
        self.physical_pages = physical_pages
        page, cell, tape = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
        self.strides = nat.GdnStateStrides()
        check(lib.spo_hybrid_verify_layout(h, ctypes.byref(page), ctypes.byref(cell), ctypes.byref(tape), ctypes.byref(self.strides)))
        self.page_bytes, self.cell_bytes, self.tape_layer_bytes = page.value, cell.value, tape.value
        self.gdn_layers = layers - layers // attention_interval
        self._keep = []

    def __del__(self):
        try:
            lib.spo_hybrid_verify_destroy(self.handle)
        except Exception:
            pass

    @classmethod
    def from_gguf(cls, backend, gguf_file, max_lanes=1, physical_pages=2, page_table_entries=None, prefill_rows=0):
        """A driver of the geometry the file's metadata names (architectures qwen35 and qwen35moe), every weight loaded
        from the file (spg_hybrid_dimensions, spo_hybrid_verify_load_gguf)."""
        d = nat.HybridDimensions()
        check(lib.spg_hybrid_dimensions(gguf_file.handle, ctypes.byref(d)))
        self = cls(backend, d.hidden, d.vocabulary, d.layers, d.q_heads, d.kv_heads, d.head_dim, d.gdn_key_heads, d.gdn_value_heads, d.experts,
                   d.top_k, d.expert_ffn, attention_interval=d.attention_interval, rotary_pairs=d.rotary_pairs,
                   normalize_heads=bool(d.normalize_heads), rope_theta=d.rope_theta, gdn_packed_width=d.gdn_packed_width, max_lanes=max_lanes,
                   physical_pages=physical_pages, page_table_entries=page_table_entries, gated_attention=bool(d.gated_attention),
                   shared_slices=d.shared_slices, shared_gate=bool(d.shared_gate), dense_ffn=d.dense_ffn, prefill_rows=prefill_rows)
        check(lib.spo_hybrid_verify_load_gguf(self.handle, gguf_file.handle))
        self._keep.append(gguf_file)
        return self

    def attends(self, layer):
        return (layer + 1) % self.dims.attention_interval == 0

    def mixer_index(self, layer):
        before = layer // self.dims.attention_interval
        return before if self.attends(layer) else layer - before

    def cell_offset(self, lane, parity):
        return (lane * 2 + (parity & 1)) * self.cell_bytes

    def tape_offset(self, lane, parity, gdn_layer):
        return ((lane * 2 + (parity & 1)) * self.gdn_layers + gdn_layer) * self.tape_layer_bytes

    def buffer(self, which, index=0):
        out = ctypes.c_void_p()
        check(lib.spo_hybrid_verify_buffer(self.handle, which, index, ctypes.byref(out)))
        return Buffer(out.value)

    def set_layer(self, layer, mixer_input, mixer_output, input_norm, post_norm, router=None, gate_images=None, up_images=None, down_images=None,
                  query_norm=None, key_norm=None, convolution_weights=None, decay_weights=None, time_bias=None, mixer_norm=None,
                  expert_format=ops.FMT_Q4K, expert_down_format=ops.FMT_Q4K, shared_scalar_gate=None, ffn=None):
        """ffn: (gate, up, down) projections of a dense model's layer, which has no router and no expert images."""
        handle = lambda b: b.handle if b is not None else None
        w = nat.HybridLayer(mixer_input.handle, mixer_output.handle, handle(input_norm), handle(post_norm), handle(query_norm),
                            handle(key_norm), handle(convolution_weights), handle(decay_weights), handle(time_bias), handle(mixer_norm),
                            handle(router), handle(gate_images), handle(up_images), handle(down_images), expert_format, expert_down_format,
                            handle(shared_scalar_gate), *([p.handle for p in ffn] if ffn else [None, None, None]))
        check(lib.spo_hybrid_verify_set_layer(self.handle, layer, ctypes.byref(w)))
        self._keep.extend([mixer_input, mixer_output, input_norm, post_norm, router, gate_images, up_images, down_images, query_norm,
                           key_norm, convolution_weights, decay_weights, time_bias, mixer_norm, shared_scalar_gate, ffn])

    def set_penalties(self, lane, repetition=1.0, presence=0.0, frequency=0.0):
        """The sampling penalties of dispatch lane `lane` for the steps encoded after; its row of the PENALTY_WORDS buffer
        (uint32 [lanes][vocabulary]; ops.Sampling.rebuild_penalty_words makes a row) holds what they read."""
        check(lib.spo_hybrid_verify_set_penalties(self.handle, lane, repetition, presence, frequency))

    def set_admission(self, lane, constrained=False, excludes_stop_tokens=False):
        """Dispatch lane `lane` of the steps encoded after admits only the tokens of its rows of the TOKEN_MASK buffer
        (uint32 [rows][ceil(vocabulary / 32)]) and / or never selects a stop token."""
        check(lib.spo_hybrid_verify_set_admission(self.handle, lane, int(constrained), int(excludes_stop_tokens)))

    def set_stop_tokens(self, stop_tokens=()):
        """Up to four tokens that end a sequence, for the steps encoded after."""
        stops = (ctypes.c_uint32 * 4)(*(list(stop_tokens) + [0xFFFFFFFF] * 4)[:4])
        check(lib.spo_hybrid_verify_set_stop_tokens(self.handle, stops))

    def set_thinking_cutoff(self, lane, row=None, end=(), also_ends=0xFFFFFFFF, waits_for_mask=False):
        """The thinking cutoff of dispatch lane `lane` for the steps encoded after: its rows of depth `row` on select the
        tokens of `end` in order; row None clears it."""
        cutoff = None if row is None else ctypes.byref(ops.Sampling.thinking_cutoff(row, end, also_ends, waits_for_mask))
        check(lib.spo_hybrid_verify_set_thinking_cutoff(self.handle, lane, cutoff))

    def set_capture(self, layers, destination):
        """After each of `layers` (ascending) every row's output goes to its slot of `destination`, bf16 [rows][len(layers) x hidden]."""
        check(lib.spo_hybrid_verify_set_capture(self.handle, (ctypes.c_uint32 * max(len(layers), 1))(*layers), len(layers),
                                                destination.handle if destination is not None else None))
        self._keep.append(destination)

    def set_head(self, embedding_format, embedding_rows, final_norm, head):
        check(lib.spo_hybrid_verify_set_head(self.handle, embedding_format, embedding_rows.handle, final_norm.handle, head.handle))
        self._keep.extend([embedding_rows, final_norm, head])

    def _lanes(self, lanes):
        return (nat.HybridLane * len(lanes))(*[l.struct() for l in lanes])

    def step_bytes(self, lanes):
        return lib.spo_hybrid_verify_step_bytes(self.handle, self._lanes(lanes), len(lanes))

    def encode(self, lanes, commit=True, graph=None):
        graph = graph or CommandGraph()
        check(lib.spo_hybrid_verify_encode(self.handle, graph.handle, self._lanes(lanes), len(lanes), int(commit)))
        graph._keep.append(self)
        return graph

    def encode_part(self, part, index, lanes, graph=None):
        graph = graph or CommandGraph()
        check(lib.spo_hybrid_verify_encode_part(self.handle, graph.handle, part, index, self._lanes(lanes), len(lanes)))
        graph._keep.append(self)
        return graph

    def encode_prefill(self, lane, table_first, committed, tokens, parity=0, first_layer=0, layer_count=0, graph=None):
        """A chunk of `tokens` prompt tokens of lane `lane`'s sequence through layers [first_layer, first_layer + layer_count)
        (0: to the last; the embedding with first_layer 0), no head; the GDN layers go from the lane's cell of `parity` to
        its other cell. Inputs as set_prefill_block writes them."""
        graph = graph or CommandGraph()
        check(lib.spo_hybrid_verify_encode_prefill(self.handle, graph.handle, lane, table_first, committed, tokens, parity, first_layer,
                                                   layer_count))
        graph._keep.append(self)
        return graph

    set_block = DenseVerify.set_block
    set_prefill_block = DenseVerify.set_prefill_block
    results = DenseVerify.results
    _results_call = "spo_hybrid_verify_results"


(DFLASH_HIDDEN, DFLASH_LOGITS, DFLASH_SELECTOR_HIDDEN, DFLASH_FINAL_HIDDEN, DFLASH_ROPE_COS, DFLASH_ROPE_SIN, DFLASH_RINGS, DFLASH_WINDOWS,
 DFLASH_CAPTURED_TARGET_HIDDEN, DFLASH_CONTEXT_ROPE_COS, DFLASH_CONTEXT_ROPE_SIN, DFLASH_CONTEXT_HIDDEN) = range(12)


class DFlashDraft:
    """model::DFlashDraft: the draft model that proposes a step's rows, and the writers of its context. The handle owns the
    step's buffers and the rings and windows of max_lanes lanes."""

    def __init__(self, backend, layers, hidden, vocabulary, intermediate, target_layers, max_lanes, context_rows=0):
        self.backend = backend
        self.layout = nat.DFlashLayout(layers, hidden, vocabulary, intermediate, target_layers)
        self.max_lanes = max_lanes
        out = ctypes.c_void_p()
        check(lib.spo_dflash_draft_create(backend.handle, ctypes.byref(self.layout), max_lanes, context_rows, ctypes.byref(out)))
        self.handle = out
        self._keep = []

    def close(self):
        if self.handle:
            lib.spo_dflash_draft_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def buffer(self, which, index=0):
        out = ctypes.c_void_p()
        check(lib.spo_dflash_draft_buffer(self.handle, which, index, ctypes.byref(out)))
        return Buffer(out.value)

    def set_layer(self, layer, **weights):
        """weights: the projections and buffers of nat.DFLASH_LAYER_FIELDS by name."""
        w = nat.DFlashLayer(*[weights[name].handle for name in nat.DFLASH_LAYER_FIELDS])
        check(lib.spo_dflash_draft_set_layer(self.handle, layer, ctypes.byref(w)))
        self._keep.extend(weights.values())

    def set_model(self, context_projection, hidden_norm, final_norm, selector, mask_embedding, head):
        check(lib.spo_dflash_draft_set_model(self.handle, context_projection.handle, hidden_norm.handle, final_norm.handle, selector.handle,
                                             mask_embedding.handle if mask_embedding is not None else None, head.handle))
        self._keep.extend([context_projection, hidden_norm, final_norm, selector, mask_embedding, head])

    def encode_decode(self, cache_lengths, graph=None):
        graph = graph or CommandGraph()
        check(lib.spo_dflash_draft_encode_decode(self.handle, graph.handle, (ctypes.c_uint32 * len(cache_lengths))(*cache_lengths),
                                                 len(cache_lengths)))
        graph._keep.append(self)
        return graph

    def encode_context_prefill(self, lane, rows, start_position, rebuild=False, graph=None):
        graph = graph or CommandGraph()
        check(lib.spo_dflash_draft_encode_context_prefill(self.handle, graph.handle, lane, rows, start_position, int(rebuild)))
        graph._keep.append(self)
        return graph

    def encode_context_commit(self, retained_rows, lane_rows, start_positions, rows, lane_cap, graph=None):
        graph = graph or CommandGraph()
        check(lib.spo_dflash_draft_encode_context_commit(self.handle, graph.handle, retained_rows.handle, lane_rows.handle,
                                                         (ctypes.c_uint32 * len(start_positions))(*start_positions), len(start_positions),
                                                         rows, lane_cap))
        graph._keep.extend([self, retained_rows, lane_rows])
        return graph


def check_results(lanes, tokens, retained, accepted, retained_rows, vocabulary, remaining=None, step_rows=None):
    """spo_verify_check_results over host arrays: lanes [(first, rows)]."""
    arr = (nat.LaneRows * len(lanes))(*[nat.LaneRows(*l) for l in lanes])
    u32 = lambda a: np.ascontiguousarray(a, np.uint32)
    tokens, retained, accepted, retained_rows = u32(tokens), u32(retained), u32(accepted), u32(retained_rows)
    rem = u32(remaining) if remaining is not None else None
    p = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)) if a is not None else None
    rows = step_rows if step_rows is not None else len(tokens)
    check(lib.spo_verify_check_results(arr, p(rem), len(lanes), rows, vocabulary, p(tokens), p(retained), p(accepted), p(retained_rows)))
