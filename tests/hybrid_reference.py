"""A random-init hybrid decoder (Gated DeltaNet and attention mixers over a mixture-of-experts FFN) for the
parity tests: its weights, the GPU model built from them, and the oracle's evaluation of each layer.
Test infrastructure only."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np

from splash_amd import ops, verify
from tests import oracle as orc
from tests.dense_reference import device_copy


class HybridModel:
    def __init__(self, seed, hidden, vocabulary, layers, q_heads, kv_heads, head_dim, gdn_key_heads, gdn_value_heads, experts, top_k,
                 expert_ffn, attention_interval=4, rope_theta=1e6, gated_attention=False, shared_slices=0, shared_gate=False, dense_ffn=0,
                 distinct_layers=None, threads=8, file_form=False):
        """`distinct_layers` weight sets are drawn (a multiple of the attention interval, so that a set's mixer is its
        layers'), layer l holding set l % distinct_layers; all of them by default. file_form: the model as a GGUF of the
        hybrid targets holds it (hybrid_model_file) -- the router, the GDN beta and alpha gates and the GDN output norm as
        fp32 values, run by the fp32 projection and read unrounded; a GDN layer's output rows in llama.cpp's tiled head
        order, which its output projection's inputs are in; a packed row padded to whole 64-column groups."""
        self.dims = dict(hidden=hidden, vocabulary=vocabulary, layers=layers, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
                         gdn_key_heads=gdn_key_heads, gdn_value_heads=gdn_value_heads, experts=experts, top_k=top_k, expert_ffn=expert_ffn,
                         attention_interval=attention_interval)
        self.rope_theta = rope_theta
        self.gated = gated_attention       # a query head's rows of the projection: its queries, then its gate
        self.shared_slices, self.shared_gate = shared_slices, shared_gate   # the shared expert, after the routed experts
        self.dense_ffn = dense_ffn         # with experts 0: a dense SwiGLU of this width in every layer
        rng = np.random.default_rng(seed)
        self.rng = rng
        D = head_dim
        conv = (2 * gdn_key_heads + gdn_value_heads) * 128
        self.file_form = file_form
        self.packed_width = (conv + gdn_value_heads * 128 + 2 * gdn_value_heads + (63 if file_form else 15)) // (64 if file_form else 16) * (64 if file_form else 16)
        # flags: 1 tiled output heads, 4 fp32 norm weights
        self.gdn_shape = orc.gdn_shape(gdn_key_heads, gdn_value_heads, packed_width=self.packed_width, flags=5 if file_form else 0)

        pool = ThreadPoolExecutor(max(1, threads))

        def quant(n, k, fmt=orc.FMT_Q4K, scale=0.02):
            return orc.quantize_rows(fmt, (rng.standard_normal((n, k)) * scale).astype(np.float32))

        def quant_many(count, n, k):
            # a layer's experts: each from a generator spawned from the model's, quantized on the pool's threads
            work = lambda g: orc.quantize_rows(orc.FMT_Q4K, (g.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))
            return list(pool.map(work, rng.spawn(count)))

        def norm(n):
            return orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(n)).astype(np.float32))
        self.distinct = layers if distinct_layers is None else distinct_layers
        assert self.distinct == layers or self.distinct % attention_interval == 0
        self.layers = []
        for l in range(self.distinct):
            if experts:
                many = experts * expert_ffn * hidden >= (1 << 24)
                w = dict(input_norm=norm(hidden), post_norm=norm(hidden), router=quant(experts, hidden, orc.FMT_Q6K, 0.05),
                         gate=quant_many(experts + shared_slices, expert_ffn, hidden) if many else [quant(expert_ffn, hidden) for _ in range(experts + shared_slices)],
                         up=quant_many(experts + shared_slices, expert_ffn, hidden) if many else [quant(expert_ffn, hidden) for _ in range(experts + shared_slices)],
                         down=quant_many(experts + shared_slices, hidden, expert_ffn) if many else [quant(hidden, expert_ffn) for _ in range(experts + shared_slices)])
            else:
                w = dict(input_norm=norm(hidden), post_norm=norm(hidden), ffn_gate=quant(dense_ffn, hidden), ffn_up=quant(dense_ffn, hidden),
                         ffn_down=quant(hidden, dense_ffn, orc.FMT_Q6K))
            if shared_gate:
                w["shared_scalar_gate"] = (rng.standard_normal(hidden) * 0.05).astype(np.float32)
            if file_form and experts:
                w["router"] = (rng.standard_normal((experts, hidden)) * 0.05).astype(np.float32)
            if self.attends(l):
                w.update(q=quant(q_heads * D * (2 if self.gated else 1), hidden), k=quant(kv_heads * D, hidden), v=quant(kv_heads * D, hidden),
                         o=quant(hidden, q_heads * D), q_norm=norm(D), k_norm=norm(D))
            else:
                # a wider spread than a dense projection's, so that the recurrence's inputs are of order one
                w.update(mixer_in=quant(self.packed_width, hidden, scale=0.06), mixer_out=quant(hidden, gdn_value_heads * 128),
                         conv_w=orc.f32_to_bf16((rng.standard_normal((conv, 4)) * 0.4).astype(np.float32)),
                         a_scale=(-np.exp(rng.uniform(-1.0, 1.0, gdn_value_heads))).astype(np.float32),
                         dt_bias=orc.f32_to_bf16(rng.uniform(-1.0, 1.0, gdn_value_heads).astype(np.float32)), mixer_norm=norm(128))
                if file_form:
                    w.update(mixer_in=quant(conv + gdn_value_heads * 128, hidden, scale=0.06),
                             gate_rows=(rng.standard_normal((2 * gdn_value_heads, hidden)) * 0.06).astype(np.float32),
                             mixer_norm=(1 + 0.1 * rng.standard_normal(128)).astype(np.float32))
            self.layers.append(w)
        self.layers = [self.layers[l % self.distinct] for l in range(layers)]
        pool.shutdown()
        self.embedding = quant(vocabulary, hidden)
        self.final_norm = norm(hidden)
        self.head = quant(vocabulary, hidden, orc.FMT_Q6K)

    def attends(self, layer):
        return (layer + 1) % self.dims["attention_interval"] == 0

    # ------------------------------------------------------------------ GPU side
    def build_gpu(self, backend, max_lanes, pages_per_lane, prefill_rows=0):
        d = self.dims
        self.pages_per_lane = pages_per_lane
        self.physical_pages = max_lanes * pages_per_lane + 1
        gpu = verify.HybridVerify(backend, d["hidden"], d["vocabulary"], d["layers"], d["q_heads"], d["kv_heads"], d["head_dim"],
                                  d["gdn_key_heads"], d["gdn_value_heads"], d["experts"], d["top_k"], d["expert_ffn"],
                                  attention_interval=d["attention_interval"], rope_theta=self.rope_theta, max_lanes=max_lanes,
                                  gated_attention=self.gated, shared_slices=self.shared_slices, shared_gate=self.shared_gate,
                                  dense_ffn=self.dense_ffn, prefill_rows=prefill_rows,
                                  physical_pages=self.physical_pages, page_table_entries=max_lanes * pages_per_lane)
        assert gpu.dims.gdn_packed_width == self.packed_width
        self.table = np.random.default_rng(99).permutation(self.physical_pages)[:max_lanes * pages_per_lane].astype(np.uint64)
        gpu.buffer(verify.PAGE_TABLE).upload(self.table)
        D, H, F = d["head_dim"], d["hidden"], d["expert_ffn"]
        P = lambda segs, k, f32=False: ops.Projection.from_native(backend, segs, k, float32=f32)
        images = lambda fmt, natives, n, k: backend.from_array(np.concatenate([ops.pack_gguf_image(fmt, x, n, k) for x in natives]))
        built = {}
        for i, w in enumerate(self.layers):
            if i >= self.distinct:      # a layer of a set already resident: its buffers again
                args, kwargs = built[i % self.distinct]
                gpu.set_layer(i, *args, **kwargs)
                continue
            common = dict(input_norm=backend.from_array(w["input_norm"]), post_norm=backend.from_array(w["post_norm"]))
            if d["experts"]:
                common.update(router=P([(orc.FMT_Q6K, d["experts"], w["router"])], H, True), gate_images=images(orc.FMT_Q4K, w["gate"], F, H),
                              up_images=images(orc.FMT_Q4K, w["up"], F, H), down_images=images(orc.FMT_Q4K, w["down"], H, F))
            else:
                common.update(ffn=(P([(orc.FMT_Q4K, self.dense_ffn, w["ffn_gate"])], H), P([(orc.FMT_Q4K, self.dense_ffn, w["ffn_up"])], H),
                                   P([(orc.FMT_Q6K, H, w["ffn_down"])], self.dense_ffn)))
            if self.shared_gate:
                common["shared_scalar_gate"] = backend.from_array(w["shared_scalar_gate"])
            if self.attends(i):
                args = (P([(orc.FMT_Q4K, d["q_heads"] * D * (2 if self.gated else 1), w["q"]), (orc.FMT_Q4K, d["kv_heads"] * D, w["k"]),
                           (orc.FMT_Q4K, d["kv_heads"] * D, w["v"])], H), P([(orc.FMT_Q4K, H, w["o"])], d["q_heads"] * D))
                kwargs = dict(query_norm=backend.from_array(w["q_norm"]), key_norm=backend.from_array(w["k_norm"]), **common)
            else:
                args = (P([(orc.FMT_Q4K, self.packed_width, w["mixer_in"])], H), P([(orc.FMT_Q4K, H, w["mixer_out"])], d["gdn_value_heads"] * 128))
                kwargs = dict(convolution_weights=backend.from_array(w["conv_w"]), decay_weights=backend.from_array(w["a_scale"]),
                              time_bias=backend.from_array(w["dt_bias"]), mixer_norm=backend.from_array(w["mixer_norm"]), **common)
            built[i] = (args, kwargs)
            gpu.set_layer(i, *args, **kwargs)
        gpu.set_head(orc.FMT_Q4K, backend.from_array(self.embedding), backend.from_array(self.final_norm),
                     P([(orc.FMT_Q6K, d["vocabulary"], self.head)], H, True))
        self.gpu = gpu
        return gpu

    def build_gpu_from_file(self, backend, path, max_lanes, pages_per_lane, prefill_rows=0):
        """The driver of the model's GGUF (hybrid_model_file): geometry and weights as the loader reads them."""
        from splash_amd import gguf
        self.pages_per_lane = pages_per_lane
        self.physical_pages = max_lanes * pages_per_lane + 1
        gpu = verify.HybridVerify.from_gguf(backend, gguf.GgufFile(str(path)), max_lanes=max_lanes, physical_pages=self.physical_pages,
                                            page_table_entries=max_lanes * pages_per_lane, prefill_rows=prefill_rows)
        assert gpu.dims.gdn_packed_width == self.packed_width
        self.table = np.random.default_rng(99).permutation(self.physical_pages)[:max_lanes * pages_per_lane].astype(np.uint64)
        gpu.buffer(verify.PAGE_TABLE).upload(self.table)
        self.gpu = gpu
        return gpu

    def seed_context(self, rng, distinct=None):
        """A seeded INT8 context in every physical page of every attention layer; `distinct` contexts are drawn, attention
        layer a holding context a % distinct (copied on the device)."""
        d, gpu = self.dims, self.gpu
        H, D, PT = d["kv_heads"], d["head_dim"], ops.PAGE_TOKENS
        helper = ops.KvPages.__new__(ops.KvPages)
        helper.kv_heads, helper.head_dim, helper.page_bytes = H, D, gpu.page_bytes
        attention_layers = d["layers"] // d["attention_interval"]
        distinct = attention_layers if distinct is None else distinct
        drawn = []
        for layer in range(distinct):
            def quant(x):
                mx = np.abs(x).max(axis=-1, keepdims=True)
                codes = np.clip(np.rint(x * np.float32(127.0) / mx), -127, 127).astype(np.int8)
                return codes, (mx[..., 0] / np.float32(127.0)).astype(np.float16).astype(np.float32)
            (kc, ks), (vc, vs) = (quant(rng.standard_normal((self.physical_pages, H, PT, D)).astype(np.float32)) for _ in range(2))
            drawn.append([kc, ks, vc, vs])
            gpu.buffer(verify.KV_POOL, layer).upload(helper.pack_pages(kc, ks, vc, vs))
        for layer in range(distinct, attention_layers):
            device_copy(gpu.backend, gpu.buffer(verify.KV_POOL, layer % distinct), gpu.buffer(verify.KV_POOL, layer),
                        self.physical_pages * gpu.page_bytes)
        self.context = [drawn[a % distinct] for a in range(attention_layers)]

    def seed_states(self, rng, lanes, parity=0):
        """Random recurrent states and convolution carries in every lane's cell of `parity`."""
        gpu, shape = self.gpu, self.gdn_shape
        states = gpu.buffer(verify.GDN_STATES)
        for lane in range(lanes):
            for g in range(gpu.gdn_layers):
                conv = orc.f32_to_bf16(rng.standard_normal((3, shape.conv_dim)).astype(np.float32))
                state = (rng.standard_normal((shape.value_heads, 128, 128)) * 0.05).astype(np.float32)
                base = gpu.cell_offset(lane, parity)
                states.upload(conv, base + g * gpu.strides.convolution_layer_bytes)
                states.upload(state, base + gpu.strides.convolution_state_bytes + g * gpu.strides.recurrent_layer_bytes)

    def read_cell(self, lane, parity, gdn_layer):
        gpu, shape = self.gpu, self.gdn_shape
        st = gpu.strides
        states = gpu.buffer(verify.GDN_STATES)
        base = gpu.cell_offset(lane, parity)
        conv = states.download(np.uint16, 3 * shape.conv_dim, base + gdn_layer * st.convolution_layer_bytes).reshape(3, shape.conv_dim)
        at = base + st.convolution_state_bytes + gdn_layer * st.recurrent_layer_bytes
        return conv.copy(), states.download(np.float32, st.recurrent_layer_bytes // 4, at).reshape(shape.value_heads, 128, 128).copy()

    def read_tape(self, lane, parity, gdn_layer):
        gpu = self.gpu
        return gpu.buffer(verify.GDN_TAPE).download(np.uint8, gpu.tape_layer_bytes, gpu.tape_offset(lane, parity, gdn_layer)).copy()

    # ------------------------------------------------------------------ oracle side
    def _project(self, fmt, native, x_bits, n):
        return orc.gemm(fmt, native, x_bits, n, want=("exact",))["exact"]

    def oracle_embedding(self, tokens):
        return orc.embed(orc.FMT_Q4K, self.embedding, self.dims["vocabulary"], self.dims["hidden"], tokens)

    def oracle_mixer_input(self, hidden, li):
        w, d = self.layers[li], self.dims
        n = orc.rms_norm(hidden, w["input_norm"])
        if self.attends(li):
            D = d["head_dim"]
            out = np.concatenate([self._project(orc.FMT_Q4K, w[name], n, width) for name, width in
                                  (("q", d["q_heads"] * D * (2 if self.gated else 1)), ("k", d["kv_heads"] * D), ("v", d["kv_heads"] * D))], axis=1)
        elif self.file_form:
            # q | k | v | z from the quantized rows, beta | alpha from the rows of floats, the padding columns nobody reads
            width = (2 * d["gdn_key_heads"] + 2 * d["gdn_value_heads"]) * 128
            out = np.concatenate([self._project(orc.FMT_Q4K, w["mixer_in"], n, width), orc.float_projection(n, w["gate_rows"]),
                                  np.zeros((n.shape[0], self.packed_width - width - 2 * d["gdn_value_heads"]))], axis=1)
        else:
            out = self._project(orc.FMT_Q4K, w["mixer_in"], n, self.packed_width)
        return orc.f32_to_bf16(out.astype(np.float32))

    def oracle_attention(self, packed, li, lanes):
        """Every lane's attention rows; stores the blocks' K/V into the layer's context arrays."""
        d, w = self.dims, self.layers[li]
        D, pairs = d["head_dim"], d["head_dim"] // 2
        kc, ks, vc, vs = self.context[li // d["attention_interval"]]
        inv = np.array([self.rope_theta ** (-i / pairs) for i in range(pairs)]).astype(np.float32)
        gates = None
        if self.gated:
            heads = packed[:, :d["q_heads"] * 2 * D].reshape(-1, d["q_heads"], 2, D)
            gates = orc.bf16_to_f32(heads[:, :, 1]).reshape(-1, d["q_heads"] * D)
            packed = np.concatenate([heads[:, :, 0].reshape(-1, d["q_heads"] * D), packed[:, d["q_heads"] * 2 * D:]], axis=1)
        out, first = [], 0
        for lane in lanes:
            rows, committed = lane.rows, lane.committed
            table = self.table[lane.table_first:lane.table_first + self.pages_per_lane].astype(np.uint32)
            pos = (committed + np.arange(rows)).astype(np.float32)
            angle = (pos[:, None] * inv[None, :]).astype(np.float32)
            cosv, sinv = np.cos(angle.astype(np.float64)).astype(np.float32), np.sin(angle.astype(np.float64)).astype(np.float32)
            q, kf, vf = orc.attention_prepare(d["q_heads"], d["kv_heads"], D, packed[first:first + rows], w["q_norm"], w["k_norm"], cosv, sinv, pairs)
            kcod, kscl = orc.kv_quantize(kf)
            vcod, vscl = orc.kv_quantize(vf)
            for r in range(rows):
                t = committed + r
                p, s = table[t // ops.PAGE_TOKENS], t % ops.PAGE_TOKENS
                kc[p, :, s], ks[p, :, s], vc[p, :, s], vs[p, :, s] = kcod[r], kscl[r], vcod[r], vscl[r]
            anc = np.array([(2 << r) - 1 for r in range(rows)], dtype=np.uint32)
            attn, _ = orc.attention(q, kc, ks, vc, vs, table, anc, committed, want64=False)
            out.append(attn.reshape(rows, d["q_heads"] * D))
            first += rows
        out = np.concatenate(out)
        if self.gated:      # attention_gate.h:27-31: bf16(bf16(value) * sigmoid(gate))
            sigmoid = np.float32(1) / (np.float32(1) + np.exp2(np.float32(-1.44269504089) * gates))
            out = orc.f32_to_bf16((orc.bf16_to_f32(out) * sigmoid).astype(np.float32))
        return out

    def oracle_attention_chunk(self, packed, li, table_first, committed):
        """A prompt chunk's attention rows: every row's K/V stored into the layer's context arrays, then each tile of
        sixteen rows a block of the sequence that ends at its last row."""
        d, w = self.dims, self.layers[li]
        D, pairs, tokens = d["head_dim"], d["head_dim"] // 2, packed.shape[0]
        kc, ks, vc, vs = self.context[li // d["attention_interval"]]
        inv = np.array([self.rope_theta ** (-i / pairs) for i in range(pairs)]).astype(np.float32)
        gates = None
        if self.gated:
            heads = packed[:, :d["q_heads"] * 2 * D].reshape(-1, d["q_heads"], 2, D)
            gates = orc.bf16_to_f32(heads[:, :, 1]).reshape(-1, d["q_heads"] * D)
            packed = np.concatenate([heads[:, :, 0].reshape(-1, d["q_heads"] * D), packed[:, d["q_heads"] * 2 * D:]], axis=1)
        table = self.table[table_first:table_first + self.pages_per_lane].astype(np.uint32)
        angle = ((committed + np.arange(tokens)).astype(np.float32)[:, None] * inv[None, :]).astype(np.float32)
        cosv, sinv = np.cos(angle.astype(np.float64)).astype(np.float32), np.sin(angle.astype(np.float64)).astype(np.float32)
        q, kf, vf = orc.attention_prepare(d["q_heads"], d["kv_heads"], D, packed, w["q_norm"], w["k_norm"], cosv, sinv, pairs)
        kcod, kscl = orc.kv_quantize(kf)
        vcod, vscl = orc.kv_quantize(vf)
        for r in range(tokens):
            t = committed + r
            p, s = table[t // ops.PAGE_TOKENS], t % ops.PAGE_TOKENS
            kc[p, :, s], ks[p, :, s], vc[p, :, s], vs[p, :, s] = kcod[r], kscl[r], vcod[r], vscl[r]
        out = []
        for first in range(0, tokens, 16):
            rows = min(16, tokens - first)
            anc = np.array([(2 << r) - 1 for r in range(rows)], dtype=np.uint32)
            attn, _ = orc.attention(np.ascontiguousarray(q[first:first + rows]), kc, ks, vc, vs, table, anc, committed + first, want64=False)
            out.append(attn.reshape(rows, d["q_heads"] * D))
        out = np.concatenate(out)
        if self.gated:
            sigmoid = np.float32(1) / (np.float32(1) + np.exp2(np.float32(-1.44269504089) * gates))
            out = orc.f32_to_bf16((orc.bf16_to_f32(out) * sigmoid).astype(np.float32))
        return out

    def oracle_gdn(self, packed, li, lanes, cells, tapes):
        """Every lane's GDN rows from its cell (conv, state) and pending tape; returns (rows, [(conv, state, tape)] it leaves)."""
        w = self.layers[li]
        out, left, first = [], [], 0
        for lane, (conv_in, state_in), tape in zip(lanes, cells, tapes):
            conv, state, step_tape, hidden = orc.gdn_decode(self.gdn_shape, packed[first:first + lane.rows], w["conv_w"], w["a_scale"], w["dt_bias"],
                                                            w["mixer_norm"], conv_in, state_in, pending_tape=tape if lane.pending_path else None,
                                                            pending_path=lane.pending_path)
            out.append(hidden)
            left.append((conv, state, step_tape))
            first += lane.rows
        return np.concatenate(out), left

    def oracle_mixer_output(self, mixed, hidden, li):
        w = self.layers[li]
        o = self._project(orc.FMT_Q4K, w["o"] if self.attends(li) else w["mixer_out"], mixed, self.dims["hidden"])
        return orc.f32_to_bf16((o + orc.bf16_to_f32(hidden)).astype(np.float32))

    def oracle_ffn(self, hidden1, li):
        """(router scores, output rows) of the layer's mixture of experts."""
        w, d = self.layers[li], self.dims
        n = orc.rms_norm(hidden1, w["post_norm"])
        if not d["experts"]:   # a dense SwiGLU: no router
            mid = orc.swiglu(self._project(orc.FMT_Q4K, w["ffn_gate"], n, self.dense_ffn), self._project(orc.FMT_Q4K, w["ffn_up"], n, self.dense_ffn))
            down = self._project(orc.FMT_Q6K, w["ffn_down"], mid, d["hidden"])
            return None, orc.f32_to_bf16((down + orc.bf16_to_f32(hidden1)).astype(np.float32))
        scores = orc.float_projection(n, w["router"]) if self.file_form else self._project(orc.FMT_Q6K, w["router"], n, d["experts"]).astype(np.float32)
        _, _, _, out = orc.moe_layer(n, hidden1, scores, d["top_k"], w["gate"], w["up"], w["down"], d["expert_ffn"],
                                     shared=self.shared_slices, shared_gate=w.get("shared_scalar_gate"))
        return scores, out

    def oracle_head(self, hidden):
        n = orc.rms_norm(hidden, self.final_norm)
        return self._project(orc.FMT_Q6K, self.head, n, self.dims["vocabulary"])


def hybrid_model_file(path, model, router_kind="f32", fused_gate_up=False, skip=(), extra=(), more_metadata=()):
    """A file_form HybridModel's GGUF as llama.cpp writes a qwen35moe (or, without experts, qwen35) model: the value heads of
    attn_qkv, attn_gate, ssm_beta, ssm_alpha, ssm_conv1d, ssm_a and ssm_dt.bias in tiled order (value head j of key head
    h at j * key heads + h), which the model holds grouped; the experts' tensors of three dimensions."""
    from tests import gguf_writer as gw
    assert model.file_form
    d = model.dims
    H, D, V, KH, VH = d["hidden"], d["head_dim"], d["vocabulary"], d["gdn_key_heads"], d["gdn_value_heads"]
    E, F, S = d["experts"], d["expert_ffn"], model.shared_slices
    per, conv_rows, value_rows = VH // KH, (2 * KH + VH) * 128, VH * 128
    arch = "qwen35moe" if E else "qwen35"
    f32 = lambda bits: orc.bf16_to_f32(bits).astype(np.float32)
    # grouped head g = h * per + j  ->  tiled position j * KH + h
    order = [h * per + j for j in range(per) for h in range(KH)]

    def tiled(rows, head_rows, first=0):
        """`rows` (an array of rows; natives as [rows][row bytes]) with the value heads from row `first` on in tiled order."""
        rows = np.asarray(rows)
        heads = rows[first:].reshape(VH, head_rows, *rows.shape[1:])
        return np.concatenate([rows[:first], heads[order].reshape(VH * head_rows, *rows.shape[1:])])
    native_rows = lambda native, n: np.asarray(native).reshape(n, -1)
    tensors = [("token_embd.weight", gw.GGML_Q4_K, [H, V], model.embedding), ("output_norm.weight", gw.GGML_F32, [H], f32(model.final_norm)),
               ("output.weight", gw.GGML_Q6_K, [H, V], model.head)]
    for i, w in enumerate(model.layers):
        p = f"blk.{i}."
        tensors += [(p + "attn_norm.weight", gw.GGML_F32, [H], f32(w["input_norm"])),
                    (p + "post_attention_norm.weight", gw.GGML_F32, [H], f32(w["post_norm"]))]
        if model.attends(i):
            q_rows = d["q_heads"] * D * (2 if model.gated else 1)
            tensors += [(p + "attn_q.weight", gw.GGML_Q4_K, [H, q_rows], w["q"]), (p + "attn_k.weight", gw.GGML_Q4_K, [H, d["kv_heads"] * D], w["k"]),
                        (p + "attn_v.weight", gw.GGML_Q4_K, [H, d["kv_heads"] * D], w["v"]),
                        (p + "attn_q_norm.weight", gw.GGML_F32, [D], f32(w["q_norm"])), (p + "attn_k_norm.weight", gw.GGML_F32, [D], f32(w["k_norm"])),
                        (p + "attn_output.weight", gw.GGML_Q4_K, [d["q_heads"] * D, H], w["o"])]
        else:
            rows = native_rows(w["mixer_in"], conv_rows + value_rows)
            tensors += [(p + "attn_qkv.weight", gw.GGML_Q4_K, [H, conv_rows], tiled(rows[:conv_rows], 128, first=2 * KH * 128)),
                        (p + "attn_gate.weight", gw.GGML_Q4_K, [H, value_rows], tiled(rows[conv_rows:], 128)),
                        (p + "ssm_beta.weight", gw.GGML_F32, [H, VH], tiled(w["gate_rows"][:VH], 1)),
                        (p + "ssm_alpha.weight", gw.GGML_F32, [H, VH], tiled(w["gate_rows"][VH:], 1)),
                        (p + "ssm_conv1d.weight", gw.GGML_F32, [4, conv_rows], tiled(f32(w["conv_w"]), 128, first=2 * KH * 128)),
                        (p + "ssm_a", gw.GGML_F32, [VH], tiled(w["a_scale"], 1)), (p + "ssm_dt.bias", gw.GGML_F32, [VH], tiled(f32(w["dt_bias"]), 1)),
                        (p + "ssm_norm.weight", gw.GGML_F32, [128], w["mixer_norm"]),
                        (p + "ssm_out.weight", gw.GGML_Q4_K, [value_rows, H], w["mixer_out"])]
        if not E:
            tensors += [(p + "ffn_gate.weight", gw.GGML_Q4_K, [H, model.dense_ffn], w["ffn_gate"]),
                        (p + "ffn_up.weight", gw.GGML_Q4_K, [H, model.dense_ffn], w["ffn_up"]),
                        (p + "ffn_down.weight", gw.GGML_Q6_K, [model.dense_ffn, H], w["ffn_down"])]
            continue
        router = {"f32": (gw.GGML_F32, w["router"]), "bf16": (gw.GGML_BF16, orc.f32_to_bf16(w["router"]))}[router_kind]
        tensors.append((p + "ffn_gate_inp.weight", router[0], [H, E], router[1]))
        cat = lambda natives: np.concatenate([np.asarray(x).ravel() for x in natives])
        if fused_gate_up:    # expert e's gate rows, then its up rows
            tensors.append((p + "ffn_gate_up_exps.weight", gw.GGML_Q4_K, [H, 2 * F, E], cat([x for e in range(E) for x in (w["gate"][e], w["up"][e])])))
        else:
            tensors += [(p + "ffn_gate_exps.weight", gw.GGML_Q4_K, [H, F, E], cat(w["gate"][:E])), (p + "ffn_up_exps.weight", gw.GGML_Q4_K, [H, F, E], cat(w["up"][:E]))]
        tensors.append((p + "ffn_down_exps.weight", gw.GGML_Q4_K, [F, H, E], cat(w["down"][:E])))
        if S:
            tensors += [(p + "ffn_gate_shexp.weight", gw.GGML_Q4_K, [H, S * F], cat(w["gate"][E:])), (p + "ffn_up_shexp.weight", gw.GGML_Q4_K, [H, S * F], cat(w["up"][E:])),
                        # a row of the shared down projection holds every slice's inputs, slice after slice
                        (p + "ffn_down_shexp.weight", gw.GGML_Q4_K, [S * F, H], np.concatenate([native_rows(x, H) for x in w["down"][E:]], axis=1))]
        if model.shared_gate:
            tensors.append((p + "ffn_gate_inp_shexp.weight", gw.GGML_F32, [H], w["shared_scalar_gate"]))
    tensors = [t for t in tensors if t[0] not in skip] + list(extra)
    a = arch + "."
    metadata = [("general.architecture", gw.STRING, arch), (a + "block_count", gw.U32, d["layers"]), (a + "embedding_length", gw.U32, H),
                (a + "attention.head_count", gw.U32, d["q_heads"]), (a + "attention.head_count_kv", gw.U32, d["kv_heads"]),
                (a + "attention.key_length", gw.U32, D), (a + "attention.value_length", gw.U32, D), (a + "rope.dimension_count", gw.U32, D),
                (a + "attention.layer_norm_rms_epsilon", gw.F32, 1e-6), (a + "rope.freq_base", gw.F32, model.rope_theta),
                (a + "full_attention_interval", gw.U32, d["attention_interval"]), (a + "ssm.conv_kernel", gw.U32, 4),
                (a + "ssm.group_count", gw.U32, KH), (a + "ssm.time_step_rank", gw.U32, VH), (a + "ssm.state_size", gw.U32, 128),
                (a + "ssm.inner_size", gw.U32, VH * 128)]
    if E:
        metadata += [(a + "expert_count", gw.U32, E), (a + "expert_used_count", gw.U32, d["top_k"]), (a + "expert_feed_forward_length", gw.U32, F),
                     (a + "expert_shared_feed_forward_length", gw.U32, S * F)]
    else:
        metadata.append((a + "feed_forward_length", gw.U32, model.dense_ffn))
    gw.write_gguf(path, metadata + list(more_metadata), tensors)
    return path
