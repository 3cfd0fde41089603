"""A random-init dense decoder for the parity tests: its weights (N(0, 0.02) quantized to Q4_K by the
oracle's quantizer), the GPU model built from them, and the oracle's own evaluation of the step.
Test infrastructure only."""
import numpy as np

from splash_amd import ops, verify
from tests import oracle as orc


class DenseModel:
    def __init__(self, seed, hidden, q_heads, kv_heads, head_dim, ffn, vocabulary, layers, rope_theta=1e6, down_format=orc.FMT_Q4K):
        self.dims = dict(hidden=hidden, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, ffn=ffn, vocabulary=vocabulary, layers=layers)
        self.rope_theta = rope_theta
        rng = np.random.default_rng(seed)
        self.rng = rng
        D = head_dim

        def quant(n, k, fmt=orc.FMT_Q4K):
            return orc.quantize_rows(fmt, (rng.standard_normal((n, k)) * 0.02).astype(np.float32))

        def norm(n):
            return orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(n)).astype(np.float32))
        self.down_format = down_format
        self.layers = []
        for _ in range(layers):
            self.layers.append(dict(q=quant(q_heads * D, hidden), k=quant(kv_heads * D, hidden), v=quant(kv_heads * D, hidden),
                                    o=quant(hidden, q_heads * D), gate=quant(ffn, hidden), up=quant(ffn, hidden),
                                    down=quant(hidden, ffn, down_format), input_norm=norm(hidden), post_norm=norm(hidden),
                                    q_norm=norm(D), k_norm=norm(D)))
        self.embedding = quant(vocabulary, hidden)
        self.final_norm = norm(hidden)
        self.head = quant(vocabulary, hidden, orc.FMT_Q6K)
        self.context = None

    # ------------------------------------------------------------------ GPU side
    def build_gpu(self, backend, max_lanes, context_tokens):
        d = self.dims
        pages = (context_tokens + ops.PAGE_TOKENS - 1) // ops.PAGE_TOKENS
        self.physical_pages = pages + 1
        gpu = verify.DenseVerify(backend, d["hidden"], d["q_heads"], d["kv_heads"], d["head_dim"], d["ffn"], d["vocabulary"],
                                 d["layers"], rope_theta=self.rope_theta, max_lanes=max_lanes, physical_pages=self.physical_pages,
                                 page_table_entries=pages)
        self.table = np.random.default_rng(99).permutation(self.physical_pages)[:pages].astype(np.uint64)
        gpu.buffer(verify.PAGE_TABLE).upload(self.table)
        D, H = d["head_dim"], d["hidden"]
        P = lambda segs, k, f32=False: ops.Projection.from_native(backend, segs, k, float32=f32)
        for i, w in enumerate(self.layers):
            gpu.set_layer(i, P([(orc.FMT_Q4K, d["q_heads"] * D, w["q"]), (orc.FMT_Q4K, d["kv_heads"] * D, w["k"]),
                                (orc.FMT_Q4K, d["kv_heads"] * D, w["v"])], H),
                          P([(orc.FMT_Q4K, H, w["o"])], d["q_heads"] * D), P([(orc.FMT_Q4K, d["ffn"], w["gate"])], H),
                          P([(orc.FMT_Q4K, d["ffn"], w["up"])], H), P([(self.down_format, H, w["down"])], d["ffn"]),
                          backend.from_array(w["input_norm"]), backend.from_array(w["post_norm"]),
                          backend.from_array(w["q_norm"]), backend.from_array(w["k_norm"]))
        gpu.set_head(orc.FMT_Q4K, backend.from_array(self.embedding), backend.from_array(self.final_norm),
                     P([(orc.FMT_Q6K, d["vocabulary"], self.head)], H, True))
        return gpu

    def seed_context(self, gpu, tokens, rng):
        """A seeded INT8 context of `tokens` tokens per layer (K/V ~ N(0, 1) quantized by the store rule)."""
        d = self.dims
        H, D, PT = d["kv_heads"], d["head_dim"], ops.PAGE_TOKENS
        self.context = []
        helper = ops.KvPages.__new__(ops.KvPages)
        helper.kv_heads, helper.head_dim, helper.page_bytes = H, D, gpu.page_bytes
        for layer in range(d["layers"]):
            k = rng.standard_normal((self.physical_pages, H, PT, D)).astype(np.float32)
            v = rng.standard_normal((self.physical_pages, H, PT, D)).astype(np.float32)

            def quant(x):
                mx = np.abs(x).max(axis=-1, keepdims=True)
                codes = np.clip(np.rint(x * np.float32(127.0) / mx), -127, 127).astype(np.int8)
                return codes, (mx[..., 0] / np.float32(127.0)).astype(np.float16).astype(np.float32)
            (kc, ks), (vc, vs) = quant(k), quant(v)
            self.context.append([kc, ks, vc, vs])
            gpu.buffer(verify.KV_POOL, layer).upload(helper.pack_pages(kc, ks, vc, vs))

    # ------------------------------------------------------------------ oracle side
    def _project(self, fmt, native, x_bits, n):
        return orc.gemm(fmt, native, x_bits, n, want=("exact",))["exact"]

    def _rope(self, rows, committed):
        pairs = self.dims["head_dim"] // 2
        inv = np.array([self.rope_theta ** (-i / pairs) for i in range(pairs)]).astype(np.float32)
        pos = (committed + np.arange(rows)).astype(np.float32)
        angle = (pos[:, None] * inv[None, :]).astype(np.float32)
        return np.cos(angle.astype(np.float64)).astype(np.float32), np.sin(angle.astype(np.float64)).astype(np.float32), pairs

    def oracle_embedding(self, tokens):
        return orc.embed(orc.FMT_Q4K, self.embedding, self.dims["vocabulary"], self.dims["hidden"], tokens)

    def oracle_layer(self, hidden, li, committed):
        """One layer from bf16 hidden rows (uint16 bits): stores the block's K/V into the layer's context."""
        d, w = self.dims, self.layers[li]
        rows, H, D = hidden.shape[0], d["hidden"], d["head_dim"]
        cosv, sinv, pairs = self._rope(rows, committed)
        anc = np.array([(2 << r) - 1 for r in range(rows)], dtype=np.uint32)
        table = self.table.astype(np.uint32)
        n = orc.rms_norm(hidden, w["input_norm"])
        qkv = np.concatenate([self._project(orc.FMT_Q4K, w[name], n, w_n) for name, w_n in
                              (("q", d["q_heads"] * D), ("k", d["kv_heads"] * D), ("v", d["kv_heads"] * D))], axis=1)
        qkv = orc.f32_to_bf16(qkv.astype(np.float32))
        q, kf, vf = orc.attention_prepare(d["q_heads"], d["kv_heads"], D, qkv, w["q_norm"], w["k_norm"], cosv, sinv, pairs)
        kc, ks, vc, vs = self.context[li]
        kcod, kscl = orc.kv_quantize(kf)
        vcod, vscl = orc.kv_quantize(vf)
        for r in range(rows):
            t = committed + r
            p, s = table[t // ops.PAGE_TOKENS], t % ops.PAGE_TOKENS
            kc[p, :, s], ks[p, :, s], vc[p, :, s], vs[p, :, s] = kcod[r], kscl[r], vcod[r], vscl[r]
        attn, _ = orc.attention(q, kc, ks, vc, vs, table, anc, committed, want64=False)
        attn = attn.reshape(rows, d["q_heads"] * D)
        o = self._project(orc.FMT_Q4K, w["o"], attn, H)
        hidden1 = orc.f32_to_bf16((o + orc.bf16_to_f32(hidden)).astype(np.float32))
        n = orc.rms_norm(hidden1, w["post_norm"])
        gate = self._project(orc.FMT_Q4K, w["gate"], n, d["ffn"]).astype(np.float32)
        up = self._project(orc.FMT_Q4K, w["up"], n, d["ffn"]).astype(np.float32)
        g16, u16 = orc.bf16_to_f32(orc.f32_to_bf16(gate)), orc.bf16_to_f32(orc.f32_to_bf16(up))
        inter = orc.f32_to_bf16((u16 * (g16 / (1 + np.exp2(np.float32(-1.4426950408889634) * g16)))).astype(np.float32))
        down = self._project(self.down_format, w["down"], inter, H)
        return orc.f32_to_bf16((down + orc.bf16_to_f32(hidden1)).astype(np.float32))

    def oracle_head(self, hidden):
        n = orc.rms_norm(hidden, self.final_norm)
        return self._project(orc.FMT_Q6K, self.head, n, self.dims["vocabulary"])

    def oracle_step(self, tokens, committed):
        rows = len(tokens)
        hidden = self.oracle_embedding(tokens)
        for li in range(self.dims["layers"]):
            hidden = self.oracle_layer(hidden, li, committed)
        logits = self.oracle_head(hidden)
        selected = np.array([orc.argmax(logits[r].astype(np.float32)) for r in range(rows)], dtype=np.uint32)
        kept, accepted, mask = orc.accept_tree(ops.chain_tree_rows([rows]), tokens, selected)
        return dict(logits=logits, selected=selected, kept=kept, accepted=accepted, retained_rows=mask)
