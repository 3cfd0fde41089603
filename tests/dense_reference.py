"""A random-init dense decoder for the parity tests: its weights (N(0, 0.02) quantized to Q4_K by the
oracle's quantizer), the GPU model built from them, and the oracle's own evaluation of the step.
Test infrastructure only."""
import ctypes
from concurrent.futures import ThreadPoolExecutor

import numpy as np

import splash_amd
from splash_amd import ops, verify
from tests import oracle as orc


def device_copy(backend, source, destination, nbytes):
    """destination <- source on the device (the copy_bytes kernel, 16-byte vectors)."""
    class P(ctypes.Structure):
        _fields_ = [("vectors", ctypes.c_uint64)]
    g = splash_amd.CommandGraph()
    g.add("copy_bytes", [source, destination], P(nbytes // 16), (2048, 1, 1), (256, 1, 1))
    backend.run(g)


class DenseModel:
    def __init__(self, seed, hidden, q_heads, kv_heads, head_dim, ffn, vocabulary, layers, rope_theta=1e6, down_format=orc.FMT_Q4K,
                 distinct_layers=None, threads=8):
        """`distinct_layers` weight sets are drawn and layer l holds set l % distinct_layers (all of them by default):
        a 64-layer model of the headline shape shares one set, as its HBM copy is what a layer adds, not new arithmetic."""
        self.dims = dict(hidden=hidden, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, ffn=ffn, vocabulary=vocabulary, layers=layers)
        self.rope_theta = rope_theta
        rng = np.random.default_rng(seed)
        self.rng = rng
        D = head_dim
        pool = ThreadPoolExecutor(max(1, threads))

        def quant(n, k, fmt=orc.FMT_Q4K):
            # large tensors: row chunks on the pool's threads, each with a generator spawned from the model's
            if n * k < (1 << 22):
                return orc.quantize_rows(fmt, (rng.standard_normal((n, k)) * 0.02).astype(np.float32))
            chunk = max(16, ((1 << 24) // k) // 16 * 16)
            starts = list(range(0, n, chunk))
            seeds = rng.spawn(len(starts))
            work = lambda a: orc.quantize_rows(fmt, (a[1].standard_normal((min(chunk, n - a[0]), k), dtype=np.float32) * np.float32(0.02)))
            return np.concatenate(list(pool.map(work, zip(starts, seeds))))

        def norm(n):
            return orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(n)).astype(np.float32))
        self.down_format = down_format
        distinct = layers if distinct_layers is None else distinct_layers
        sets = []
        for _ in range(distinct):
            sets.append(dict(q=quant(q_heads * D, hidden), k=quant(kv_heads * D, hidden), v=quant(kv_heads * D, hidden),
                             o=quant(hidden, q_heads * D), gate=quant(ffn, hidden), up=quant(ffn, hidden),
                             down=quant(hidden, ffn, down_format), input_norm=norm(hidden), post_norm=norm(hidden),
                             q_norm=norm(D), k_norm=norm(D)))
        self.distinct = distinct
        self.layers = [sets[l % distinct] for l in range(layers)]
        self.embedding = quant(vocabulary, hidden)
        self.final_norm = norm(hidden)
        self.head = quant(vocabulary, hidden, orc.FMT_Q6K)
        self.context = None
        pool.shutdown()

    # ------------------------------------------------------------------ GPU side
    def build_gpu(self, backend, max_lanes, context_tokens, prefill_rows=0):
        """context_tokens: the most tokens a lane's pages hold, one number for every lane or a list with one a lane;
        lane i's logical pages start at entry self.table_first[i] of the page table."""
        d = self.dims
        per_lane = list(context_tokens) if isinstance(context_tokens, (list, tuple)) else [context_tokens] * max_lanes
        lane_pages = [(t + ops.PAGE_TOKENS - 1) // ops.PAGE_TOKENS for t in per_lane]
        pages = sum(lane_pages)
        self.table_first = [sum(lane_pages[:i]) for i in range(len(lane_pages))]
        self.physical_pages = pages + 1
        gpu = verify.DenseVerify(backend, d["hidden"], d["q_heads"], d["kv_heads"], d["head_dim"], d["ffn"], d["vocabulary"],
                                 d["layers"], rope_theta=self.rope_theta, max_lanes=max_lanes, physical_pages=self.physical_pages,
                                 page_table_entries=pages, prefill_rows=prefill_rows)
        self.table = np.random.default_rng(99).permutation(self.physical_pages)[:pages].astype(np.uint64)
        gpu.buffer(verify.PAGE_TABLE).upload(self.table)
        D, H = d["head_dim"], d["hidden"]
        P = lambda segs, k, f32=False: ops.Projection.from_native(backend, segs, k, float32=f32)
        built = []
        for w in self.layers[:self.distinct]:
            built.append((P([(orc.FMT_Q4K, d["q_heads"] * D, w["q"]), (orc.FMT_Q4K, d["kv_heads"] * D, w["k"]),
                             (orc.FMT_Q4K, d["kv_heads"] * D, w["v"])], H),
                          P([(orc.FMT_Q4K, H, w["o"])], d["q_heads"] * D), P([(orc.FMT_Q4K, d["ffn"], w["gate"])], H),
                          P([(orc.FMT_Q4K, d["ffn"], w["up"])], H), P([(self.down_format, H, w["down"])], d["ffn"]),
                          backend.from_array(w["input_norm"]), backend.from_array(w["post_norm"]),
                          backend.from_array(w["q_norm"]), backend.from_array(w["k_norm"])))
        for i in range(d["layers"]):
            gpu.set_layer(i, *built[i % self.distinct])
        gpu.set_head(orc.FMT_Q4K, backend.from_array(self.embedding), backend.from_array(self.final_norm),
                     P([(orc.FMT_Q6K, d["vocabulary"], self.head)], H, True))
        return gpu

    def seed_context(self, gpu, tokens, rng, distinct=None):
        """A seeded INT8 context per layer (K/V ~ N(0, 1) quantized by the store rule) over every physical page.
        `distinct` contexts are drawn, layer l holding context l % distinct (copied on the device)."""
        d = self.dims
        H, D, PT = d["kv_heads"], d["head_dim"], ops.PAGE_TOKENS
        distinct = d["layers"] if distinct is None else distinct
        drawn = []
        helper = ops.KvPages.__new__(ops.KvPages)
        helper.kv_heads, helper.head_dim, helper.page_bytes = H, D, gpu.page_bytes
        for layer in range(distinct):
            def quant(x):
                mx = np.abs(x).max(axis=-1, keepdims=True)
                codes = np.clip(np.rint(x * np.float32(127.0) / mx), -127, 127).astype(np.int8)
                return codes, (mx[..., 0] / np.float32(127.0)).astype(np.float16).astype(np.float32)
            kc, ks = quant(rng.standard_normal((self.physical_pages, H, PT, D), dtype=np.float32))
            vc, vs = quant(rng.standard_normal((self.physical_pages, H, PT, D), dtype=np.float32))
            drawn.append([kc, ks, vc, vs])
            gpu.buffer(verify.KV_POOL, layer).upload(helper.pack_pages(kc, ks, vc, vs))
        nbytes = self.physical_pages * gpu.page_bytes
        for layer in range(distinct, d["layers"]):
            device_copy(gpu.backend, gpu.buffer(verify.KV_POOL, layer % distinct), gpu.buffer(verify.KV_POOL, layer), nbytes)
        # layers of one drawn context share its arrays: the oracle's stores of a block land in the slots the GPU's do
        self.context = [drawn[l % distinct] for l in range(d["layers"])]

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

    # One layer in five stages, each from bf16 rows (uint16 bits), so that a test can feed every stage the GPU's own
    # rows of the stage before (the buffers the driver leaves them in) and no rounding difference compounds.
    def oracle_qkv(self, hidden, li):
        d, w = self.dims, self.layers[li]
        D = d["head_dim"]
        n = orc.rms_norm(hidden, w["input_norm"])
        qkv = np.concatenate([self._project(orc.FMT_Q4K, w[name], n, w_n) for name, w_n in
                              (("q", d["q_heads"] * D), ("k", d["kv_heads"] * D), ("v", d["kv_heads"] * D))], axis=1)
        return orc.f32_to_bf16(qkv.astype(np.float32))

    def oracle_attention(self, qkv, li, committed, table_first=0, want64=False):
        """Head norms, RoPE, the INT8 store of the block's keys and values into the layer's context, attention."""
        d, w = self.dims, self.layers[li]
        rows, D = qkv.shape[0], d["head_dim"]
        cosv, sinv, pairs = self._rope(rows, committed)
        anc = np.array([(2 << r) - 1 for r in range(rows)], dtype=np.uint32)
        table = self.table[table_first:].astype(np.uint32)
        q, kf, vf = orc.attention_prepare(d["q_heads"], d["kv_heads"], D, qkv, w["q_norm"], w["k_norm"], cosv, sinv, pairs)
        kc, ks, vc, vs = self.context[li]
        kcod, kscl = orc.kv_quantize(kf)
        vcod, vscl = orc.kv_quantize(vf)
        for r in range(rows):
            t = committed + r
            p, s = table[t // ops.PAGE_TOKENS], t % ops.PAGE_TOKENS
            kc[p, :, s], ks[p, :, s], vc[p, :, s], vs[p, :, s] = kcod[r], kscl[r], vcod[r], vscl[r]
        attn, attn64 = orc.attention(q, kc, ks, vc, vs, table, anc, committed, want64=want64)
        attn = attn.reshape(rows, d["q_heads"] * D)
        return (attn, attn64.reshape(rows, d["q_heads"] * D)) if want64 else attn

    def oracle_output(self, attn, hidden, li):
        o = self._project(orc.FMT_Q4K, self.layers[li]["o"], attn, self.dims["hidden"])
        return orc.f32_to_bf16((o + orc.bf16_to_f32(hidden)).astype(np.float32))

    def oracle_ffn_rows(self, hidden1, li, deferred=False):
        """deferred: the norm as the step's residual projections leave it to the projection after them -- the operand is
        bf16(h w) (an exact product, rounded once) and the row's inverse RMS multiplies the projection's sums -- in place of
        the norm pass's bf16((h inv) w): the same arithmetic with the operand's one rounding taken before the scale."""
        d, w = self.dims, self.layers[li]
        if deferred:
            h = orc.bf16_to_f32(hidden1).astype(np.float64)
            n = orc.f32_to_bf16((h * orc.bf16_to_f32(w["post_norm"]).astype(np.float64)).astype(np.float32))
            inv = 1.0 / np.sqrt((h * h).mean(axis=1, keepdims=True) + 1e-6)
        else:
            n, inv = orc.rms_norm(hidden1, w["post_norm"]), 1.0
        gate = (self._project(orc.FMT_Q4K, w["gate"], n, d["ffn"]) * inv).astype(np.float32)
        up = (self._project(orc.FMT_Q4K, w["up"], n, d["ffn"]) * inv).astype(np.float32)
        g16, u16 = orc.bf16_to_f32(orc.f32_to_bf16(gate)), orc.bf16_to_f32(orc.f32_to_bf16(up))
        return orc.f32_to_bf16((u16 * (g16 / (1 + np.exp2(np.float32(-1.4426950408889634) * g16)))).astype(np.float32))

    def oracle_down(self, inter, hidden1, li):
        down = self._project(self.down_format, self.layers[li]["down"], inter, self.dims["hidden"])
        return orc.f32_to_bf16((down + orc.bf16_to_f32(hidden1)).astype(np.float32))

    def oracle_layer(self, hidden, li, committed, table_first=0):
        """One layer from bf16 hidden rows (uint16 bits) of a lane whose pages start at entry `table_first` of the page
        table: stores the block's K/V into the layer's context."""
        attn = self.oracle_attention(self.oracle_qkv(hidden, li), li, committed, table_first)
        hidden1 = self.oracle_output(attn, hidden, li)
        return self.oracle_down(self.oracle_ffn_rows(hidden1, li), hidden1, li)

    def oracle_head(self, hidden):
        n = orc.rms_norm(hidden, self.final_norm)
        return self._project(orc.FMT_Q6K, self.head, n, self.dims["vocabulary"])

    def oracle_step(self, tokens, committed, table_first=0):
        rows = len(tokens)
        hidden = self.oracle_embedding(tokens)
        for li in range(self.dims["layers"]):
            hidden = self.oracle_layer(hidden, li, committed, table_first)
        logits = self.oracle_head(hidden)
        selected = np.array([orc.argmax(logits[r].astype(np.float32)) for r in range(rows)], dtype=np.uint32)
        kept, accepted, mask = orc.accept_tree(ops.chain_tree_rows([rows]), tokens, selected)
        return dict(logits=logits, selected=selected, kept=kept, accepted=accepted, retained_rows=mask)
