"""A random-init DFlash draft for the parity tests: its weights (N(0, 0.02) rows quantized to Q4_K by the oracle's
quantizer, the head to Q6_K), the GPU model built from them, and the oracle's own evaluation of the draft's forward pass
and of its context writers, composed of the oracle's operators. Test infrastructure only."""
import numpy as np

from splash_amd import ops, verify
from tests import oracle as orc

ROWS, QH, KVH, D, WINDOW = 8, 32, 8, 128, 2048
RING = ops.DRAFT_RING_BYTES // 2    # bf16 values of a ring


def bits(values):
    return orc.f32_to_bf16(np.asarray(values, np.float32))


def rope_tables(positions, theta=1e7):
    """cos, sin fp32 [len(positions)][64] of position x theta^(-i / 64)."""
    inv = np.array([theta ** (-i / 64) for i in range(64)]).astype(np.float32)
    angle = (np.asarray(positions, np.float32)[:, None] * inv[None, :]).astype(np.float32).astype(np.float64)
    return np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)


class DraftModel:
    def __init__(self, seed, hidden, vocabulary, intermediate, layers, target_layers=2):
        self.hidden, self.vocabulary, self.intermediate, self.layer_count, self.target_layers = hidden, vocabulary, intermediate, layers, target_layers
        rng = np.random.default_rng(seed)
        self.rng = rng
        quant = lambda n, k, fmt=orc.FMT_Q4K, scale=0.02: orc.quantize_rows(fmt, (rng.standard_normal((n, k)) * scale).astype(np.float32))
        norm = lambda n: bits(1 + 0.1 * rng.standard_normal(n))
        # a convolution's base weights: the row itself near one, the row before it small, in both stages
        conv = lambda: bits(np.stack([1 + 0.1 * rng.standard_normal(hidden), 0.2 * rng.standard_normal(hidden),
                                      1 + 0.1 * rng.standard_normal(hidden), 0.2 * rng.standard_normal(hidden)]))
        self.layers = [dict(input_norm=norm(hidden), attention_convolution=conv(), attention_dynamic=quant(hidden // 4, hidden),
                            qkv=quant(6144, hidden), query_norm=norm(D), key_norm=norm(D), output=quant(hidden, 4096),
                            post_attention_norm=norm(hidden), mlp_convolution=conv(), mlp_dynamic=quant(hidden // 4, hidden),
                            gate=quant(intermediate, hidden), up=quant(intermediate, hidden), down=quant(hidden, intermediate))
                       for _ in range(layers)]
        self.context_projection = quant(hidden, target_layers * hidden)
        self.hidden_norm, self.final_norm = norm(hidden), norm(hidden)
        self.selector = quant(256, hidden)
        self.mask_embedding = bits(rng.standard_normal(hidden))
        self.head = quant(vocabulary, hidden, orc.FMT_Q6K)

    # ------------------------------------------------------------------ GPU side
    def build_gpu(self, backend, max_lanes, context_rows=0, head_ranges=None):
        """head_ranges: [(first, count)] rows of the head the draft's logits cover (a vocabulary subset); all of them by default."""
        gpu = verify.DFlashDraft(backend, self.layer_count, self.hidden, self.vocabulary, self.intermediate, self.target_layers, max_lanes,
                                 context_rows)
        P = lambda native, n, k, fmt=orc.FMT_Q4K, f32=False: ops.Projection.from_native(backend, [(fmt, n, native)], k, float32=f32)
        H, F = self.hidden, self.intermediate
        for index, w in enumerate(self.layers):
            gpu.set_layer(index, attention_dynamic=P(w["attention_dynamic"], H // 4, H), qkv=P(w["qkv"], 6144, H), output=P(w["output"], H, 4096),
                          mlp_dynamic=P(w["mlp_dynamic"], H // 4, H), gate=P(w["gate"], F, H), up=P(w["up"], F, H), down=P(w["down"], H, F),
                          **{name: backend.from_array(w[name]) for name in ("input_norm", "attention_convolution", "query_norm", "key_norm",
                                                                             "post_attention_norm", "mlp_convolution")})
        head = P(self.head, self.vocabulary, H, orc.FMT_Q6K, True)
        gpu.set_model(P(self.context_projection, H, self.target_layers * H), backend.from_array(self.hidden_norm),
                      backend.from_array(self.final_norm), P(self.selector, 256, H), backend.from_array(self.mask_embedding),
                      head.rows(head_ranges) if head_ranges else head)
        return gpu

    # ------------------------------------------------------------------ oracle side
    @staticmethod
    def _project(native, x_bits, n, fmt=orc.FMT_Q4K):
        return orc.gemm(fmt, native, x_bits, n, want=("exact",))["exact"]

    def _rows(self, native, x_bits, n):
        return bits(self._project(native, x_bits, n))

    def oracle_layer(self, hidden, index, rings, cache_lengths, cosines, sines):
        """hidden bf16 bits [lanes * 8][hidden]; rings [lanes][layers][2][RING] bf16 bits; cosines / sines [lanes][16][64]."""
        w = self.layers[index]
        lanes = len(cache_lengths)
        n = orc.rms_norm(hidden, w["input_norm"])
        dynamic = self._rows(w["attention_dynamic"], n, self.hidden // 4)
        convolved = orc.draft_conv(n, dynamic, w["attention_convolution"], None, False)
        qkv = self._rows(w["qkv"], convolved, 6144)
        q, k, v = orc.draft_prepare(qkv, w["query_norm"], w["key_norm"], cosines, sines)
        attention = np.empty((lanes, ROWS, QH, D), np.float64)
        for lane in range(lanes):
            keys, values = rings[lane][index][0].reshape(KVH, WINDOW, D), rings[lane][index][1].reshape(KVH, D, WINDOW)
            for head in range(KVH):
                rows = orc.draft_attention(q[lane, 4 * head:4 * head + 4].reshape(32, D), keys[head], values[head], k[lane, head], v[lane, head],
                                           cache_lengths[lane])
                attention[lane, :, 4 * head:4 * head + 4] = rows.reshape(4, ROWS, D).transpose(1, 0, 2)
        attention = bits(attention.reshape(lanes * ROWS, 4096))
        projected = self._rows(w["output"], attention, self.hidden)
        residual = orc.draft_conv(projected, dynamic, w["attention_convolution"], hidden, True)
        n = orc.rms_norm(residual, w["post_attention_norm"])
        dynamic = self._rows(w["mlp_dynamic"], n, self.hidden // 4)
        convolved = orc.draft_conv(n, dynamic, w["mlp_convolution"], None, False)
        gate, up = self._project(w["gate"], convolved, self.intermediate), self._project(w["up"], convolved, self.intermediate)
        g16, u16 = orc.bf16_to_f32(bits(gate)), orc.bf16_to_f32(bits(up))
        intermediate = bits(u16 * (g16 / (1 + np.exp2(np.float32(-1.4426950408889634) * g16))))
        projected = self._rows(w["down"], intermediate, self.hidden)
        return orc.draft_conv(projected, dynamic, w["mlp_convolution"], residual, True)

    def oracle_decode(self, hidden, rings, cache_lengths, cosines, sines):
        """Returns the hidden rows after every layer, the final norm's rows, the logits (fp64) and the selector's rows."""
        after = []
        for index in range(self.layer_count):
            hidden = self.oracle_layer(hidden, index, rings, cache_lengths, cosines, sines)
            after.append(hidden)
        final = orc.rms_norm(hidden, self.final_norm)
        return after, final, self._project(self.head, final, self.vocabulary, orc.FMT_Q6K), self._rows(self.selector, final, 256)

    def oracle_context_hidden(self, captured):
        return orc.rms_norm(self._rows(self.context_projection, captured, self.hidden), self.hidden_norm)

    def oracle_context_kv(self, context_hidden, index):
        """bf16 bits [rows][2048]: the key and value rows of layer `index`'s q|k|v projection."""
        qkv = self.layers[index]["qkv"]
        row_bytes = qkv.size // 6144
        return self._rows(qkv.reshape(6144, row_bytes)[4096:].ravel(), context_hidden, 2048)
