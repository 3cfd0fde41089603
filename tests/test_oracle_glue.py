"""Independent pins of the oracle's glue functions: RMS norm, RoPE tables, the q/k prepare of a
block's rows, SiLU / SwiGLU, the sigmoid router and the shared expert's gate. Each is compared with a
float64 statement written from the mathematics, not from the oracle's code, and each test carries a
case that a plausible mistake (no epsilon, the neighbouring pair, a flipped sign, a missing
renormalization) fails."""
import numpy as np

from tests import oracle as orc


def _bf16_step(values):
    """One bf16 step at each value's magnitude (8 significant bits)."""
    return np.maximum(np.abs(values), 2.0 ** -126) * 2.0 ** -7


def _bits(values):
    return orc.f32_to_bf16(np.asarray(values, np.float32))


# ------------------------------------------------------------------ RMS norm (normalization.metal:59-99)
def test_rms_norm_equals_the_float64_statement_within_a_bf16_step():
    rng = np.random.default_rng(11)
    for width in (64, 1000, 5120):
        x = _bits(rng.standard_normal((7, width)) * rng.uniform(0.01, 30, (7, 1)))
        w = _bits(1 + 0.2 * rng.standard_normal(width))
        got = orc.bf16_to_f32(orc.rms_norm(x, w)).astype(np.float64)
        xf, wf = orc.bf16_to_f32(x).astype(np.float64), orc.bf16_to_f32(w).astype(np.float64)
        want = xf / np.sqrt((xf * xf).mean(axis=1, keepdims=True) + 1e-6) * wf
        assert np.all(np.abs(got - want) <= _bf16_step(want)), width


def test_rms_norm_epsilon_and_mean_are_those_of_the_rule():
    # A row of tiny values: sum x^2 / W is far below 1e-6, so out = x / sqrt(1e-6) * w = 1000 x w. Without the
    # epsilon the row would come out at unit RMS (about 1); with the sum in place of the mean, off by sqrt(W).
    width = 256
    x = _bits(np.full((1, width), 2.0 ** -20))
    w = _bits(np.ones(width))
    got = orc.bf16_to_f32(orc.rms_norm(x, w))
    want = 2.0 ** -20 / np.sqrt(2.0 ** -40 + 1e-6)
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * want)
    assert abs(want - 1000 * 2.0 ** -20) < 1e-6 * want * 1000
    # A constant row of ones with unit weights is itself (the mean, not the sum, sits under the root).
    ones = _bits(np.ones((2, 384)))
    assert np.array_equal(orc.rms_norm(ones, _bits(np.ones(384))), ones)
    # The weight multiplies the normalized value: twice the weight, twice the row (exact in bf16).
    x = _bits(np.random.default_rng(0).standard_normal((3, 512)))
    one = orc.bf16_to_f32(orc.rms_norm(x, _bits(np.ones(512))))
    two = orc.bf16_to_f32(orc.rms_norm(x, _bits(np.full(512, 2.0))))
    assert np.array_equal(two, 2 * one)
    # zero rows stay zero (the epsilon keeps the inverse finite)
    assert not orc.rms_norm(np.zeros((1, 128), np.uint16), _bits(np.ones(128))).any()


# ------------------------------------------------------------------ RoPE tables (rope.metal:51-80)
def test_rope_tables_are_the_cosine_and_sine_of_position_times_frequency():
    pairs = 64
    invfreq = np.array([1e6 ** (-i / pairs) for i in range(pairs)], np.float32)
    depth = np.array([0, 1, 2, 2, 3, 1, 15], np.uint32)
    for anchor in (0, 1, 511, 32768, 131071):
        cosv, sinv = orc.rope_tables(anchor, depth, invfreq)
        angle = ((anchor + depth).astype(np.float32)[:, None] * invfreq[None, :]).astype(np.float32).astype(np.float64)
        # the angle is an fp32 product; a float cos/sin of it is within a few ulps of 1 of the exact one
        assert np.abs(cosv - np.cos(angle)).max() <= 4e-7 and np.abs(sinv - np.sin(angle)).max() <= 4e-7, anchor
        assert np.abs(cosv.astype(np.float64) ** 2 + sinv.astype(np.float64) ** 2 - 1).max() <= 1e-6
    cosv, sinv = orc.rope_tables(0, np.zeros(3, np.uint32), invfreq)
    assert np.all(cosv == 1) and np.all(sinv == 0)                       # position 0: the identity rotation
    # rows of equal depth share a position (tree siblings), rows of different depth do not
    cosv, sinv = orc.rope_tables(100, depth, invfreq)
    assert np.array_equal(cosv[2], cosv[3]) and np.array_equal(sinv[1], sinv[5]) and not np.array_equal(sinv[1], sinv[2])


# ------------------------------------------------------------------ q/k prepare (attention_qkv_prepare.h:28-91)
def _prepare_case(rng, q_heads, kv_heads, D, rows, pairs, scale=1.0):
    width = (q_heads + 2 * kv_heads) * D
    qkv = _bits(rng.standard_normal((rows, width)) * scale)
    qw, kw = _bits(1 + 0.3 * rng.standard_normal(D)), _bits(1 + 0.3 * rng.standard_normal(D))
    angle = rng.uniform(-np.pi, np.pi, (rows, pairs))
    cosv, sinv = np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)
    return qkv, qw, kw, cosv, sinv


def _prepare_float64(qkv, qw, kw, cosv, sinv, q_heads, kv_heads, D, pairs):
    """The rule in float64 with a complex rotation: dimension i < P of a head pairs with dimension i + P."""
    rows = qkv.shape[0]
    x = orc.bf16_to_f32(qkv).astype(np.float64)
    heads = x[:, :(q_heads + kv_heads) * D].reshape(rows, q_heads + kv_heads, D)
    w = np.concatenate([np.tile(orc.bf16_to_f32(qw).astype(np.float64), (q_heads, 1)),
                        np.tile(orc.bf16_to_f32(kw).astype(np.float64), (kv_heads, 1))])
    n = heads / np.sqrt((heads * heads).mean(axis=2, keepdims=True) + 1e-6) * w[None]
    z = (n[..., :pairs] + 1j * n[..., pairs:2 * pairs]) * (cosv.astype(np.float64) + 1j * sinv.astype(np.float64))[:, None, :]
    out = n.copy()
    out[..., :pairs], out[..., pairs:2 * pairs] = z.real, z.imag
    v = x[:, (q_heads + kv_heads) * D:].reshape(rows, kv_heads, D)
    return out[:, :q_heads], out[:, q_heads:], v, n


def test_prepare_is_norm_then_rotation_of_pairs_half_a_head_apart():
    rng = np.random.default_rng(21)
    for q_heads, kv_heads, D, pairs in ((4, 2, 64, 32), (8, 1, 128, 64), (2, 2, 128, 32)):   # the last rotates part of a head
        qkv, qw, kw, cosv, sinv = _prepare_case(rng, q_heads, kv_heads, D, 5, pairs)
        q, k, v = orc.attention_prepare(q_heads, kv_heads, D, qkv, qw, kw, cosv, sinv, pairs)
        wq, wk, wv, n = _prepare_float64(qkv, qw, kw, cosv, sinv, q_heads, kv_heads, D, pairs)
        # two bf16 roundings (the normalized value, then the rotated one): each within a step of the magnitudes involved
        bound = _bf16_step(wq) + 2 * _bf16_step(np.abs(n[:, :q_heads]).max(axis=2, keepdims=True) * np.ones_like(wq))
        assert np.all(np.abs(orc.bf16_to_f32(q) - wq) <= bound)
        bound = _bf16_step(wk) + 2 * _bf16_step(np.abs(n[:, q_heads:]).max(axis=2, keepdims=True) * np.ones_like(wk))
        assert np.all(np.abs(k - wk) <= bound)
        assert np.array_equal(v, wv.astype(np.float32))                                 # values pass through unchanged
        cos = (orc.bf16_to_f32(q).astype(np.float64) * wq).sum() / np.sqrt((orc.bf16_to_f32(q).astype(np.float64) ** 2).sum() * (wq ** 2).sum())
        assert cos >= 0.99999


def test_prepare_pairing_and_sign_fail_a_wrong_rotation():
    # One head whose normalized value is a one-hot at dimension 3, rotated by +90 degrees in pair 3: the value
    # must move to dimension 3 + P with a plus sign (b' = b cos + a sin). A rotation of neighbours (2i, 2i + 1)
    # would move it to dimension 2 or 4, and a flipped sign would give -1.
    D, pairs = 64, 32
    row = np.zeros((1, 3 * D))
    row[0, 3] = 1.0            # query head
    row[0, D + 3] = 1.0        # key head
    qkv = _bits(row)
    cosv, sinv = np.ones((1, pairs), np.float32), np.zeros((1, pairs), np.float32)
    cosv[0, 3], sinv[0, 3] = 0.0, 1.0
    q, k, _ = orc.attention_prepare(1, 1, D, qkv, None, None, cosv, sinv, pairs)      # no norm weights: rows as they are
    assert orc.bf16_to_f32(q)[0, 0, 3 + pairs] == 1.0 and np.count_nonzero(q) == 1
    assert k[0, 0, 3 + pairs] == 1.0 and np.count_nonzero(k) == 1
    # the other way round: a one-hot in the second half moves to the first half with a minus sign
    row[:] = 0
    row[0, 3 + pairs] = 1.0
    q, _, _ = orc.attention_prepare(1, 1, D, _bits(row), None, None, cosv, sinv, pairs)
    assert orc.bf16_to_f32(q)[0, 0, 3] == -1.0 and np.count_nonzero(q) == 1


def test_prepare_zero_angle_is_the_norm_and_rotation_keeps_pair_lengths():
    rng = np.random.default_rng(22)
    q_heads, kv_heads, D, pairs, rows = 4, 2, 128, 64, 6
    qkv, qw, kw, cosv, sinv = _prepare_case(rng, q_heads, kv_heads, D, rows, pairs)
    ident = np.ones_like(cosv), np.zeros_like(sinv)
    q0, k0, _ = orc.attention_prepare(q_heads, kv_heads, D, qkv, qw, kw, *ident, pairs)
    # zero angle: exactly the per-head RMS norm, one rounding, which the float64 rule gives within a step
    _, _, _, n = _prepare_float64(qkv, qw, kw, *ident, q_heads, kv_heads, D, pairs)
    assert np.all(np.abs(orc.bf16_to_f32(q0) - n[:, :q_heads]) <= _bf16_step(n[:, :q_heads]))
    # the per-head normalization divides by the head's own RMS: with unit weights every head leaves at unit RMS
    ones = _bits(np.ones(D))
    q1, k1, _ = orc.attention_prepare(q_heads, kv_heads, D, qkv, ones, ones, *ident, pairs)
    assert np.abs(np.sqrt((orc.bf16_to_f32(q1).astype(np.float64) ** 2).mean(axis=2)) - 1).max() <= 4e-3
    assert np.abs(np.sqrt((k1.astype(np.float64) ** 2).mean(axis=2)) - 1).max() <= 4e-3
    # a rotation keeps each pair's length (to the bf16 roundings)
    q, k, _ = orc.attention_prepare(q_heads, kv_heads, D, qkv, qw, kw, cosv, sinv, pairs)
    a0, a = orc.bf16_to_f32(q0).astype(np.float64), orc.bf16_to_f32(q).astype(np.float64)
    len0 = np.hypot(a0[..., :pairs], a0[..., pairs:])
    len1 = np.hypot(a[..., :pairs], a[..., pairs:])
    assert np.all(np.abs(len0 - len1) <= 3 * _bf16_step(len0) + 1e-30)
    # the epsilon: a head of tiny values comes out at x * 1000 * w, not at unit RMS
    tiny = _bits(np.full((1, 3 * D), 2.0 ** -20))
    qt, _, _ = orc.attention_prepare(1, 1, D, tiny, ones, ones, np.ones((1, pairs), np.float32), np.zeros((1, pairs), np.float32), pairs)
    want = 2.0 ** -20 / np.sqrt(2.0 ** -40 + 1e-6)
    assert np.all(np.abs(orc.bf16_to_f32(qt) - want) <= 2.0 ** -8 * want)


# ------------------------------------------------------------------ SiLU / SwiGLU (activation.h:8-16, gguf_linear.metal:34-71)
def test_silu_and_swiglu_against_float64():
    rng = np.random.default_rng(31)
    x = np.concatenate([rng.standard_normal(2000) * 4, [0.0, -0.0, 1.0, -1.0, 20.0, -20.0, 88.0, -88.0, 1e-8]]).astype(np.float32)
    want = x.astype(np.float64) / (1 + np.exp(-x.astype(np.float64)))
    got = orc.silu(x)
    # exp2(-x log2 e) in fp32: the product's rounding moves the exponent by |x| 2^-24, so the relative error grows with |x|
    assert np.all(np.abs(got - want) <= 2e-7 * (2 + 1.5 * np.abs(x)) * np.abs(want) + 1e-44)
    assert orc.silu(np.float32(0))[()] == 0 and orc.silu(np.float32(-88))[()] <= 0      # x sigmoid(x), not x sigmoid(-x)
    assert abs(float(orc.silu(np.float32(1))[()]) - 0.7310585786300049) < 1e-7
    assert abs(float(orc.silu(np.float32(-1))[()]) + 0.2689414213699951) < 1e-7
    gate = (rng.standard_normal(3000) * 3).astype(np.float32)
    up = (rng.standard_normal(3000) * 3).astype(np.float32)
    got = orc.bf16_to_f32(orc.swiglu(gate, up)).astype(np.float64)
    g16 = orc.bf16_to_f32(orc.f32_to_bf16(gate)).astype(np.float64)                    # both operands round to bf16 first
    u16 = orc.bf16_to_f32(orc.f32_to_bf16(up)).astype(np.float64)
    want = u16 * g16 / (1 + np.exp(-g16))
    assert np.all(np.abs(got - want) <= _bf16_step(want))
    # the gate is the activated operand: up = 1 gives silu(gate), gate = large gives up * gate
    assert orc.bf16_to_f32(orc.swiglu(np.float32([-30.0]), np.float32([1.0])))[0] > -1e-10
    assert orc.bf16_to_f32(orc.swiglu(np.float32([1.0]), np.float32([-30.0])))[0] == orc.bf16_to_f32(_bits([-30 * 0.7310585786300049]))[0]


# ------------------------------------------------------------------ sigmoid router, shared expert (moe.metal:23-113)
def test_sigmoid_router_weighs_by_normalized_sigmoids_of_the_selected_scores():
    rng = np.random.default_rng(41)
    rows, experts, k = 30, 64, 6
    scores = (rng.standard_normal((rows, experts)) * 2).astype(np.float32)
    scores[2, :] = 0.5                                                    # all equal: ids 0..k-1, weights 1/k each
    scores[3, :] = -40.0
    scores[3, 9] = 3.0                                                    # one expert far above the rest
    selected, weights = orc.moe_route(scores, k, sigmoid_router=True)
    order = np.lexsort((np.arange(experts)[None, :].repeat(rows, 0), -scores.astype(np.float64)), axis=1)[:, :k]
    assert np.array_equal(selected, order.astype(np.uint32))              # the selection is the softmax router's
    picked = np.take_along_axis(scores.astype(np.float64), order, axis=1)
    sig = 1 / (1 + np.exp(-picked))
    want = sig / sig.sum(axis=1, keepdims=True)
    assert np.abs(weights - want).max() <= 3e-7
    assert np.abs(weights.sum(axis=1) - 1).max() <= 1e-6                  # normalized (a bare sigmoid would sum above 1)
    assert np.array_equal(selected[2], np.arange(k)) and np.abs(weights[2] - 1 / k).max() <= 1e-7
    assert selected[3, 0] == 9 and weights[3, 0] > 0.999999
    # it is not the softmax: for scores 0 and ln 3 the softmax gives 1/4, 3/4, the sigmoids 0.5 and 0.75 -> 0.4, 0.6
    two = np.full((1, 4), -80.0, np.float32)
    two[0, 1], two[0, 2] = 0.0, np.log(3.0)
    s, w = orc.moe_route(two, 2, sigmoid_router=True)
    assert list(s[0]) == [2, 1] and np.abs(w[0] - [0.6, 0.4]).max() <= 1e-6
    s, w = orc.moe_route(two, 2)
    assert list(s[0]) == [2, 1] and np.abs(w[0] - [0.75, 0.25]).max() <= 1e-6


def test_shared_expert_gate_is_the_sigmoid_of_the_rows_product_with_the_gate():
    rng = np.random.default_rng(42)
    rows, hidden = 9, 2048
    x = _bits(rng.standard_normal((rows, hidden)))
    gate = (rng.standard_normal(hidden) * 0.05).astype(np.float32)
    got = orc.moe_shared_weights(x, gate)
    dot = (orc.bf16_to_f32(x).astype(np.float64) * gate.astype(np.float64)).sum(axis=1)
    want = 1 / (1 + np.exp(-dot))
    absdot = (np.abs(orc.bf16_to_f32(x).astype(np.float64)) * np.abs(gate.astype(np.float64))).sum(axis=1)
    assert np.all(np.abs(got - want) <= 0.25 * 2.0 ** -18 * absdot + 2e-7)   # an fp32 sum of 2048 terms under a slope of 1/4
    # closed forms: a zero gate weighs 1/2; a one-hot gate picks one input; the sign is sigmoid(+dot)
    assert np.all(orc.moe_shared_weights(x, np.zeros(hidden, np.float32)) == 0.5)
    onehot = np.zeros(hidden, np.float32)
    onehot[777] = 2.0
    want = 1 / (1 + np.exp(-2.0 * orc.bf16_to_f32(x[:, 777]).astype(np.float64)))
    assert np.abs(orc.moe_shared_weights(x, onehot) - want).max() <= 2e-7
    big = _bits(np.full((1, hidden), 1.0))
    assert orc.moe_shared_weights(big, np.full(hidden, 0.01, np.float32))[0] > 0.999999
    # through the router: shared slices follow the routed experts, each at the row's gate weight
    scores = rng.standard_normal((rows, 16)).astype(np.float32)
    selected, weights = orc.moe_route(scores, 4, shared=2, x_bits=x, shared_gate=gate)
    assert np.array_equal(selected[:, 4:], np.tile([16, 17], (rows, 1)).astype(np.uint32))
    assert np.array_equal(weights[:, 4], got) and np.array_equal(weights[:, 5], got)
    _, ungated = orc.moe_route(scores, 4, shared=1)
    assert np.all(ungated[:, 4] == 1.0)


# ------------------------------------------------------------------ embedding gather (embedding.metal:10-18)
def test_embedding_rows_are_the_golden_dequantization_rounded_to_bf16():
    vocab, hidden = 256, 1024
    for _, fmt in orc.ALL_FORMATS:
        table = orc.fixture(fmt, vocab, hidden, 7 + fmt)                 # the fixture the reference's goldens hash
        values = orc.dequant_rows(fmt, table, vocab, hidden)             # pinned by those goldens
        tokens = np.array([0, 255, 17, 17, 256, 0xFFFFFFFF, 3], np.uint32)
        got = orc.embed(fmt, table, vocab, hidden, tokens)
        for r, t in enumerate(tokens):
            want = orc.f32_to_bf16(values[t]) if t < vocab else np.zeros(hidden, np.uint16)   # a token past the table reads zeros
            assert np.array_equal(got[r], want), (fmt, r)


# ------------------------------------------------------------------ float projection (gguf_float.metal:1-8)
def test_float_projection_differs_from_the_fp64_product_by_fp32_accumulation_only():
    rng = np.random.default_rng(17)
    for rows, n, k in ((5, 24, 2048), (1, 7, 8), (33, 130, 200)):
        x = _bits(rng.standard_normal((rows, k)) * 3)
        w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
        got = orc.float_projection(x, w).astype(np.float64)
        xf = orc.bf16_to_f32(x).astype(np.float64)
        want = xf @ w.astype(np.float64).T
        bound = 2.0 ** -24 * (k / 4 + 3) * (np.abs(xf) @ np.abs(w.astype(np.float64)).T)   # a chain of k / 4 sums, then two more
        assert np.all(np.abs(got - want) <= bound + 1e-30), (rows, n, k)
        # BF16 weights give the bits of the F32 tensor of their values
        wb = _bits(w)
        assert orc.float_projection(x, wb).tobytes() == orc.float_projection(x, orc.bf16_to_f32(wb)).tobytes()


def test_float_projection_adds_in_four_chains_by_input_modulo_four():
    """Sums only this order gives: 2^24 in chain 0 swallows the ones of chain 0 and not those of the other chains; a
    sequential sum, or pairs of neighbours, would give other values."""
    k = 16
    x = _bits(np.ones((1, k)))
    w = np.ones((1, k), np.float32)
    w[0, 0] = 2.0 ** 24
    # chain 0: 2^24 + 1 + 1 + 1 rounds to 2^24 each time; chains 1..3: 4 each; (2^24 + 4) + 8 = 2^24 + 12
    assert orc.float_projection(x, w)[0, 0] == np.float32(2.0 ** 24 + 12)
    w[0, 0], w[0, 13] = 1.0, 2.0 ** 24
    # chain 1 now ends with 2^24: 3 + 2^24 is exact; (4 + (2^24 + 3)) -> 2^24 + 8 (ties to even), then + 8
    assert orc.float_projection(x, w)[0, 0] == np.float32(np.float32(np.float32(4) + np.float32(2.0 ** 24 + 3)) + np.float32(8))
    # fused multiply-adds: a product's low bits reach the sum
    x2 = _bits(np.array([[1 + 2.0 ** -7, 1.0, 0, 0, 0, 0, 0, 0]]))
    w2 = np.array([[1 + 2.0 ** -20, -1.0, 0, 0, 0, 0, 0, 0]], np.float32)
    exact = (1 + 2.0 ** -7) * (1 + 2.0 ** -20) - 1.0
    assert orc.float_projection(x2, w2)[0, 0] == np.float32(np.float32((1 + 2.0 ** -7) * (1 + 2.0 ** -20)) + np.float32(-1.0))
    assert abs(float(orc.float_projection(x2, w2)[0, 0]) - exact) <= 2.0 ** -24
