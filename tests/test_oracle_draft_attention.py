"""Independent pins of the oracle's draft attention block (oracle/draft_attention.cpp): each function against a float64
statement in numpy written from the operator's description (the reference's runtime/ops/DraftAttention.hpp and
metal/abi/DraftAttention.h), with cases a plausible mistake fails: the other tap or stage of a convolution, the
neighbouring RoPE pair or a flipped sign, a slot off by one, a window one position too long, the causal mask the
current rows do not have."""
import numpy as np
import pytest

from tests import oracle as orc

ROWS, QH, KVH, D, WINDOW = 8, 32, 8, 128, 2048


def _bits(values):
    return orc.f32_to_bf16(np.asarray(values, np.float32))


def _f64(bits):
    return orc.bf16_to_f32(bits).astype(np.float64)


def _bf16_step(values):
    return np.maximum(np.abs(values), 2.0 ** -126) * 2.0 ** -7


# ------------------------------------------------------------------ the dynamic convolution (draft.metal:7-44)
@pytest.mark.parametrize("finish", [False, True])
def test_convolution_on_dyadic_inputs_is_the_float64_statement(finish):
    """Values k / 8 with small k, as the reference's test draws them (draft_attention_metal_test.mm:325-329, :374-398):
    every product and sum is exact in fp32, so the rounded fp64 statement is the result bit for bit."""
    rng = np.random.default_rng(5)
    hidden, lanes = 256, 2
    dyadic = lambda shape: _bits(rng.integers(-12, 13, shape) / 8.0)
    x, residual = dyadic((lanes * ROWS, hidden)), dyadic((lanes * ROWS, hidden))
    dynamic, base = dyadic((lanes * ROWS, 4 * hidden // 16)), dyadic((4, hidden))
    got = orc.draft_conv(x, dynamic, base, residual, finish)
    xf, rf, bf = _f64(x).reshape(lanes, ROWS, hidden), _f64(residual).reshape(lanes, ROWS, hidden), _f64(base)
    dyn = _f64(dynamic).reshape(lanes, ROWS, 2, 2, hidden // 16).repeat(16, axis=-1)   # [stage][tap][channel]
    stage = 1 if finish else 0
    want = xf * (bf[2 * stage] + dyn[:, :, stage, 0])
    want[:, 1:] += xf[:, :-1] * (bf[2 * stage + 1] + dyn[:, 1:, stage, 1])   # the row before, of the same lane; row 0 has none
    if finish:
        want += rf
    assert np.array_equal(got, _bits(want.reshape(lanes * ROWS, hidden)))
    # the other stage's weights give another result: the stages are not interchangeable
    assert not np.array_equal(got, orc.draft_conv(x, dynamic, base, residual, not finish))


def test_convolution_on_random_inputs_stays_within_a_bf16_step():
    rng = np.random.default_rng(6)
    hidden = 512
    x, residual = _bits(rng.standard_normal((ROWS, hidden))), _bits(rng.standard_normal((ROWS, hidden)))
    dynamic, base = _bits(rng.standard_normal((ROWS, 4 * hidden // 16)) * 0.3), _bits(rng.standard_normal((4, hidden)))
    got = _f64(orc.draft_conv(x, dynamic, base, residual, True))
    xf, bf = _f64(x), _f64(base)
    dyn = _f64(dynamic).reshape(ROWS, 2, 2, hidden // 16).repeat(16, axis=-1)
    want = xf * (bf[2] + dyn[:, 1, 0]) + _f64(residual)
    want[1:] += xf[:-1] * (bf[3] + dyn[1:, 1, 1])
    assert np.all(np.abs(got - want) <= _bf16_step(want) + 1e-6)


# ------------------------------------------------------------------ preparation (draft.metal:46-105)
def _prepared_head(x_bits, w_bits, cosines, sines):
    x, w = _f64(x_bits), _f64(w_bits)
    n = _f64(_bits(x / np.sqrt((x * x).mean() + 1e-6) * w))    # rounded to bf16 before the rotation
    return np.concatenate([n[:64] * cosines - n[64:] * sines, n[64:] * cosines + n[:64] * sines])


def test_preparation_normalizes_rotates_and_groups():
    rng = np.random.default_rng(7)
    lanes = 2
    qkv = _bits(rng.standard_normal((lanes * ROWS, 6144)) * rng.uniform(0.1, 4, (lanes * ROWS, 1)))
    qn, kn = _bits(1 + 0.2 * rng.standard_normal(D)), _bits(1 + 0.2 * rng.standard_normal(D))
    angles = rng.uniform(0, 6.28, (lanes, 16, 64))
    cosines, sines = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    q, k, v = orc.draft_prepare(qkv, qn, kn, cosines, sines)
    for lane, row, head in [(0, 0, 0), (0, 3, 17), (1, 7, 31), (1, 2, 5)]:
        packed = qkv[lane * ROWS + row]
        want = _prepared_head(packed[head * D:(head + 1) * D], qn, cosines[lane, row].astype(np.float64), sines[lane, row].astype(np.float64))
        # the normalized value's own rounding moves the rotated one by up to a step of the larger of the pair
        bound = _bf16_step(want) + 2.0 ** -8 * np.abs(_f64(q[lane, head, row])).max()
        assert np.all(np.abs(_f64(q[lane, head, row]) - want) <= bound), (lane, row, head)
        if head < KVH:
            want = _prepared_head(packed[4096 + head * D:4096 + (head + 1) * D], kn, cosines[lane, row].astype(np.float64),
                                  sines[lane, row].astype(np.float64))
            assert np.all(np.abs(_f64(k[lane, head, row]) - want) <= _bf16_step(want) + 2.0 ** -8 * np.abs(want).max())
            assert np.array_equal(v[lane, head, :, row], packed[5120 + head * D:5120 + (head + 1) * D])


def test_preparation_pairs_dimension_i_with_i_plus_64():
    """A quarter turn (cos 0, sin 1) of one pair alone: out[i] = -n[i + 64], out[i + 64] = n[i], every other dimension as it was."""
    rng = np.random.default_rng(8)
    qkv = _bits(rng.standard_normal((ROWS, 6144)))
    ones = _bits(np.ones(D))
    cosines, sines = np.ones((1, 16, 64), np.float32), np.zeros((1, 16, 64), np.float32)
    plain, _, _ = orc.draft_prepare(qkv, ones, ones, cosines, sines)
    cosines[0, 2, 5], sines[0, 2, 5] = 0.0, 1.0
    turned, _, _ = orc.draft_prepare(qkv, ones, ones, cosines, sines)
    n = _f64(plain[0, 9, 2])
    t = _f64(turned[0, 9, 2])
    assert t[5] == -n[69] and t[69] == n[5]
    keep = np.ones(D, bool)
    keep[[5, 69]] = False
    assert np.array_equal(turned[0, 9, 2][keep], plain[0, 9, 2][keep])
    assert np.array_equal(turned[0, 9, 3], plain[0, 9, 3])     # RoPE row 2 turns query row 2 alone


# ------------------------------------------------------------------ the ring writers (draft_context_kv.h:10-45)
def test_context_rows_land_in_the_slots_of_their_positions():
    rng = np.random.default_rng(9)
    rows = 6
    context = _bits(rng.standard_normal((rows, 2048)))
    kn = _bits(1 + 0.1 * rng.standard_normal(D))
    angles = rng.uniform(0, 6.28, (16, 64))
    cosines, sines = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    keys, values = np.full((KVH, WINDOW, D), 0x1234, np.uint16), np.full((KVH, D, WINDOW), 0x1234, np.uint16)
    source, positions, rope = [4, 1, 5], [2046, 2047, 2048], [0, 1, 2]       # the third wraps to slot 0
    orc.draft_context_write(context, kn, cosines, sines, source, positions, rope, keys, values)
    touched = np.zeros(WINDOW, bool)
    for src, position, r in zip(source, positions, rope):
        slot = position % WINDOW
        touched[slot] = True
        for head in (0, 7):
            want = _prepared_head(context[src, head * D:(head + 1) * D], kn, cosines[r].astype(np.float64), sines[r].astype(np.float64))
            assert np.all(np.abs(_f64(keys[head, slot]) - want) <= _bf16_step(want) + 2.0 ** -8 * np.abs(want).max())
            assert np.array_equal(values[head, :, slot], context[src, 1024 + head * D:1024 + (head + 1) * D])
    assert np.all(keys[:, ~touched] == 0x1234) and np.all(values[:, :, ~touched] == 0x1234)


# ------------------------------------------------------------------ the attention (DraftAttention.hpp:80-110)
def _dense_attention(queries, ring_keys, ring_values, query_keys, query_values, cache):
    """Row r at position cache + r: softmax over the ring's positions max(0, cache + r - 2047) .. cache - 1 and the eight
    current rows, all of them (a block's rows see each other both ways)."""
    q = _f64(queries)
    out = np.empty((32, D))
    for row in range(32):
        position = cache + row % ROWS
        history = np.arange(max(0, position - (WINDOW - 1)), cache)
        k = np.concatenate([_f64(ring_keys)[history % WINDOW], _f64(query_keys)])
        v = np.concatenate([_f64(ring_values)[:, history % WINDOW].T, _f64(query_values).T])
        s = k @ q[row] / np.sqrt(D)
        w = np.exp(s - s.max())
        out[row] = w @ v / w.sum()
    return out


@pytest.mark.parametrize("cache", [0, 1, 130, 2040, 2047, 2048, 2050, 5000])
def test_attention_is_the_dense_softmax_over_each_rows_window(cache):
    rng = np.random.default_rng(100 + cache)
    queries = _bits(rng.standard_normal((32, D)))
    ring_keys, ring_values = _bits(rng.standard_normal((WINDOW, D))), _bits(rng.standard_normal((D, WINDOW)))
    query_keys, query_values = _bits(rng.standard_normal((ROWS, D))), _bits(rng.standard_normal((D, ROWS)))
    got = orc.draft_attention(queries, ring_keys, ring_values, query_keys, query_values, cache)
    want = _dense_attention(queries, ring_keys, ring_values, query_keys, query_values, cache)
    assert np.abs(got - want).max() < 1e-9


def test_attention_window_ends_exactly_2047_positions_back():
    """One position carries a huge value: row r sees it only while it is inside the row's own window, so at cache 2050 the
    position 3 + r' is visible to rows r <= r' alone."""
    rng = np.random.default_rng(3)
    cache = 2050
    queries = _bits(np.ones((32, D)) * 0.1)
    ring_keys, ring_values = _bits(np.zeros((WINDOW, D))), _bits(rng.standard_normal((D, WINDOW)) * 0.01)
    marked = 6     # position 6: the oldest position of row 3's window (cache + 3 - 2047)
    ring_values[:, marked % WINDOW] = _bits(np.full(D, 100.0))
    got = orc.draft_attention(queries, ring_keys, ring_values, _bits(np.zeros((ROWS, D))), _bits(np.zeros((D, ROWS))), cache)
    sees = got[:, 0] > 0.04     # uniform weights: 100 / 2055 where visible
    assert sees.reshape(4, ROWS).tolist() == [[r <= 3 for r in range(ROWS)]] * 4


# ------------------------------------------------------------------ the context window (draft_context_window.h:37-64)
def test_window_codes_restore_within_half_a_step_and_keep_other_slots():
    rng = np.random.default_rng(12)
    width, rows, start = 256, 5, 2046
    context = _bits(rng.standard_normal((8, width)) * rng.uniform(0.1, 10, (8, 1)))
    context[3, :64] = _bits(np.full(64, 1.5))           # a constant group: scale 0, every code 0
    window = np.full(orc.draft_window_bytes(width), 0xAB, np.uint8)
    source = [7, 3, 0, 2, 5]
    orc.draft_window_store(context, source, start, window)
    restored = _f64(orc.draft_window_load(window, rows, start, width))
    pairs = window[WINDOW * width // 2:].view(np.float16).reshape(WINDOW, width // 64, 2).astype(np.float64)
    for i, src in enumerate(source):
        slot = (start + i) % WINDOW
        x = _f64(context[src]).reshape(-1, 64)
        scale, minimum = pairs[slot, :, 0:1], pairs[slot, :, 1:2]
        low, high = x.min(axis=1, keepdims=True), x.max(axis=1, keepdims=True)
        assert np.all(np.abs(minimum - low) <= np.abs(low) * 2.0 ** -11 + 1e-7)
        assert np.all(np.abs(scale - (high - low) / 15) <= (high - low) / 15 * 2.0 ** -10 + 1e-7)
        # a code is the nearest step from the stored minimum, clamped to 0..15: past code 15 a value may lie up to
        # the stored scale's rounding (15 * scale * 2^-11) beyond the last step
        bound = scale / 2 + 15 * scale * 2.0 ** -10 + _bf16_step(x) + np.abs(low) * 2.0 ** -10
        assert np.all(np.abs(restored[i].reshape(-1, 64) - x) <= bound)
        codes = window[slot * width // 2:(slot + 1) * width // 2]
        unpacked = np.stack([codes & 15, codes >> 4], axis=1).reshape(-1, 64)
        want = np.clip(np.rint((x - minimum) / np.where(scale > 0, scale, 1)), 0, 15) * (scale > 0)
        assert (unpacked != want).mean() < 0.01        # fp32 against fp64 quotients differ only at exact halves
    assert np.all(restored[1][:64] == 1.5)
    slots = [(start + i) % WINDOW for i in range(rows)]
    others = np.ones(WINDOW, bool)
    others[slots] = False
    assert np.all(window[:WINDOW * width // 2].reshape(WINDOW, -1)[others] == 0xAB)
    assert np.all(window[WINDOW * width // 2:].reshape(WINDOW, -1)[others] == 0xAB)
