"""Synthetic inputs of a Gated DeltaNet layer for the oracle and GPU tests."""
import numpy as np

from tests import oracle as orc


def make_layer(rng, key_heads, value_heads, float_norm=False):
    shape = orc.gdn_shape(key_heads, value_heads, flags=4 if float_norm else 0)
    conv_w = orc.f32_to_bf16((rng.standard_normal((shape.conv_dim, 4)) * 0.4).astype(np.float32))
    a_scale = (-np.exp(rng.uniform(-1.0, 1.0, value_heads))).astype(np.float32)   # decay = exp(a_scale softplus) in (0, 1)
    dt_bias = orc.f32_to_bf16(rng.uniform(-1.0, 1.0, value_heads).astype(np.float32))
    norm = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    norm_weight = norm if float_norm else orc.f32_to_bf16(norm)
    return shape, conv_w, a_scale, dt_bias, norm_weight


def make_rows(rng, shape, rows):
    return orc.f32_to_bf16(rng.standard_normal((rows, shape.packed_width)).astype(np.float32))


def make_state(rng, shape):
    conv = orc.f32_to_bf16(rng.standard_normal((3, shape.conv_dim)).astype(np.float32))
    state = (rng.standard_normal((shape.value_heads, 128, 128)) * 0.05).astype(np.float32)
    return conv, state


def ulps(a_bits, b_bits):
    """Distance in bf16 steps between two arrays of bf16 bit patterns (same-sign finite values)."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, 0x8000 - x, x)
    return np.abs(key(np.asarray(a_bits)) - key(np.asarray(b_bits)))


def make_tree(rng, rows):
    """A random tree over `rows` block rows, row 0 its root: each row's parent is an earlier row. Returns the
    rows' path masks (bit j: row j is on the row's path, itself included)."""
    masks = np.zeros(rows, np.uint32)
    masks[0] = 1
    for r in range(1, rows):
        masks[r] = masks[int(rng.integers(0, r))] | np.uint32(1 << r)
    return masks


def path_rows(mask):
    return [j for j in range(32) if (int(mask) >> j) & 1]


def tree_rows_array(masks):
    """The 8-byte tree rows (uint32 ancestors, uint16 parent, uint16 depth) of path masks."""
    out = np.zeros((len(masks), 2), np.uint32)
    for r, m in enumerate(masks):
        path = path_rows(m)
        parent = path[-2] if len(path) > 1 else 0xFFFF
        out[r] = (int(m), parent | ((len(path) - 1) << 16))
    return out


def check_prefill_against_fp64(shape, conv_w, a_scale, dt_bias, norm, packed, conv_in, state_in, got):
    """The reference's checks of its prefill (gdn_metal_test.mm:236-409) on the dict `got` of a chunk's outputs: each
    pass against fp64 arithmetic over the pass's own inputs, with the reference's bounds."""
    f = lambda bits: orc.bf16_to_f32(np.asarray(bits)).astype(np.float64)
    rnd = lambda x: f(orc.f32_to_bf16(np.asarray(x, np.float64).astype(np.float32)))
    step = lambda ref: np.maximum(np.abs(ref), 1e-30) * 0.0078125
    tokens, kh, vh, C = packed.shape[0], shape.key_heads, shape.value_heads, shape.conv_dim
    # prepare: convolution + SiLU rounded where the kernel rounds, q/k normed per head (:236-284): within 2 bf16 steps
    inputs = np.concatenate([f(conv_in), f(packed[:, :C])])
    w = f(conv_w)
    conv = sum(inputs[tap:tap + tokens] * w[None, :, tap] for tap in range(4))
    conv = rnd(conv)
    conv = rnd(conv / (1 + np.exp(-conv)))
    for which, name, scale in ((0, "queries", 0.0078125), (1, "keys", 0.08838834765)):
        heads = conv[:, which * kh * 128:(which + 1) * kh * 128].reshape(tokens, kh, 128)
        inverse = 1 / np.sqrt((heads ** 2).mean(axis=2, keepdims=True) + 1e-6)
        ref = rnd(rnd(heads * inverse) * scale).reshape(tokens, kh * 128)
        assert np.all(np.abs(f(got[name]) - ref) <= 2 * step(ref)), name
    ref = conv[:, 2 * kh * 128:]
    assert np.all(np.abs(f(got["values"]) - ref) <= 2 * step(ref))
    # gates (:288-312): beta within a bf16 step; the decay between those of the softplus's bf16 neighbours
    b = f(packed[:, C + vh * 128:C + vh * 128 + vh])
    ref = rnd(1 / (1 + np.exp(-b)))
    assert np.all(np.abs(f(got["beta"]) - ref) <= step(ref))
    x = rnd(f(packed[:, C + vh * 128 + vh:C + vh * 128 + 2 * vh]) + f(dt_bias)[None, :])
    nearest = orc.f32_to_bf16((np.log1p(np.exp(-np.abs(x))) + np.maximum(x, 0)).astype(np.float32)).astype(np.int32)
    a = a_scale.astype(np.float64)[None, :]
    low, high = np.exp(a * f((nearest + 1).astype(np.uint16))), np.exp(a * f((nearest - 1).astype(np.uint16)))
    assert np.all((got["decay"] >= low * (1 - 1e-5) - 1e-30) & (got["decay"] <= high * (1 + 1e-5) + 1e-30))
    # carry (:315-326): the last three inputs seen
    assert np.array_equal(got["conv_out"], np.concatenate([conv_in, packed[:, :C]])[tokens:tokens + 3])
    # the recurrence in fp64 from the pass's own q, k, v and gates (:328-381): rows within a bf16 step + 1e-5, state 1e-5
    q, k, v = f(got["queries"]), f(got["keys"]), f(got["values"])
    S = state_in.astype(np.float64).copy()
    per = vh // kh
    rows = np.zeros((tokens, vh, 128))
    for t in range(tokens):
        kt = np.repeat(k[t].reshape(kh, 128), per, axis=0)
        qt = np.repeat(q[t].reshape(kh, 128), per, axis=0)
        S *= got["decay"][t].astype(np.float64)[:, None, None]
        memory = np.einsum("hrc,hc->hr", S, kt)
        delta = (v[t].reshape(vh, 128) - memory) * f(got["beta"][t])[:, None]
        S += delta[:, :, None] * kt[:, None, :]
        rows[t] = np.einsum("hrc,hc->hr", S, qt)
    error = np.abs(f(got["recurrent"]).reshape(tokens, vh, 128) - rows)
    assert np.all(error <= step(rows) + 1e-5), (error / (step(rows) + 1e-5)).max()
    assert np.abs(got["state_out"] - S).max() <= 1e-5
    # gated norm of the pass's own rows (:383-411): within 2 bf16 steps, at most 1 % off the fp64 rounding
    own = f(got["recurrent"]).reshape(tokens, vh, 128)
    weight = norm.astype(np.float64) if norm.dtype == np.float32 else f(norm)
    normalized = rnd(own / np.sqrt((own ** 2).mean(axis=2, keepdims=True) + 1e-6) * weight)
    z = f(packed[:, C:C + vh * 128]).reshape(tokens, vh, 128)
    ref = rnd(normalized * z / (1 + np.exp(-z))).reshape(tokens, vh * 128)
    hidden = f(got["hidden"])
    assert np.all(np.abs(hidden - ref) <= 2 * step(ref))
    assert (hidden != ref).mean() <= 0.01
