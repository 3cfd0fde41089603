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
