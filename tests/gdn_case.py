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
