"""The oracle's state codec against the reference's own CPU restatement and the closed form (CPU)."""
import numpy as np
import pytest

from tests import oracle as orc
from tests.state_codec_case import running_state, with_non_finite


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref was not built (no reference tree)")
@pytest.mark.parametrize("rows,columns", [(64, 128), (3, 32), (16, 256)])
def test_codes_equal_the_compiled_reference(rows, columns):
    rng = np.random.default_rng(rows)
    for state in (running_state(rng, rows, columns), with_non_finite(running_state(rng, rows, columns))):
        assert np.array_equal(orc.state_codes(state), orc.state_codes(state, library=orc.ref))


def test_restored_values_lie_within_half_a_step():
    """state_codec_metal_test.mm:8-10: every decoded value is within half its block's step of the value coded."""
    rng = np.random.default_rng(2)
    state = running_state(rng, 64, 128)
    image = orc.state_codes(state)
    restored = orc.state_values(image, 64, 128)
    scales = orc.bf16_to_f32(image[64 * 128:].view(np.uint16)).reshape(64, 4)
    step = np.repeat(scales, 32, axis=1).astype(np.float64)
    # the scale is the block's largest magnitude over 127 rounded to bf16: a value at the top of its block may clamp
    gap = np.abs(restored.astype(np.float64) - state.astype(np.float64))
    clamped = np.abs(state.astype(np.float64)) > 127 * step
    normal = step >= 2.0 ** -126                                      # a subnormal bf16 scale keeps few bits of amax / 127
    assert np.all(gap[~clamped] <= step[~clamped] / 2 * (1 + 1e-6))
    assert np.all(gap[clamped & normal] <= step[clamped & normal])   # bf16 rounds the scale down by at most 2^-9
    codes = image[:64 * 128].view(np.int8).reshape(64, 128)
    assert np.all(codes[0, :32] == 0) and scales[0, 0] == 0          # a block of zeros
    assert np.abs(codes).max() == 127 and codes.min() >= -127
    # ties round to even: values k + 0.5 over a scale of exactly 1/8 ... the block of halves
    block = state.reshape(-1, 32)[8]
    scale = scales.reshape(-1)[8]
    assert np.array_equal(codes.reshape(-1, 32)[8], np.clip(np.rint(block / scale), -127, 127).astype(np.int8))


def test_a_block_that_is_not_finite_restores_as_nan():
    """common/state_codec.h:12-16: a NaN scale, so every value of the block restores as NaN and no other does."""
    rng = np.random.default_rng(3)
    clean = running_state(rng, 16, 128)
    state = with_non_finite(clean)
    image = orc.state_codes(state)
    restored = orc.state_values(image, 16, 128).reshape(-1, 32)
    bad = ~np.isfinite(state.reshape(-1, 32)).all(axis=1)
    assert bad.sum() == 3
    assert np.isnan(restored[bad]).all() and np.isfinite(restored[~bad]).all()
    scales = image[16 * 128:].view(np.uint16)
    assert np.all(scales[bad] == 0x7FC0)
    good = orc.state_codes(clean)
    keep = np.repeat(~bad, 32)
    assert np.array_equal(image[:16 * 128][keep], good[:16 * 128][keep])
