"""The routing oracle against a stable sort and the softmax's closed form (moe.metal:23-113)."""
import numpy as np

from tests import oracle as orc


def test_route_is_a_stable_descending_sort_with_softmax_weights():
    rng = np.random.default_rng(5)
    scores = rng.standard_normal((40, 128)).astype(np.float32)
    scores[3, 10:20] = scores[3, 5]          # ties: the lowest ids win, in id order
    scores[4, :] = 0.25                      # every expert equal
    scores[5, 7] = np.float32(3.0)
    scores[5, 90] = np.float32(3.0)
    selected, weights = orc.moe_route(scores, 8)
    order = np.lexsort((np.arange(128)[None, :].repeat(40, 0), -scores.astype(np.float64)), axis=1)[:, :8]
    assert np.array_equal(selected, order.astype(np.uint32))
    assert np.array_equal(selected[4], np.arange(8))
    assert list(selected[5][:2]) == [7, 90]
    picked = np.take_along_axis(scores.astype(np.float64), order, axis=1)
    want = np.exp(picked - picked[:, :1])
    want /= want.sum(axis=1, keepdims=True)
    assert np.abs(weights - want).max() <= 2e-7
    assert np.abs(weights.sum(axis=1) - 1).max() <= 1e-6
    assert np.all(np.diff(weights, axis=1) <= 0)


def test_combine_is_the_weighted_sum_in_rank_order():
    rng = np.random.default_rng(6)
    rows, k, hidden = 5, 4, 64
    y = orc.f32_to_bf16(rng.standard_normal((rows, k, hidden)).astype(np.float32))
    w = rng.uniform(0, 1, (rows, k)).astype(np.float32)
    res = orc.f32_to_bf16(rng.standard_normal((rows, hidden)).astype(np.float32))
    got = orc.moe_combine(y, w, res)
    value = orc.bf16_to_f32(res).copy()
    for r in range(k):
        value = value + w[:, r:r + 1] * orc.bf16_to_f32(y[:, r])          # float32, rank order
    assert np.array_equal(got, orc.f32_to_bf16(value))
    # a single route of weight one onto a zero residual returns the expert's row
    one = orc.moe_combine(y[:, :1], np.ones((rows, 1), np.float32), np.zeros((rows, hidden), np.uint16))
    assert np.array_equal(one, y[:, 0])
