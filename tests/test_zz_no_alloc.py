"""The greedy selection that allocates nothing (spo_sampling_greedy_rows_static) against the entry point it is a
variant of (spo_sampling_add_verify with greedy lanes), through the C ABI: bit-exact tokens on two calls in a row,
the second over fewer rows and a smaller vocabulary, so that anything the first call left in the library's device
array would show."""
import ctypes

import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

pytestmark = pytest.mark.gpu


def _hip():
    return ctypes.CDLL("libamdhip64.so")


def _existing(backend, logits, V, stride):
    rows = logits.shape[0]
    sizes = ops.Sampling.workspace(rows)
    b = dict(logits=backend.from_array(logits), tokens=backend.allocate_buffer(rows * 4), partial_values=backend.allocate_buffer(sizes[0]),
             partial_indices=backend.allocate_buffer(sizes[1]), draft_probabilities=None, uniforms=None, masses=backend.allocate_buffer(sizes[2]),
             ranges=backend.allocate_buffer(sizes[3]), decisions=backend.allocate_buffer(sizes[4]), input_tokens=None, tree_rows=None)
    g = splash_amd.CommandGraph()
    ops.Sampling.add_verify(g, b, V, stride, [(0, rows)], [0.0])
    backend.run(g)
    return b["tokens"].download(np.uint32)


def _rows(rng, rows, V, stride):
    logits = rng.standard_normal((rows, stride)).astype(np.float32)
    logits[:, V:] = 100.0                                  # past the vocabulary: never read
    if rows > 6:
        logits[1, [7, V // 2, V - 1]] = 9.0                # a three-way tie: the lowest id
        logits[2, :V] = -np.inf                            # nothing selectable: the sentinel
        logits[3, :V] = np.nan
        logits[4, V - 1] = 50.0                            # the last token
        logits[5, rng.random(stride) < 0.5] = np.nan
        logits[6, :V] = 1.0                                # all equal: id 0
    return logits


def test_static_greedy_rows_equal_the_workspace_entry_point_on_two_calls(backend):
    print("case static greedy rows", flush=True)
    hip = _hip()
    rng = np.random.default_rng(17)
    stream = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
    try:
        for rows, V, stride, s in ((16, 151936, 151936, None), (5, 32000, 32064, stream)):   # the second call is smaller
            logits = _rows(rng, rows, V, stride)
            device_logits = backend.from_array(logits)
            tokens = backend.allocate_buffer(rows * 4)
            tokens.fill(0xEE)
            ops.Sampling.greedy_rows_static(device_logits, rows, V, stride, tokens, s)
            assert hip.hipStreamSynchronize(s) == 0
            got = tokens.download(np.uint32)
            want = _existing(backend, logits, V, stride)
            assert np.array_equal(got, want), (rows, got, want)
            assert np.array_equal(got, np.array([orc.argmax(logits[r, :V]) for r in range(rows)], np.uint32))
        # the largest call the array holds, then one row
        for rows in (ops.Sampling.STATIC_MAXIMUM_ROWS, 1):
            logits = _rows(rng, rows, 4096, 4096)
            device_logits, tokens = backend.from_array(logits), backend.allocate_buffer(rows * 4)
            ops.Sampling.greedy_rows_static(device_logits, rows, 4096, 4096, tokens, stream)
            assert hip.hipStreamSynchronize(stream) == 0
            assert np.array_equal(tokens.download(np.uint32), np.array([orc.argmax(logits[r]) for r in range(rows)], np.uint32))
    finally:
        hip.hipStreamDestroy(stream)


def test_static_greedy_rows_rejects_what_it_cannot_hold(backend):
    logits, tokens = backend.allocate_buffer(4096), backend.allocate_buffer(4096)
    for rows, V, stride in ((ops.Sampling.STATIC_MAXIMUM_ROWS + 1, 4, 4), (0, 4, 4), (1, 0, 4), (1, 8, 4)):
        with pytest.raises(ValueError):
            ops.Sampling.greedy_rows_static(logits, rows, V, stride, tokens)
