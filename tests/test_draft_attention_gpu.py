"""ops::DraftAttention on the GPU against the oracle (the cases of the reference's draft_attention_metal_test.mm): the
dynamic convolutions and the q/k/v preparation bit for bit; the attention of a lane's eight rows over its rings and
themselves within the reference's bound (0.02 + 0.02 |x| of the fp64 rows) at its cache lengths (empty, short, one
below and at the window, wrapping, far past it); the ring writers (prompt rows, a step's retained rows through the
device's lane rows and masks) and the 4-bit context window byte for byte; what the operator refuses."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

pytestmark = pytest.mark.gpu

ROWS, QH, KVH, D, WINDOW = 8, 32, 8, 128, 2048
RING = ops.DRAFT_RING_BYTES


def bits(values):
    return orc.f32_to_bf16(np.asarray(values, np.float32))


def rope(rng, rows):
    angles = rng.uniform(0, 6.28, (rows, 64))
    return np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)


def lane_rows_array(pairs):
    return np.array(pairs, np.uint32).reshape(-1, 2)


@pytest.mark.parametrize("hidden,lanes", [(5120, 1), (2560, 3), (2048, 4), (3072, 8)])
def test_convolution_and_preparation_equal_the_oracle(backend, hidden, lanes):
    print(f"case draft surrounding phases hidden={hidden} lanes={lanes}", flush=True)
    rng = np.random.default_rng(hidden + lanes)
    op = ops.DraftAttention(hidden, lanes)
    x, residual = bits(rng.standard_normal((lanes * ROWS, hidden))), bits(rng.standard_normal((lanes * ROWS, hidden)))
    dynamic, base = bits(rng.standard_normal((lanes * ROWS, 4 * hidden // 16)) * 0.3), bits(rng.standard_normal((4, hidden)))
    bx, br, bd, bb = (backend.from_array(a) for a in (x, residual, dynamic, base))
    for finish in (False, True):
        out = backend.allocate_buffer(op.convolution_bytes)
        graph = splash_amd.CommandGraph()
        op.add_convolution(graph, bx, bd, bb, br if finish else None, out, finish)
        backend.run(graph)
        assert np.array_equal(out.download(np.uint16).reshape(x.shape), orc.draft_conv(x, dynamic, base, residual, finish)), finish
    qkv = bits(rng.standard_normal((lanes * ROWS, 6144)) * rng.uniform(0.1, 4, (lanes * ROWS, 1)))
    qn, kn = bits(1 + 0.2 * rng.standard_normal(D)), bits(1 + 0.2 * rng.standard_normal(D))
    cosines, sines = (a.reshape(lanes, 16, 64) for a in rope(rng, lanes * 16))
    grouped = backend.allocate_buffer(op.grouped_queries_bytes)
    keys, values = backend.allocate_buffer(op.query_keys_bytes), backend.allocate_buffer(op.query_values_bytes)
    graph = splash_amd.CommandGraph()
    # the RoPE tables hold exactly what the kernel reads: the last lane's first eight rows end them
    trimmed = lambda t: backend.from_array(np.ascontiguousarray(t.reshape(-1, 64)[:(lanes - 1) * 16 + ROWS]))
    op.add_prepare(graph, backend.from_array(qkv), grouped, backend.from_array(qn), backend.from_array(kn), trimmed(cosines), trimmed(sines),
                   keys, values)
    backend.run(graph)
    q, k, v = orc.draft_prepare(qkv, qn, kn, cosines, sines)
    assert np.array_equal(grouped.download(np.uint16)[:q.size].reshape(q.shape), q)
    assert np.array_equal(keys.download(np.uint16).reshape(k.shape), k)
    assert np.array_equal(values.download(np.uint16).reshape(v.shape), v)


@pytest.mark.parametrize("cache_lengths", [(0,), (2048, 2047), (2100, 4094, 6143), (262137, 4094, 500, 6143), (512, 513, 1024, 1536),
                                           (2046, 2049, 4095, 4096), (8191, 262144), (1, 127, 128, 129, 2045, 3000, 33, 70000)])
def test_attention_over_the_rings_and_the_current_rows(backend, cache_lengths):
    print(f"case draft attention cache lengths={cache_lengths}", flush=True)
    lanes = len(cache_lengths)
    rng = np.random.default_rng(sum(cache_lengths) + lanes)
    op = ops.DraftAttention(5120, lanes)
    unit = lambda shape: bits(rng.uniform(-1, 1, shape))
    queries = unit((lanes, KVH, 32, D))
    ring_keys, ring_values = unit((lanes, KVH, WINDOW, D)), unit((lanes, KVH, D, WINDOW))
    query_keys, query_values = unit((lanes, KVH, ROWS, D)), unit((lanes, KVH, D, ROWS))
    # lane l's rings: keys, then values, after a gap the kernel must not read (NaN: a weight of zero times it is NaN)
    stride = 2 * RING + 4096
    raw = np.full(lanes * stride // 2, 0x7FC0, np.uint16)
    for lane in range(lanes):
        at = lane * stride // 2
        raw[at:at + RING // 2] = ring_keys[lane].ravel()
        raw[at + RING // 2:at + RING] = ring_values[lane].ravel()
    rings = backend.from_array(raw)
    grouped = backend.allocate_buffer(op.grouped_queries_bytes)
    grouped.upload(queries)
    graph = splash_amd.CommandGraph()
    op.add_decode(graph, grouped, rings, [lane * stride for lane in range(lanes)], [lane * stride + RING for lane in range(lanes)],
                  backend.from_array(query_keys), backend.from_array(query_values), list(cache_lengths))
    assert len(graph.kernels()) == 2
    backend.run(graph)
    got = orc.bf16_to_f32(grouped.download(np.uint16)[:lanes * ROWS * 4096]).reshape(lanes, ROWS, QH, D)
    assert np.all(np.isfinite(got))
    worst = 0.0
    for lane in range(lanes):
        for head in range(KVH):
            want = orc.draft_attention(queries[lane, head], ring_keys[lane, head], ring_values[lane, head], query_keys[lane, head],
                                       query_values[lane, head], cache_lengths[lane]).reshape(4, ROWS, D)
            mine = got[lane, :, 4 * head:4 * head + 4].transpose(1, 0, 2)    # [query head of the group][row][dimension]
            error = np.abs(mine - want)
            assert np.all(error <= 0.02 + 0.02 * np.abs(want)), (lane, head, float(error.max()))
            worst = max(worst, float(error.max()))
    print(f"  largest difference from the fp64 rows {worst:.5f}", flush=True)
    assert worst < 4e-3      # the rounding of a bf16 output of magnitude below one, and of bf16 weights


def test_a_lanes_rows_do_not_depend_on_the_other_lanes(backend):
    print("case draft attention batching", flush=True)
    rng = np.random.default_rng(77)
    caches = [3000, 17, 2047]
    unit = lambda shape: bits(rng.uniform(-1, 1, shape))
    queries, query_keys, query_values = unit((3, KVH, 32, D)), unit((3, KVH, ROWS, D)), unit((3, KVH, D, ROWS))
    rings = backend.from_array(unit((3, 2, RING // 2)))
    outputs = []
    for chosen in ([0, 1, 2], [2], [1, 0]):
        op = ops.DraftAttention(2048, len(chosen))
        grouped = backend.allocate_buffer(op.grouped_queries_bytes)
        grouped.upload(np.ascontiguousarray(queries[chosen]))
        graph = splash_amd.CommandGraph()
        op.add_decode(graph, grouped, rings, [2 * RING * l for l in chosen], [2 * RING * l + RING for l in chosen],
                      backend.from_array(np.ascontiguousarray(query_keys[chosen])), backend.from_array(np.ascontiguousarray(query_values[chosen])),
                      [caches[l] for l in chosen])
        backend.run(graph)
        outputs.append(dict(zip(chosen, grouped.download(np.uint16)[:len(chosen) * ROWS * 4096].reshape(len(chosen), -1))))
    assert np.array_equal(outputs[0][2], outputs[1][2]) and np.array_equal(outputs[0][1], outputs[2][1]) and np.array_equal(outputs[0][0], outputs[2][0])


def test_context_rows_reach_their_slots(backend):
    """Prompt rows from a start position that wraps the ring, then a step's retained rows: lane rows and masks read from
    the device, the path's i-th row at the lane's start position plus i under the lane's RoPE row i."""
    print("case draft context writers", flush=True)
    rng = np.random.default_rng(21)
    op = ops.DraftAttention(2048, 3)
    kn = bits(1 + 0.1 * rng.standard_normal(D))
    raw = bits(rng.standard_normal((3, 2, RING // 2)))
    rings = backend.from_array(raw)
    want = raw.copy()
    keys_of = lambda lane: want[lane, 0].reshape(KVH, WINDOW, D)
    values_of = lambda lane: want[lane, 1].reshape(KVH, D, WINDOW)
    # prefill: 300 rows of lane 1 from position 1900 (the last 152 wrap)
    tokens, start = 300, 1900
    context = bits(rng.standard_normal((tokens, 2048)))
    cosines, sines = rope(rng, tokens)
    graph = splash_amd.CommandGraph()
    op.add_context_prefill(graph, backend.from_array(context), backend.from_array(kn), backend.from_array(cosines), backend.from_array(sines),
                           rings, 2 * RING, 3 * RING, tokens, start)
    backend.run(graph)
    orc.draft_context_write(context, kn, cosines, sines, np.arange(tokens), start + np.arange(tokens), np.arange(tokens), keys_of(1), values_of(1))
    assert np.array_equal(rings.download(np.uint16).reshape(raw.shape), want)
    # commit: a step of 3 lanes (5, 16 and 9 rows); lane 0 retained rows 0, 2, 3; lane 1 all sixteen; lane 2 seven of its
    # nine and a stray bit past them, which names no row of the lane and writes nothing
    lane_rows = lane_rows_array([(0, 5), (5, 16), (21, 9)])
    retained = np.array([0b01101, 0xFFFF, 0b100000110110111], np.uint32)
    starts = [2040, 70000, 5]
    step_rows = 30
    context = bits(rng.standard_normal((step_rows, 2048)))
    cosines, sines = rope(rng, 3 * 16)
    graph = splash_amd.CommandGraph()
    op.add_context_commit(graph, backend.from_array(context), backend.from_array(kn), backend.from_array(cosines), backend.from_array(sines),
                          rings, [0, 2 * RING, 4 * RING], [RING, 3 * RING, 5 * RING], backend.from_array(retained),
                          backend.from_array(lane_rows), starts, step_rows, 16)
    backend.run(graph)
    for lane in range(3):
        path = [b for b in range(32) if retained[lane] >> b & 1 and b < lane_rows[lane, 1]]
        orc.draft_context_write(context, kn, cosines, sines, lane_rows[lane, 0] + np.array(path), starts[lane] + np.arange(len(path)),
                                16 * lane + np.arange(len(path)), keys_of(lane), values_of(lane))
    assert np.array_equal(rings.download(np.uint16).reshape(raw.shape), want)


@pytest.mark.parametrize("width", [2048, 5120])
def test_context_window_bytes_are_the_oracles(backend, width):
    print(f"case draft context window width={width}", flush=True)
    rng = np.random.default_rng(width)
    size = ops.DraftAttention.window_bytes(width)
    assert size == orc.draft_window_bytes(width) == WINDOW * (width // 2 + width // 64 * 4)
    window = backend.from_array(np.full(size, 0xAB, np.uint8))
    want = np.full(size, 0xAB, np.uint8)
    rows, start = 40, 2030
    context = bits(rng.standard_normal((rows, width)) * rng.uniform(0.01, 20, (rows, 1)))
    context[5, 64:128] = bits(np.full(64, -2.25))      # a constant group
    graph = splash_amd.CommandGraph()
    ops.DraftAttention.add_window_store(graph, backend.from_array(context), window, rows, start, width)
    backend.run(graph)
    orc.draft_window_store(context, np.arange(rows), start, want)
    assert np.array_equal(window.download(np.uint8), want)
    # a lane's retained rows of a step, as the context commit picks them
    step = bits(rng.standard_normal((20, width)))
    graph = splash_amd.CommandGraph()
    ops.DraftAttention.add_window_commit(graph, backend.from_array(step), window, backend.from_array(np.array([0b1011001], np.uint32)),
                                         backend.from_array(lane_rows_array([(9, 11)])), 20, 16, 2046, width)
    backend.run(graph)
    orc.draft_window_store(step, 9 + np.array([0, 3, 4, 6]), 2046, want)
    assert np.array_equal(window.download(np.uint8), want)
    # and back
    loaded = backend.allocate_buffer(48 * width * 2)
    graph = splash_amd.CommandGraph()
    ops.DraftAttention.add_window_load(graph, window, loaded, 48, 2020, width)
    backend.run(graph)
    assert np.array_equal(loaded.download(np.uint16).reshape(48, width), orc.draft_window_load(want, 48, 2020, width))


def test_mask_rows_fill_rows_one_to_seven(backend):
    print("case draft mask rows", flush=True)
    rng = np.random.default_rng(2)
    width, lanes = 2560, 3
    rows = bits(rng.standard_normal((lanes * ROWS, width)))
    mask = bits(rng.standard_normal(width))
    buffer = backend.from_array(rows)
    graph = splash_amd.CommandGraph()
    ops.DraftAttention.add_mask_rows(graph, backend.from_array(mask), buffer, width, lanes)
    backend.run(graph)
    want = rows.reshape(lanes, ROWS, width).copy()
    want[:, 1:] = mask
    assert np.array_equal(buffer.download(np.uint16).reshape(want.shape), want)


def test_the_operator_refuses_what_it_cannot_run(backend):
    print("case draft attention refusals", flush=True)
    op = ops.DraftAttention(2048, 2)
    small = backend.allocate_buffer(64)
    big = backend.allocate_buffer(op.grouped_queries_bytes)
    rings = backend.allocate_buffer(4 * RING)
    graph = splash_amd.CommandGraph()
    with pytest.raises(splash_amd.SplashError):      # a ring that ends past its buffer
        op.add_decode(graph, big, rings, [0, 2 * RING], [RING, 3 * RING + 16], big, big, [0, 0])
    with pytest.raises(splash_amd.SplashError):      # grouped queries without room for the partials
        op.add_decode(graph, backend.allocate_buffer(2 * ROWS * 4096 * 2), rings, [0, 2 * RING], [RING, 3 * RING], big, big, [0, 0])
    with pytest.raises(splash_amd.SplashError):      # fewer cache lengths than lanes
        op.add_decode(graph, big, rings, [0], [RING], big, big, [0])
    with pytest.raises(splash_amd.SplashError):
        op.add_convolution(graph, small, big, big, None, big, False)
    with pytest.raises(splash_amd.SplashError):      # a window of a width that is no whole number of groups
        ops.DraftAttention.add_window_store(graph, big, big, 4, 0, 2080)
    with pytest.raises(splash_amd.SplashError):      # more rows than a verify block's
        ops.DraftAttention.add_window_commit(graph, big, backend.allocate_buffer(ops.DraftAttention.window_bytes(2048)), small, small, 40, 17, 0, 2048)
    assert len(graph.kernels()) == 0
