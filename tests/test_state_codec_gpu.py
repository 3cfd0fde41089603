"""The cached form of recurrent layers on the GPU against the oracle, byte for byte (state_codec_metal_test.mm): the
codes and bf16 scales of every block and the values decoded from them, over fp32 and bf16 running states, layers apart
by their own strides, rows that leave most of a workgroup idle and write nothing past their layer, blocks that are not
finite, and the extents the operator refuses."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc
from tests.state_codec_case import running_state, with_non_finite

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def backend():
    b = splash_amd.Backend(0)
    yield b
    b.close()


def as_state(values, bf16):
    """The running state's bytes, and the fp32 values it holds."""
    if not bf16:
        return values.astype(np.float32), values.astype(np.float32)
    bits = orc.f32_to_bf16(values.astype(np.float32))
    return bits, orc.bf16_to_f32(bits)


def run_case(backend, rows, columns, layers, bf16, padding, non_finite=False):
    rng = np.random.default_rng(rows * 31 + layers)
    element = 2 if bf16 else 4
    state_bytes = rows * columns * element
    codes_bytes = ops.StateCodec.layer_bytes(rows, columns)
    state_stride, codes_stride = state_bytes + padding, (codes_bytes + padding + 3) // 4 * 4   # layers start on 16 and 4 bytes
    shape = ops.StateCodec.shape(layers, rows, columns, state_stride, codes_stride, bf16)
    raw = np.zeros(layers * state_stride, dtype=np.uint8)
    held = []
    for layer in range(layers):
        values = running_state(rng, rows, columns)
        if non_finite:
            values = with_non_finite(values)
        stored, wide = as_state(values, bf16)
        raw[layer * state_stride:layer * state_stride + state_bytes] = stored.view(np.uint8).reshape(-1)
        held.append(wide)
    guard = 0xA5
    state = backend.from_array(raw)
    codes = backend.from_array(np.full(layers * codes_stride, guard, dtype=np.uint8))
    restored = backend.from_array(np.full(layers * state_stride, guard, dtype=np.uint8))
    graph = splash_amd.CommandGraph()
    ops.StateCodec.add_quantize(graph, state, codes, shape)
    ops.StateCodec.add_dequantize(graph, codes, restored, shape)
    backend.run(graph)
    got_codes, got_state = codes.download(np.uint8), restored.download(np.uint8)
    for layer in range(layers):
        want = orc.state_codes(held[layer])
        mine = got_codes[layer * codes_stride:layer * codes_stride + codes_bytes]
        assert np.array_equal(mine, want), (layer, np.flatnonzero(mine != want)[:8])
        assert np.all(got_codes[layer * codes_stride + codes_bytes:(layer + 1) * codes_stride] == guard)   # nothing past the layer
        values = orc.state_values(want, rows, columns)
        stored = orc.f32_to_bf16(values) if bf16 else values
        back = got_state[layer * state_stride:layer * state_stride + state_bytes]
        expected = stored.view(np.uint8).reshape(-1)
        if non_finite:   # NaN payloads aside: compare what is finite bit for bit, and NaN as NaN
            view = back.view(np.uint16 if bf16 else np.float32)
            wide = orc.bf16_to_f32(view) if bf16 else view
            nan = np.isnan(values.reshape(-1))
            assert np.isnan(wide[nan]).all() and nan.sum() == 3 * 32
            assert np.array_equal(back.view(np.uint16 if bf16 else np.uint32)[~nan], expected.view(np.uint16 if bf16 else np.uint32)[~nan])
        else:
            assert np.array_equal(back, expected)
        assert np.all(got_state[layer * state_stride + state_bytes:(layer + 1) * state_stride] == guard)
    return held, got_codes


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,columns,layers,padding", [(4096, 128, 3, 0), (2048, 128, 2, 4096), (3, 32, 2, 16), (48, 128, 1, 0),
                                                         (16, 256, 5, 64)])
def test_codes_and_restored_values_equal_the_oracle(backend, rows, columns, layers, bf16, padding):
    print(f"case state codec rows={rows} columns={columns} layers={layers} bf16={bf16} padding={padding}", flush=True)
    held, got_codes = run_case(backend, rows, columns, layers, bf16, padding)
    # state_codec_metal_test.mm:8-10: the state restores within the bound measured on the models, a relative error of 1 %
    codes_bytes = ops.StateCodec.layer_bytes(rows, columns)
    restored = orc.state_values(got_codes[:codes_bytes], rows, columns)
    rows_used = min(rows, 9 * 32 // columns + 1)   # the case's special blocks (subnormal, huge) are in its first rows
    a, b = held[0][rows_used:].astype(np.float64), restored[rows_used:].astype(np.float64)
    if a.size:
        assert np.linalg.norm(a - b) <= 0.01 * np.linalg.norm(a)


@pytest.mark.parametrize("bf16", [False, True])
def test_blocks_that_are_not_finite_restore_as_nan(backend, bf16):
    print(f"case state codec non-finite bf16={bf16}", flush=True)
    run_case(backend, 64, 128, 2, bf16, 0, non_finite=True)


def test_copy_keeps_the_running_format(backend):
    """StateCodec::addCopy: each layer's state bytes as they are, between the two strides."""
    rng = np.random.default_rng(5)
    rows, columns, layers = 96, 128, 3
    state_bytes = rows * columns * 4
    shape = ops.StateCodec.shape(layers, rows, columns, state_bytes + 256, state_bytes + 1024)
    raw = rng.integers(0, 256, layers * (state_bytes + 256), dtype=np.uint8)
    source = backend.from_array(raw)
    destination = backend.from_array(np.full(layers * (state_bytes + 1024), 0x5A, dtype=np.uint8))
    graph = splash_amd.CommandGraph()
    ops.StateCodec.add_copy(graph, source, destination, shape)
    backend.run(graph)
    got = destination.download(np.uint8)
    for layer in range(layers):
        assert np.array_equal(got[layer * (state_bytes + 1024):][:state_bytes], raw[layer * (state_bytes + 256):][:state_bytes])
        assert np.all(got[layer * (state_bytes + 1024) + state_bytes:(layer + 1) * (state_bytes + 1024)] == 0x5A)


def test_extents_are_checked_before_anything_is_added(backend):
    """state_codec_metal_test.mm:259-276: a buffer that ends before the last layer does, and shapes that hold no
    whole blocks, are refused."""
    rows, columns, layers = 32, 128, 2
    shape = ops.StateCodec.shape(layers, rows, columns)
    state = backend.allocate_buffer(layers * rows * columns * 4)
    codes = backend.allocate_buffer(layers * ops.StateCodec.layer_bytes(rows, columns))
    graph = splash_amd.CommandGraph()
    short_state = backend.allocate_buffer(layers * rows * columns * 4 - 16)
    short_codes = backend.allocate_buffer(layers * ops.StateCodec.layer_bytes(rows, columns) - 2)
    for s, c in ((short_state, codes), (state, short_codes)):
        with pytest.raises(splash_amd.SplashError):
            ops.StateCodec.add_quantize(graph, s, c, shape)
        with pytest.raises(splash_amd.SplashError):
            ops.StateCodec.add_dequantize(graph, c, s, shape)
    for bad in (ops.StateCodec.shape(0, rows, columns), ops.StateCodec.shape(layers, rows, 48),
                ops.StateCodec.shape(layers, rows, columns, rows * columns * 4 - 16), ops.StateCodec.shape(layers, rows, columns, None, 100)):
        with pytest.raises(splash_amd.SplashError):
            ops.StateCodec.add_quantize(graph, state, codes, bad)
    with pytest.raises(splash_amd.SplashError):
        ops.StateCodec.add_copy(graph, state, codes, shape)   # the cached layer is smaller than the state it would keep
    assert len(graph) == 0
    ops.StateCodec.add_quantize(graph, state, codes, shape)
    assert graph.kernels() == ["state_quantize"]


def test_a_lane_restored_from_its_coded_state_goes_on_within_a_percent(backend):
    """State capture end to end: a Gated DeltaNet lane's cell (what GDN::addFold or a step leaves) is coded, restored
    into another cell by the codec, and the lane's next block runs from both. The restored state is within the 1 %
    the reference measured on its models (state_codec_metal_test.mm:8-10), the coded form is the oracle's byte for
    byte, and the block's outputs from the restored cell stay within a percent of those from the exact one."""
    print("case state codec restores a GDN lane", flush=True)
    from tests.gdn_case import make_rows, make_state
    from tests.test_gdn_gpu import Layer
    rng = np.random.default_rng(41)
    key_heads, value_heads = 4, 8
    layer = Layer(backend, rng, key_heads, value_heads, lanes=1, cells=4)
    conv, state = make_state(rng, layer.shape)
    layer.write_cell(0, 0, conv, state)
    first = make_rows(rng, layer.shape, 16)
    layer.step([(0, first, 0, 0, 0, 1)])                       # cell 1: the state before the block; tape 0: its rows
    second = make_rows(rng, layer.shape, 16)
    exact = layer.step([(0, second, 0xFFFF, 1, 1, 2)])[0]      # folds the sixteen rows, runs the next block; cell 2 holds the fold
    conv2, state2 = layer.read_cell(0, 2)
    # code cell 2's recurrent layer, restore it into cell 3 beside a copy of the convolution carry
    st, gdn = layer.gdn.strides, layer.gdn
    rows, columns = value_heads * 128, 128
    shape = ops.StateCodec.shape(1, rows, columns, st.recurrent_layer_bytes, ops.StateCodec.layer_bytes(rows, columns))
    view = lambda cell: layer.states.view(layer.cell(0, cell) + st.convolution_state_bytes, st.recurrent_layer_bytes)
    codes = backend.allocate_buffer(ops.StateCodec.layer_bytes(rows, columns))
    graph = splash_amd.CommandGraph()
    ops.StateCodec.add_quantize(graph, view(2), codes, shape)
    ops.StateCodec.add_dequantize(graph, codes, view(3), shape)
    backend.run(graph)
    assert np.array_equal(codes.download(np.uint8), orc.state_codes(state2.reshape(rows, columns)))
    layer.states.upload(np.ascontiguousarray(conv2), layer.cell(0, 3))
    _, restored = layer.read_cell(0, 3)
    assert np.linalg.norm(restored - state2) <= 0.01 * np.linalg.norm(state2)
    third = make_rows(rng, layer.shape, 16)
    from_exact = layer.step([(0, third, 0, 0, 2, 1)])[0]
    from_restored = layer.step([(0, third, 0, 0, 3, 1)])[0]
    a, b = orc.bf16_to_f32(from_exact).astype(np.float64), orc.bf16_to_f32(from_restored).astype(np.float64)
    assert np.linalg.norm(a - b) <= 0.01 * np.linalg.norm(a), np.linalg.norm(a - b) / np.linalg.norm(a)
    assert np.isfinite(b).all() and exact.shape == from_exact.shape
