"""Gated DeltaNet verify step on the GPU against the oracle, and the tape protocol's invariants
(fold == next step, a rejected suffix never reaches the state, lanes are independent) through the C ABI."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc
from tests.gdn_case import check_prefill_against_fp64, make_layer, make_rows, make_state, make_tree, path_rows, tree_rows_array, ulps

pytestmark = pytest.mark.gpu


class Layer:
    """One GDN layer's weights on the device, and cells and tape slots for `lanes` lanes."""

    def __init__(self, backend, rng, key_heads, value_heads, lanes, layers=1, float_norm=False, cells=3):
        self.backend = backend
        self.shape, self.conv_w, self.a_scale, self.dt_bias, self.norm = make_layer(rng, key_heads, value_heads, float_norm)
        self.float_norm = float_norm
        self.gdn = ops.GDN(key_heads, value_heads, layers=layers)
        self.lanes, self.cells = lanes, cells
        self.states = backend.allocate_buffer(self.gdn.cell_bytes * cells * lanes)
        self.tape = backend.allocate_buffer(self.gdn.tape_layer_bytes * layers * 2 * lanes)
        self.weights = dict(convolution_weights=backend.from_array(self.conv_w), decay_weights=backend.from_array(self.a_scale),
                            time_bias=backend.from_array(self.dt_bias), mixer_norm=backend.from_array(self.norm))

    def cell(self, lane, which):
        return (lane * self.cells + which) * self.gdn.cell_bytes

    def slot(self, lane, parity, layer=0):
        return ((lane * 2 + parity) * self.gdn.layers + layer) * self.gdn.tape_layer_bytes

    def write_cell(self, lane, which, conv, state, layer=0):
        st = self.gdn.strides
        self.states.upload(np.ascontiguousarray(conv), self.cell(lane, which) + layer * st.convolution_layer_bytes)
        self.states.upload(np.ascontiguousarray(state), self.cell(lane, which) + st.convolution_state_bytes + layer * st.recurrent_layer_bytes)

    def read_cell(self, lane, which, layer=0):
        st = self.gdn.strides
        raw = self.states.download(np.uint8)
        base = self.cell(lane, which)
        conv = raw[base + layer * st.convolution_layer_bytes:][:3 * self.shape.conv_dim * 2].view(np.uint16).reshape(3, self.shape.conv_dim)
        at = base + st.convolution_state_bytes + layer * st.recurrent_layer_bytes
        state = raw[at:at + st.recurrent_layer_bytes].view(np.float32).reshape(self.shape.value_heads, 128, 128)
        return conv.copy(), state.copy()

    def read_tape(self, lane, parity, layer=0):
        raw = self.tape.download(np.uint8)
        return raw[self.slot(lane, parity, layer):][:self.gdn.tape_layer_bytes].copy()

    def step(self, blocks, layer=0):
        """blocks: [(lane, packed rows, pending_path, parity, current cell, next cell[, path masks])]; a block without
        masks is a chain. Returns hidden rows per block."""
        packed = np.concatenate([b[1] for b in blocks])
        rows = packed.shape[0]
        hidden = self.backend.allocate_buffer(rows * self.shape.value_heads * 128 * 2)
        tree = np.concatenate([tree_rows_array(b[6] if len(b) > 6 else [(2 << r) - 1 for r in range(b[1].shape[0])]) for b in blocks])
        lanes, first = [], 0
        for lane, block, path, parity, cur, nxt in (b[:6] for b in blocks):
            lanes.append(dict(first_row=first, rows=block.shape[0], pending_path=path, pending_tape=self.slot(lane, parity ^ 1, layer),
                              step_tape=self.slot(lane, parity, layer), current_cell=self.cell(lane, cur), next_cell=self.cell(lane, nxt)))
            first += block.shape[0]
        graph = splash_amd.CommandGraph()
        width = self.shape.value_heads * 128
        table = self.backend.allocate_buffer(ops.gguf_table_bytes(width, rows))
        buffers = dict(packed=self.backend.from_array(packed), states=self.states, tape=self.tape, hidden=hidden,
                       tree_rows=self.backend.from_array(tree), hidden_table=table, **self.weights)
        self.gdn.add_decode(graph, buffers, layer, lanes, float_norm=self.float_norm)
        self.backend.run(graph)
        out = hidden.download(np.uint16).reshape(rows, width)
        # the hidden rows also left as the activation table of the projection that reads them: bit for bit the table
        # pass's, piece by piece of 64 rows (rows of a tile past the step's keep what the buffer held)
        orc.assert_table_holds(table.download(np.uint8), out, lambda count: ops.gguf_table_bytes(width, count))
        return [out[l["first_row"]:l["first_row"] + l["rows"]] for l in lanes]


@pytest.mark.parametrize("heads,float_norm", [((2, 4), False), ((16, 32), True)])
def test_step_matches_the_oracle(backend, heads, float_norm):
    """gdn_decode_metal_test.mm:373-598: k/v rows, gates, the folded state and the gated outputs. The GPU's
    exp2 and log2 differ from the host's in their last bits, so rows may move by a bf16 step."""
    print(f"case gdn step heads={heads}", flush=True)
    rng = np.random.default_rng(21)
    layer = Layer(backend, rng, *heads, lanes=1, float_norm=float_norm)
    shape = layer.shape
    conv_in, state_in = make_state(rng, shape)
    first, second = make_rows(rng, shape, 16), make_rows(rng, shape, 9)
    layer.write_cell(0, 0, conv_in, state_in)
    (hidden0,) = layer.step([(0, first, 0, 0, 0, 1)])
    conv0, state0, tape0, want0 = orc.gdn_decode(shape, first, layer.conv_w, layer.a_scale, layer.dt_bias, layer.norm, conv_in, state_in)
    got_conv, got_state = layer.read_cell(0, 1)
    assert np.array_equal(got_conv, conv0) and got_state.tobytes() == state0.tobytes()   # nothing pending: copied
    got = orc.gdn_split_tape(shape, layer.read_tape(0, 0))
    want = orc.gdn_split_tape(shape, tape0)
    assert np.array_equal(got[0], want[0])
    assert ulps(got[1], want[1]).max() <= 1 and (ulps(got[1], want[1]) > 0).mean() < 0.01
    assert ulps(got[3], want[3]).max() <= 1
    assert np.all(np.abs(got[2] - want[2]) <= 1e-5 * want[2] + 1e-12)

    def close(got_bits, want_bits):
        g, w = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(want_bits).astype(np.float64)
        scale = np.abs(w).reshape(w.shape[0], -1, 128).max(axis=2, keepdims=True).repeat(128, axis=2).reshape(w.shape)
        error = np.abs(g - w)
        assert np.all(error <= 2.0 ** -6 * np.abs(w) + 2.0 ** -7 * scale), error.max()
        assert (ulps(got_bits, want_bits) <= 1).mean() >= 0.97
    close(hidden0, want0)
    # second step: folds the first 11 rows; the oracle folds the GPU's own tape so that only the fold is compared
    path = (1 << 11) - 1
    (hidden1,) = layer.step([(0, second, path, 1, 1, 2)])
    conv1, state1, _, want1 = orc.gdn_decode(shape, second, layer.conv_w, layer.a_scale, layer.dt_bias, layer.norm, got_conv, got_state,
                                             pending_tape=layer.read_tape(0, 0), pending_path=path)
    got_conv1, got_state1 = layer.read_cell(0, 2)
    assert np.array_equal(got_conv1, conv1)
    assert np.abs(got_state1 - state1).max() <= 1e-4 * np.abs(state1).max()     # state: 1e-4 relative (:531)
    close(hidden1, want1)


def test_fold_rollback_and_lane_independence(backend):
    """Bitwise on the GPU: the fold of a step's accepted rows is the cell the next step writes; a step of only
    the accepted rows leaves the same cell; lanes of one dispatch equal each alone; one chain equals its pieces."""
    print("case gdn invariants", flush=True)
    rng = np.random.default_rng(22)
    lanes = 3
    layer = Layer(backend, rng, 4, 8, lanes=lanes, cells=4)
    shape = layer.shape
    cells = [make_state(rng, shape) for _ in range(lanes)]
    firsts = [make_rows(rng, shape, r) for r in (16, 8, 3)]
    seconds = [make_rows(rng, shape, r) for r in (5, 16, 1)]
    accepted = [7, 8, 0]
    for lane in range(lanes):
        layer.write_cell(lane, 0, *cells[lane])
    hidden_a = layer.step([(lane, firsts[lane], 0, 0, 0, 1) for lane in range(lanes)])
    paths = [(1 << a) - 1 for a in accepted]
    hidden_b = layer.step([(lane, seconds[lane], paths[lane], 1, 1, 2) for lane in range(lanes)])
    after = [layer.read_cell(lane, 2) for lane in range(lanes)]
    tapes = [layer.read_tape(lane, 0) for lane in range(lanes)]
    for lane in range(lanes):
        # each lane alone, from scratch, in a fresh layer object sharing the weights
        solo = Layer(backend, np.random.default_rng(22), 4, 8, lanes=1, cells=4)
        solo.write_cell(0, 0, *cells[lane])
        (ha,) = solo.step([(0, firsts[lane], 0, 0, 0, 1)])
        (hb,) = solo.step([(0, seconds[lane], paths[lane], 1, 1, 2)])
        assert np.array_equal(ha, hidden_a[lane]) and np.array_equal(hb, hidden_b[lane])
        conv, state = solo.read_cell(0, 2)
        assert np.array_equal(conv, after[lane][0]) and state.tobytes() == after[lane][1].tobytes()
        assert np.array_equal(solo.read_tape(0, 0), tapes[lane])
        if not accepted[lane]:
            assert state.tobytes() == cells[lane][1].tobytes()
            continue
        # the fold alone of the accepted rows into cell 3
        retained = backend.from_array(np.array([paths[lane]], np.uint32))
        graph = splash_amd.CommandGraph()
        solo.gdn.add_fold(graph, solo.states, solo.tape, retained, solo.slot(0, 0), solo.cell(0, 1), solo.cell(0, 3), accepted[lane])
        backend.run(graph)
        fconv, fstate = solo.read_cell(0, 3)
        assert np.array_equal(fconv, conv) and fstate.tobytes() == state.tobytes()
        # the same against the oracle's fold of the GPU's tape: identical arithmetic, identical bits
        c1, s1 = solo.read_cell(0, 1)
        rc, oconv, ostate = orc.gdn_fold(shape, c1, s1, solo.read_tape(0, 0), paths[lane], accepted[lane])
        assert rc == 0 and np.array_equal(oconv, fconv) and ostate.tobytes() == fstate.tobytes()
        # a step of only the accepted rows, wholly accepted: rejection costs nothing
        again = Layer(backend, np.random.default_rng(22), 4, 8, lanes=1, cells=4)
        again.write_cell(0, 0, *cells[lane])
        (hc,) = again.step([(0, firsts[lane][:accepted[lane]], 0, 0, 0, 1)])
        assert np.array_equal(hc, hidden_a[lane][:accepted[lane]])
        (hd,) = again.step([(0, seconds[lane], paths[lane], 1, 1, 2)])
        assert np.array_equal(hd, hb)
        conv2, state2 = again.read_cell(0, 2)
        assert np.array_equal(conv2, conv) and state2.tobytes() == state.tobytes()
        if accepted[lane] + seconds[lane].shape[0] <= 16:
            chain = Layer(backend, np.random.default_rng(22), 4, 8, lanes=1, cells=4)
            chain.write_cell(0, 0, *cells[lane])
            (he,) = chain.step([(0, np.concatenate([firsts[lane][:accepted[lane]], seconds[lane]]), 0, 0, 0, 1)])
            assert np.array_equal(he[accepted[lane]:], hb)


def test_full_size_step_keeps_the_invariants(backend):
    """35B-A3B shape (16 key heads, 32 value heads), batch 8 of 16-row blocks: fold == next step bitwise."""
    print("case gdn full size", flush=True)
    rng = np.random.default_rng(23)
    lanes = 8
    layer = Layer(backend, rng, 16, 32, lanes=lanes, cells=4)
    shape = layer.shape
    for lane in range(lanes):
        layer.write_cell(lane, 0, *make_state(rng, shape))
    layer.step([(lane, make_rows(rng, shape, 16), 0, 0, 0, 1) for lane in range(lanes)])
    paths = [(1 << (1 + 2 * lane)) - 1 for lane in range(lanes)]
    layer.step([(lane, make_rows(rng, shape, 16), paths[lane], 1, 1, 2) for lane in range(lanes)])
    for lane in range(lanes):
        retained = backend.from_array(np.array([paths[lane]], np.uint32))
        graph = splash_amd.CommandGraph()
        layer.gdn.add_fold(graph, layer.states, layer.tape, retained, layer.slot(lane, 0), layer.cell(lane, 1), layer.cell(lane, 3), 1 + 2 * lane)
        backend.run(graph)
        conv, state = layer.read_cell(lane, 2)
        fconv, fstate = layer.read_cell(lane, 3)
        assert np.array_equal(conv, fconv) and state.tobytes() == fstate.tobytes()


@pytest.mark.parametrize("heads", [(2, 4), (16, 32)])
def test_tree_blocks(backend, heads):
    """A block that is not a chain: against the oracle's tree form (same order of operations: a bf16 step where the
    GPU's exp2 differs), every row's tape entries bit for bit those of its path run as a chain on the GPU, its
    output the chain's up to the reordering of the path form; a chain lane beside a tree lane in one dispatch is
    unchanged; and the step after folds an accepted path of the tree to the state its chain leaves, bit for bit."""
    print(f"case gdn tree heads={heads}", flush=True)
    rng = np.random.default_rng(25)
    layer = Layer(backend, rng, *heads, lanes=2, cells=4)
    shape, vh = layer.shape, layer.shape.value_heads
    rows = 16
    cells = [make_state(rng, shape) for _ in range(2)]
    blocks = [make_rows(rng, shape, rows), make_rows(rng, shape, 7)]
    previous = make_rows(rng, shape, 6)
    pending = 0b101101
    masks = make_tree(rng, rows)
    for lane in range(2):
        layer.write_cell(lane, 0, *cells[lane])
    layer.step([(0, previous, 0, 0, 0, 1), (1, previous, 0, 0, 0, 1)])
    hidden_tree, hidden_chain = layer.step([(0, blocks[0], pending, 1, 1, 2, masks), (1, blocks[1], pending, 1, 1, 2)])
    conv_b, state_b = layer.read_cell(0, 1)
    want = orc.gdn_decode(shape, blocks[0], layer.conv_w, layer.a_scale, layer.dt_bias, layer.norm, conv_b, state_b,
                          pending_tape=layer.read_tape(0, 0), pending_path=pending, ancestors=masks)
    got_conv, got_state = layer.read_cell(0, 2)
    assert np.array_equal(got_conv, want[0])
    assert np.abs(got_state - want[1]).max() <= 1e-4 * np.abs(want[1]).max()

    def close(got_bits, want_bits, relative=2.0 ** -6, of_row=2.0 ** -7):
        g, w = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(want_bits).astype(np.float64)
        scale = np.abs(w).reshape(-1, vh, 128).max(axis=2, keepdims=True).repeat(128, axis=2).reshape(w.shape)
        assert np.all(np.abs(g - w) <= relative * np.abs(w) + of_row * scale), np.abs(g - w).max()
    close(hidden_tree, want[3])
    assert (ulps(hidden_tree, want[3]) <= 1).mean() >= 0.97
    # the chain lane beside it equals the chain lane alone
    solo = Layer(backend, np.random.default_rng(25), *heads, lanes=2, cells=4)
    solo.write_cell(1, 0, *cells[1])
    solo.step([(1, previous, 0, 0, 0, 1)])
    (alone,) = solo.step([(1, blocks[1], pending, 1, 1, 2)])
    assert np.array_equal(alone, hidden_chain)
    # each tree row against its path run as a chain on the GPU
    tape_tree = orc.gdn_split_tape(shape, layer.read_tape(0, 1))
    deepest = max(range(rows), key=lambda r: bin(int(masks[r])).count("1"))
    for r in sorted({deepest, rows - 1, 1}):
        path = path_rows(masks[r])
        chain = Layer(backend, np.random.default_rng(25), *heads, lanes=1, cells=4)
        chain.write_cell(0, 0, *cells[0])
        chain.step([(0, previous, 0, 0, 0, 1)])
        (hc,) = chain.step([(0, blocks[0][path], pending, 1, 1, 2)])
        tape_chain = orc.gdn_split_tape(shape, chain.read_tape(0, 1))
        last = len(path) - 1
        for part in range(4):
            assert np.array_equal(tape_tree[part][r], tape_chain[part][last]), (r, part)
        close(hidden_tree[r:r + 1], hc[last:last + 1], of_row=2.0 ** -8)
        if r != deepest:
            continue
        # accept the deepest row's path: the next step's cell and outputs are those after the chain
        nxt = make_rows(rng, shape, 4)
        (ha,) = layer.step([(0, nxt, int(masks[r]), 0, 2, 3)])
        (hb,) = chain.step([(0, nxt, (1 << len(path)) - 1, 0, 2, 3)])
        conv_a, state_a = layer.read_cell(0, 3)
        conv_c, state_c = chain.read_cell(0, 3)
        assert np.array_equal(conv_a, conv_c) and state_a.tobytes() == state_c.tobytes() and np.array_equal(ha, hb)


def test_gdn_rejects_bad_arguments(backend):
    rng = np.random.default_rng(24)
    layer = Layer(backend, rng, 2, 4, lanes=1)
    rows = make_rows(rng, layer.shape, 4)
    with pytest.raises(ValueError):
        layer.step([(0, rows, 0, 0, 0, 0)])            # reads and writes one cell
    with pytest.raises(ValueError):
        layer.step([(0, make_rows(rng, layer.shape, 17), 0, 0, 0, 1)])
    graph = splash_amd.CommandGraph()
    buffers = dict(packed=backend.from_array(rows), states=layer.states, tape=layer.tape,
                   hidden=backend.allocate_buffer(4 * layer.shape.value_heads * 256),
                   tree_rows=backend.from_array(tree_rows_array([1, 3, 7])), **layer.weights)
    lane = dict(first_row=0, rows=4, step_tape=0, current_cell=0, next_cell=layer.gdn.cell_bytes)
    with pytest.raises(ValueError, match="tree rows"):
        layer.gdn.add_decode(graph, buffers, 0, [lane])        # three tree rows for a block of four
    with pytest.raises(ValueError):
        ops.GDN(3, 4)
    assert len(graph) == 0


class Chunk:
    """A prompt chunk through GDN::addPrefill on a Layer's cells; returns the passes' rows as arrays."""

    def __init__(self, layer, tokens):
        self.layer, self.tokens = layer, tokens
        self.work = layer.gdn.prefill_workspace(layer.backend, tokens)

    def run(self, packed, lane, current, nxt, captures=(), tiled_heads=False):
        layer = self.layer
        graph = splash_amd.CommandGraph()
        buffers = dict(packed=layer.backend.from_array(packed), states=layer.states, **layer.weights, **self.work)
        layer.gdn.add_prefill(graph, buffers, 0, packed.shape[0], layer.cell(lane, current), layer.cell(lane, nxt),
                              captures=[(t, layer.cell(lane, c)) for t, c in captures], tiled_heads=tiled_heads,
                              float_norm=layer.float_norm)
        layer.backend.run(graph)
        shape, tokens = layer.shape, packed.shape[0]
        kw, vw, vh = shape.key_heads * 128, shape.value_heads * 128, shape.value_heads
        take = lambda name, dtype, width: self.work[name].download(dtype)[:tokens * width].reshape(tokens, width).copy()
        conv_out, state_out = layer.read_cell(lane, nxt)
        return dict(queries=take("queries", np.uint16, kw), keys=take("keys", np.uint16, kw), values=take("values", np.uint16, vw),
                    decay=take("decay", np.float32, vh), beta=take("beta", np.uint16, vh), recurrent=take("recurrent_rows", np.uint16, vw),
                    hidden=take("hidden", np.uint16, vw), conv_out=conv_out, state_out=state_out)


@pytest.mark.parametrize("heads,tokens,float_norm", [((2, 4), 1, False), ((2, 4), 53, False), ((16, 32), 100, True), ((2, 2), 2048, False)])
def test_prefill_passes_the_reference_checks_and_matches_the_oracle(backend, heads, tokens, float_norm):
    """gdn_metal_test.mm:215-418: each pass of the chunk against fp64 arithmetic over the pass's own inputs, under the
    reference's bounds; and the chunk against the oracle's, whose exp2 and log2 differ from the GPU's in their last bits."""
    print(f"case gdn prefill heads={heads} tokens={tokens}", flush=True)
    rng = np.random.default_rng(41)
    layer = Layer(backend, rng, *heads, lanes=1, float_norm=float_norm)
    shape = layer.shape
    conv_in, state_in = make_state(rng, shape)
    packed = make_rows(rng, shape, tokens)
    layer.write_cell(0, 0, conv_in, state_in)
    got = Chunk(layer, tokens).run(packed, 0, 0, 1)
    check_prefill_against_fp64(shape, layer.conv_w, layer.a_scale, layer.dt_bias, layer.norm, packed, conv_in, state_in, got)
    if tokens > 512:
        return
    want = orc.gdn_prefill(shape, packed, layer.conv_w, layer.a_scale, layer.dt_bias, layer.norm, conv_in, state_in)
    assert np.array_equal(got["conv_out"], want["conv_out"])
    for name in ("queries", "keys", "values"):
        assert ulps(got[name], want[name]).max() <= 1 and (ulps(got[name], want[name]) > 0).mean() < 0.01, name
    assert ulps(got["beta"], want["beta"]).max() <= 1
    assert np.all(np.abs(got["decay"] - want["decay"]) <= 1e-5 * want["decay"] + 1e-12)
    assert np.abs(got["state_out"] - want["state_out"]).max() <= 1e-4 * np.abs(want["state_out"]).max()


def test_prefill_leaves_the_cell_of_the_same_rows_as_accepted_blocks(backend):
    """Bitwise on the GPU: a chunk's k, v and gates are the tape's, and the cell it leaves is the one the same rows leave
    as verify blocks accepted whole (a step per block, then the fold of the last); a chunk in runs with captures equals
    the chunk whole, and each capture the chunk that ends there (gdn_metal_test.mm:426-480, :560-700)."""
    print("case gdn prefill invariants", flush=True)
    rng = np.random.default_rng(42)
    layer = Layer(backend, rng, 4, 8, lanes=1, cells=6)
    shape = layer.shape
    conv_in, state_in = make_state(rng, shape)
    tokens = 45
    packed = make_rows(rng, shape, tokens)
    layer.write_cell(0, 0, conv_in, state_in)
    chunk = Chunk(layer, tokens)
    whole = chunk.run(packed, 0, 0, 1)
    # the same rows as blocks of 16, 16 and 13, each accepted whole
    kw = shape.key_heads * 128
    cells, path, parity, retained = (0, 2), 0, 0, None
    for first, rows in ((0, 16), (16, 16), (32, 13)):
        layer.step([(0, packed[first:first + rows], path, parity, cells[0], cells[1])])
        _, kv, decay, beta = orc.gdn_split_tape(shape, layer.read_tape(0, parity))
        assert np.array_equal(kv[:rows, :kw], whole["keys"][first:first + rows])
        assert np.array_equal(kv[:rows, kw:], whole["values"][first:first + rows])
        assert decay[:rows].tobytes() == whole["decay"][first:first + rows].tobytes()
        assert np.array_equal(beta[:rows], whole["beta"][first:first + rows])
        path, parity, cells = (1 << rows) - 1, parity ^ 1, (cells[1], cells[0] if cells[0] != 0 else 3)
    graph = splash_amd.CommandGraph()
    layer.gdn.add_fold(graph, layer.states, layer.tape, backend.from_array(np.array([path], np.uint32)), layer.slot(0, parity ^ 1),
                       layer.cell(0, cells[0]), layer.cell(0, 4), 13)
    backend.run(graph)
    conv, state = layer.read_cell(0, 4)
    assert np.array_equal(conv, whole["conv_out"]) and state.tobytes() == whole["state_out"].tobytes()
    # runs: captures after 7 and 32 rows
    layer.write_cell(0, 0, conv_in, state_in)
    runs = chunk.run(packed, 0, 0, 1, captures=[(7, 2), (32, 3)])
    for name in whole:
        assert runs[name].tobytes() == whole[name].tobytes(), name
    for count, cell in ((7, 2), (32, 3)):
        layer.write_cell(0, 0, conv_in, state_in)
        part = Chunk(layer, count).run(packed[:count], 0, 0, 5)
        conv, state = layer.read_cell(0, cell)
        assert np.array_equal(conv, part["conv_out"]) and state.tobytes() == part["state_out"].tobytes()
    with pytest.raises(ValueError):
        chunk.run(packed, 0, 0, 0)                       # a run reads and writes different cells
    with pytest.raises(ValueError):
        chunk.run(packed, 0, 0, 1, captures=[(45, 2)])   # a capture lies inside the rows


def test_prefill_head_order(backend):
    """Tiled heads leave at (h % heads per key) * key heads + h / heads per key (gdn_metal_test.mm:703-745)."""
    rng = np.random.default_rng(43)
    layer = Layer(backend, rng, 2, 4, lanes=1)
    conv_in, state_in = make_state(rng, layer.shape)
    packed = make_rows(rng, layer.shape, 9)
    layer.write_cell(0, 0, conv_in, state_in)
    chunk = Chunk(layer, 9)
    grouped = chunk.run(packed, 0, 0, 1)
    tiled = chunk.run(packed, 0, 0, 1, tiled_heads=True)
    assert tiled["state_out"].tobytes() == grouped["state_out"].tobytes()
    g, t = grouped["hidden"].reshape(9, 4, 128), tiled["hidden"].reshape(9, 4, 128)
    for head in range(4):
        assert np.array_equal(t[:, (head % 2) * 2 + head // 2], g[:, head])
