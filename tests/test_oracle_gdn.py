"""The GDN oracle against the fp64 textbook recurrence (the check the reference's own test makes,
gdn_decode_metal_test.mm:373-598, with its tolerances) and against the invariants of the tape
protocol: a fold equals what the next step holds, a rejected suffix never reaches the state."""
import numpy as np
import pytest

from tests import oracle as orc
from tests.gdn_case import check_prefill_against_fp64, make_layer, make_rows, make_state, make_tree, path_rows, ulps


def test_step_matches_the_fp64_recurrence():
    rng = np.random.default_rng(3)
    shape, conv_w, a_scale, dt_bias, norm = make_layer(rng, 2, 4)
    rows = 16
    packed = make_rows(rng, shape, rows)
    conv_in, state_in = make_state(rng, shape)
    _, state0, tape, hidden = orc.gdn_decode(shape, packed, conv_w, a_scale, dt_bias, norm, conv_in, state_in)
    assert np.array_equal(state0, state_in)          # nothing pending: the state before the rows is the state
    inputs, kv, decay, beta = orc.gdn_split_tape(shape, tape)
    kv64, beta64, decay64, state64, out64 = orc.gdn_reference(shape, packed, conv_w, a_scale, dt_bias, conv_in, state_in)
    assert np.array_equal(inputs[:rows], packed[:, :shape.conv_dim])
    # k/v rows within 3 bf16 steps (:425-429), beta within 2 (:451), decay 1e-4 relative with one bf16 step on the softplus (:457-468)
    assert ulps(kv[:rows], orc.f32_to_bf16(kv64.astype(np.float32))).max() <= 3
    assert ulps(beta[:rows], orc.f32_to_bf16(beta64.astype(np.float32))).max() <= 2
    vh = shape.value_heads
    x = (orc.bf16_to_f32(packed[:, shape.conv_dim + vh * 128 + vh:shape.conv_dim + vh * 128 + 2 * vh]).astype(np.float64)
         + orc.bf16_to_f32(dt_bias).astype(np.float64)[None, :])
    softplus = np.maximum(x, 0) + np.log1p(np.exp(-np.abs(x)))
    # bf16(a + dt_bias) and bf16(softplus) each move the exponent by up to half a bf16 step
    assert np.all(np.abs(decay[:rows] - decay64) <= decay64 * (1e-4 + np.abs(a_scale)[None, :] * (np.abs(x) + softplus) * 2.0 ** -8))
    # the state after the rows, through the next step's fold: 1e-4 relative to the state's scale (:531)
    _, state1, _, _ = orc.gdn_decode(shape, make_rows(rng, shape, 1), conv_w, a_scale, dt_bias, norm, conv_in, state_in,
                                     pending_tape=tape, pending_path=(1 << rows) - 1)
    # the fp64 reference ran on unrounded k, v and gates: bound by the rounding of those (bf16 inputs, 16 rows)
    assert np.abs(state1 - state64).max() <= 2e-2 * np.abs(state64).max()
    # hidden rows: gate the fp64 outputs the same way; a few bf16 steps, nearly all exact or one step
    z = orc.bf16_to_f32(packed[:, shape.conv_dim:shape.conv_dim + vh * 128]).astype(np.float64).reshape(rows, vh, 128)
    w = orc.bf16_to_f32(norm).astype(np.float64)
    normed = out64 / np.sqrt((out64 ** 2).mean(axis=2, keepdims=True) + 1e-6) * w
    want = orc.f32_to_bf16((normed * z / (1 + np.exp(-z))).astype(np.float32)).reshape(rows, vh * 128)
    # q, k and v enter the recurrence rounded to bf16 (2^-9 each), so an output carries a few bf16 steps of
    # its own size plus a cancellation term of its row's size (:590-598)
    got, ref = orc.bf16_to_f32(hidden).astype(np.float64), orc.bf16_to_f32(want).astype(np.float64)
    scale = np.abs(ref).reshape(rows, vh, 128).max(axis=2, keepdims=True).repeat(128, axis=2).reshape(rows, vh * 128)
    error = np.abs(got - ref)
    assert np.all(error <= 2.0 ** -5 * np.abs(ref) + 2.0 ** -6 * scale)
    assert (error <= 2.0 ** -7 * np.abs(ref) + 2.0 ** -9 * scale).mean() >= 0.9


def test_one_row_is_the_closed_form():
    """S' = d S + beta (v - d S k) k^T and o = S' q, in fp64 sums, from the tape's own k, v and gates."""
    rng = np.random.default_rng(4)
    shape, conv_w, a_scale, dt_bias, norm = make_layer(rng, 1, 2)
    packed = make_rows(rng, shape, 1)
    conv_in, state_in = make_state(rng, shape)
    _, _, tape, _ = orc.gdn_decode(shape, packed, conv_w, a_scale, dt_bias, norm, conv_in, state_in)
    _, kv, decay, beta = orc.gdn_split_tape(shape, tape)
    _, state1, _, _ = orc.gdn_decode(shape, make_rows(rng, shape, 2), conv_w, a_scale, dt_bias, norm, conv_in, state_in,
                                     pending_tape=tape, pending_path=1)
    for h in range(2):
        k = orc.bf16_to_f32(kv[0, :128]).astype(np.float64)
        v = orc.bf16_to_f32(kv[0, 128 + 128 * h:256 + 128 * h]).astype(np.float64)
        d, b = float(decay[0, h]), float(orc.bf16_to_f32(beta[0, h:h + 1])[0])
        S = state_in[h].astype(np.float64) * d
        want = S + b * np.outer(v - S @ k, k)
        assert np.abs(state1[h] - want).max() <= 1e-5 * np.abs(want).max()
        got, _ = orc.gdn_step(state_in[h], k, v, d, b)
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()


@pytest.mark.parametrize("accepted", [0, 1, 5, 16])
def test_fold_and_rollback(accepted):
    """The state a step writes holds exactly the accepted rows of the step before (a rejected suffix
    never reaches it), the fold of those rows alone is that state bit for bit, and the block's outputs
    are those of the same tokens run as one chain."""
    rng = np.random.default_rng(10 + accepted)
    shape, conv_w, a_scale, dt_bias, norm = make_layer(rng, 2, 4)
    conv_in, state_in = make_state(rng, shape)
    first = make_rows(rng, shape, 16)
    second = make_rows(rng, shape, 7)
    conv0, state0, tape0, hidden_first = orc.gdn_decode(shape, first, conv_w, a_scale, dt_bias, norm, conv_in, state_in)
    path = (1 << accepted) - 1
    conv1, state1, tape1, hidden1 = orc.gdn_decode(shape, second, conv_w, a_scale, dt_bias, norm, conv0, state0,
                                                   pending_tape=tape0 if accepted else None, pending_path=path)
    # the same tokens as one history: the accepted rows, then the second block
    if accepted:
        rc, conv_f, state_f = orc.gdn_fold(shape, conv0, state0, tape0, path, accepted)
        assert rc == 0
        assert np.array_equal(conv_f, conv1) and state_f.tobytes() == state1.tobytes()
        # a step of only the accepted rows, wholly accepted, leaves the same state: rejection costs nothing
        convA, stateA, tapeA, hiddenA = orc.gdn_decode(shape, first[:accepted], conv_w, a_scale, dt_bias, norm, conv_in, state_in)
        assert np.array_equal(hiddenA, hidden_first[:accepted])
        convB, stateB, _, hiddenB = orc.gdn_decode(shape, second, conv_w, a_scale, dt_bias, norm, convA, stateA,
                                                   pending_tape=tapeA, pending_path=path)
        assert np.array_equal(convB, conv1) and stateB.tobytes() == state1.tobytes() and np.array_equal(hiddenB, hidden1)
        if accepted + 7 <= 16:
            # and one chain of accepted + 7 rows gives the second block's outputs bit for bit
            _, _, _, hidden_chain = orc.gdn_decode(shape, np.concatenate([first[:accepted], second]), conv_w, a_scale, dt_bias, norm,
                                                   conv_in, state_in)
            assert np.array_equal(hidden_chain[accepted:], hidden1)
        rc, _, _ = orc.gdn_fold(shape, conv0, state0, tape0, path, accepted + 1)
        assert rc == 1                                   # a path shorter than the rows asked for folds nothing
    else:
        assert np.array_equal(conv1, conv_in) and state1.tobytes() == state_in.tobytes()


def test_tree_rows_are_the_chains_of_their_paths():
    """A tree block (gdn.metal:417-478): every row's tape entries are bit for bit those of its path run as a chain
    (the convolution follows the path), its output is the chain's up to the fp32 reordering of the path form
    S_-1 z_-1 + sum c_j v_j, and within the fp64 recurrence's bounds along the path; a tree whose rows happen to
    be a chain is the chain bit for bit; the state the step writes does not depend on the tree."""
    rng = np.random.default_rng(31)
    shape, conv_w, a_scale, dt_bias, norm = make_layer(rng, 2, 4)
    rows, vh = 12, shape.value_heads
    packed = make_rows(rng, shape, rows)
    conv_in, state_in = make_state(rng, shape)
    previous = make_rows(rng, shape, 5)
    conv0, state0, tape0, _ = orc.gdn_decode(shape, previous, conv_w, a_scale, dt_bias, norm, conv_in, state_in)
    pending = 0b10011      # rows 0, 1, 4 of the previous step were accepted
    args = (conv_w, a_scale, dt_bias, norm, conv0, state0)
    chain = orc.gdn_decode(shape, packed, *args, pending_tape=tape0, pending_path=pending)
    as_tree = orc.gdn_decode(shape, packed, *args, pending_tape=tape0, pending_path=pending,
                             ancestors=[(2 << r) - 1 for r in range(rows)])
    for a, b in zip(chain, as_tree):
        assert np.array_equal(a, b)
    masks = make_tree(rng, rows)
    assert any(int(m) != (2 << r) - 1 for r, m in enumerate(masks))
    conv1, state1, tape1, hidden = orc.gdn_decode(shape, packed, *args, pending_tape=tape0, pending_path=pending, ancestors=masks)
    assert np.array_equal(conv1, chain[0]) and state1.tobytes() == chain[1].tobytes()
    inputs, kv, decay, beta = orc.gdn_split_tape(shape, tape1)
    assert np.array_equal(inputs[:rows], packed[:, :shape.conv_dim])
    # the fp64 check starts from the state after the pending rows (state1) and the convolution carry they leave
    for r in range(rows):
        path = path_rows(masks[r])
        along = packed[path]
        _, _, tape_c, hidden_c = orc.gdn_decode(shape, along, *args, pending_tape=tape0, pending_path=pending)
        ci, ckv, cdecay, cbeta = orc.gdn_split_tape(shape, tape_c)
        last = len(path) - 1
        assert np.array_equal(kv[r], ckv[last]) and np.array_equal(beta[r], cbeta[last]) and np.array_equal(decay[r], cdecay[last])
        got = orc.bf16_to_f32(hidden[r]).astype(np.float64)
        want = orc.bf16_to_f32(hidden_c[last]).astype(np.float64)
        scale = np.abs(want).reshape(vh, 128).max(axis=1, keepdims=True).repeat(128, axis=1).reshape(-1)
        # the two forms round differently before the output norm: a bf16 step of the value, a fraction of one of the row
        assert np.all(np.abs(got - want) <= 2.0 ** -6 * np.abs(want) + 2.0 ** -8 * scale), (r, np.abs(got - want).max())
        assert (ulps(hidden[r], hidden_c[last]) <= 1).mean() >= 0.95
        kv64, beta64, decay64, state64, out64 = orc.gdn_reference(shape, along, conv_w, a_scale, dt_bias, conv1, state1)
        z = orc.bf16_to_f32(packed[r, shape.conv_dim:shape.conv_dim + vh * 128]).astype(np.float64).reshape(vh, 128)
        w = orc.bf16_to_f32(norm).astype(np.float64)
        o = out64[last]
        normed = o / np.sqrt((o ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
        ref = orc.bf16_to_f32(orc.f32_to_bf16((normed * z / (1 + np.exp(-z))).astype(np.float32))).astype(np.float64).reshape(-1)
        rscale = np.abs(ref).reshape(vh, 128).max(axis=1, keepdims=True).repeat(128, axis=1).reshape(-1)
        assert np.all(np.abs(got - ref) <= 2.0 ** -5 * np.abs(ref) + 2.0 ** -6 * rscale)


def test_a_tree_path_folds_like_its_chain():
    """Accepting a path of a tree step: the next step's state is bit for bit the state after the path's rows run
    as a chain, and the fold of the path alone is that state."""
    rng = np.random.default_rng(32)
    shape, conv_w, a_scale, dt_bias, norm = make_layer(rng, 1, 2)
    rows = 9
    packed = make_rows(rng, shape, rows)
    conv_in, state_in = make_state(rng, shape)
    masks = make_tree(rng, rows)
    leaf = max(range(rows), key=lambda r: bin(int(masks[r])).count("1"))
    path = int(masks[leaf])
    args = (conv_w, a_scale, dt_bias, norm)
    conv0, state0, tape0, _ = orc.gdn_decode(shape, packed, *args, conv_in, state_in, ancestors=masks)
    nxt = make_rows(rng, shape, 3)
    conv1, state1, _, hidden1 = orc.gdn_decode(shape, nxt, *args, conv0, state0, pending_tape=tape0, pending_path=path)
    along = packed[path_rows(path)]
    convc, statec, tapec, _ = orc.gdn_decode(shape, along, *args, conv_in, state_in)
    conv2, state2, _, hidden2 = orc.gdn_decode(shape, nxt, *args, convc, statec, pending_tape=tapec, pending_path=(1 << len(along)) - 1)
    assert np.array_equal(conv1, conv2) and state1.tobytes() == state2.tobytes() and np.array_equal(hidden1, hidden2)
    rc, convf, statef = orc.gdn_fold(shape, conv0, state0, tape0, path, len(along))
    assert rc == 0 and np.array_equal(convf, conv1) and statef.tobytes() == state1.tobytes()


def _prefill_case(seed, heads, tokens, float_norm=False):
    rng = np.random.default_rng(seed)
    shape, conv_w, a_scale, dt_bias, norm = make_layer(rng, *heads, float_norm=float_norm)
    packed = make_rows(rng, shape, tokens)
    conv_in, state_in = make_state(rng, shape)
    return shape, conv_w, a_scale, dt_bias, norm, packed, conv_in, state_in


@pytest.mark.parametrize("heads,tokens,float_norm", [((2, 4), 40, False), ((1, 2), 1, True), ((2, 2), 19, False)])
def test_prefill_matches_the_fp64_checks_of_the_reference(heads, tokens, float_norm):
    case = _prefill_case(31, heads, tokens, float_norm)
    shape, conv_w, a_scale, dt_bias, norm, packed, conv_in, state_in = case
    got = orc.gdn_prefill(shape, packed, conv_w, a_scale, dt_bias, norm, conv_in, state_in)
    check_prefill_against_fp64(*case, got)


def test_prefill_leaves_the_state_of_the_same_rows_as_accepted_blocks():
    """A chunk's k, v and gates are the tape's, and its cell is, bit for bit, the one the rows leave when they enter as
    verify blocks that are accepted whole (a decode step per block, the next step's fold after it)."""
    shape, conv_w, a_scale, dt_bias, norm, packed, conv_in, state_in = _prefill_case(32, (2, 4), 40)
    got = orc.gdn_prefill(shape, packed, conv_w, a_scale, dt_bias, norm, conv_in, state_in)
    conv, state, tape, path = conv_in, state_in, None, 0
    kw = shape.key_heads * 128
    for first, rows in ((0, 16), (16, 16), (32, 8)):
        conv, state, tape, _ = orc.gdn_decode(shape, packed[first:first + rows], conv_w, a_scale, dt_bias, norm, conv, state,
                                              pending_tape=tape, pending_path=path)
        path = (1 << rows) - 1
        _, kv, decay, beta = orc.gdn_split_tape(shape, tape)
        assert np.array_equal(kv[:rows, :kw], got["keys"][first:first + rows])
        assert np.array_equal(kv[:rows, kw:], got["values"][first:first + rows])
        assert decay[:rows].tobytes() == got["decay"][first:first + rows].tobytes()
        assert np.array_equal(beta[:rows], got["beta"][first:first + rows])
    rc, conv, state = orc.gdn_fold(shape, conv, state, tape, path, 8)
    assert rc == 0
    assert np.array_equal(conv, got["conv_out"]) and state.tobytes() == got["state_out"].tobytes()


def test_prefill_in_two_runs_is_the_chunk():
    """gdn_metal_test.mm:426-480: a chunk continued from the cell its first rows left equals the chunk run whole."""
    shape, conv_w, a_scale, dt_bias, norm, packed, conv_in, state_in = _prefill_case(33, (2, 4), 37)
    whole = orc.gdn_prefill(shape, packed, conv_w, a_scale, dt_bias, norm, conv_in, state_in)
    first = orc.gdn_prefill(shape, packed[:21], conv_w, a_scale, dt_bias, norm, conv_in, state_in)
    second = orc.gdn_prefill(shape, packed[21:], conv_w, a_scale, dt_bias, norm, first["conv_out"], first["state_out"])
    for name in ("queries", "keys", "values", "beta", "recurrent", "hidden"):
        assert np.array_equal(np.concatenate([first[name], second[name]]), whole[name]), name
    assert np.concatenate([first["decay"], second["decay"]]).tobytes() == whole["decay"].tobytes()
    assert np.array_equal(second["conv_out"], whole["conv_out"]) and second["state_out"].tobytes() == whole["state_out"].tobytes()
