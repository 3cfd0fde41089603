"""End-to-end parity of the hybrid mixture-of-experts verify step (BASELINE.json config 5 at a small shape: three Gated
DeltaNet layers and one attention layer, 16 experts top-2) against the oracle, through the C ABI: every layer
teacher-forced from the GPU's own layer input, the step's parts bitwise the whole step, greedy acceptance exact,
and the state rollback across two steps of two lanes (the accepted path of the first step is what the second folds)."""
import numpy as np
import pytest

import splash_amd

from splash_amd import ops, verify
from tests import oracle as orc
from tests.gdn_case import ulps
from tests.hybrid_reference import HybridModel
from tests.test_verify_step_gpu import close_bf16

pytestmark = pytest.mark.gpu

SHAPE = dict(hidden=256, vocabulary=1024, layers=4, q_heads=8, kv_heads=2, head_dim=128, gdn_key_heads=2, gdn_value_heads=4,
             experts=16, top_k=2, expert_ffn=256)


def sure_routes(scores, top_k):
    """Rows whose k-th and (k + 1)-th scores are far enough apart that a last-bit difference cannot reroute them."""
    ordered = -np.sort(-scores, axis=1)
    return (ordered[:, top_k - 1] - ordered[:, top_k]) > 1e-3 * np.abs(scores).max()


def check_step(backend, model, gpu, lanes, tokens, checked_layers=None, deep=False):
    """Runs the step whole, then part by part, each layer (or each of `checked_layers`) against the oracle from the GPU's
    own input rows, cells and tapes. Returns the step's results."""
    d = model.dims
    H, V = d["hidden"], d["vocabulary"]
    rows = sum(l.rows for l in lanes)
    gpu.set_block(lanes, tokens)
    backend.run(gpu.encode(lanes, commit=True))
    whole_logits = gpu.buffer(verify.LOGITS).download(np.float32, rows * V).reshape(rows, V)
    results = gpu.results(lanes)
    hidden_of = lambda i=0: gpu.buffer(verify.HIDDEN, i).download(np.uint16, rows * H).reshape(rows, H)
    backend.run(gpu.encode_part(0, 0, lanes))
    assert np.array_equal(hidden_of(), model.oracle_embedding(tokens))
    for layer in range(d["layers"]):
        if checked_layers is not None and layer not in checked_layers:
            backend.run(gpu.encode_part(1, layer, lanes))
            continue
        print(f"  layer {layer} ({'attention' if model.attends(layer) else 'GDN'})", flush=True)
        before = hidden_of()
        g = gpu.mixer_index(layer)
        if not model.attends(layer):
            cells = [model.read_cell(i, l.parity, g) for i, l in enumerate(lanes)]
            tapes = [model.read_tape(i, l.parity ^ 1, g) for i, l in enumerate(lanes)]
        backend.run(gpu.encode_part(1, layer, lanes))
        packed = model.oracle_mixer_input(before, layer)
        if model.attends(layer):
            mixed = model.oracle_attention(packed, layer, lanes)
        else:
            mixed, left = model.oracle_gdn(packed, layer, lanes, cells, tapes)
            for i, l in enumerate(lanes):
                conv, state = model.read_cell(i, l.parity ^ 1, g)
                assert np.array_equal(conv, left[i][0]), (layer, i)
                assert np.abs(state - left[i][1]).max() <= 1e-4 * np.abs(left[i][1]).max(), (layer, i)
        hidden1 = model.oracle_mixer_output(mixed, before, layer)
        ok, detail = close_bf16(hidden_of(1), hidden1)
        assert ok, ("mixer", layer, detail)
        # the FFN from the GPU's own mixer output
        scores, want = model.oracle_ffn(hidden_of(1), layer)
        sure = sure_routes(scores, d["top_k"]) if scores is not None else np.ones(rows, dtype=bool)   # a dense FFN routes nothing
        # with eight of 128 experts a row's eighth and ninth scores are close more often than with two of sixteen
        assert sure.mean() >= (0.9 if d["experts"] <= 16 else 0.75)
        ok, detail = close_bf16(hidden_of()[sure], want[sure])
        assert ok, ("ffn", layer, detail)
    final = hidden_of()
    backend.run(gpu.encode_part(2, 0, lanes))
    logits = gpu.buffer(verify.LOGITS).download(np.float32, rows * V).reshape(rows, V)
    # A part starts with a norm pass over its input rows; inside the whole step the combine before it wrote that
    # table without the rows' inverse RMS, which the reading projection applies to its sums: one bf16 operand
    # rounding apart at every layer, so the two chains agree as two bf16 pipelines do, not bit for bit.
    part_cos = (logits.astype(np.float64) * whole_logits).sum() / np.sqrt((logits.astype(np.float64) ** 2).sum() * (whole_logits.astype(np.float64) ** 2).sum())
    row_gap = np.abs(logits - whole_logits).max(axis=1)
    print("parts against the whole step: cosine", part_cos, "largest difference by row", np.round(row_gap, 4), flush=True)
    # (`deep`: over tens of layers that one rounding a layer is carried on and grows: cosine >= 0.998, as two runs of any
    # bf16 pipeline of that depth agree)
    if deep:
        assert part_cos >= 0.998, part_cos
    else:
        assert part_cos >= 0.9995 and np.median(row_gap) <= 2e-2 and row_gap.max() <= 1e-1, (part_cos, row_gap)
    want_logits = model.oracle_head(final)
    cos = (logits.astype(np.float64) * want_logits).sum() / np.sqrt((logits.astype(np.float64) ** 2).sum() * (want_logits ** 2).sum())
    assert cos >= 0.9999 and np.abs(logits - want_logits).max() <= 2e-2, (cos, np.abs(logits - want_logits).max())
    # greedy acceptance of the whole step's own logits, lane by lane, is exact
    selected, retained, accepted, masks = results
    first = 0
    for i, l in enumerate(lanes):
        picks = np.array([orc.argmax(whole_logits[first + r]) for r in range(l.rows)], dtype=np.uint32)
        kept, acc, mask = orc.accept_tree(ops.chain_tree_rows([l.rows]), tokens[first:first + l.rows], picks)
        assert retained[i] == len(kept) and accepted[i] == acc and masks[i] == mask
        assert np.array_equal(selected[first:first + len(kept)], kept)
        first += l.rows
    return logits, results


def test_config5_two_steps_with_rollback(backend):
    print("case config 5 hybrid two steps", flush=True)
    model = HybridModel(seed=41, **SHAPE)
    gpu = model.build_gpu(backend, max_lanes=2, pages_per_lane=2)
    rng = np.random.default_rng(5)
    model.seed_context(rng)
    model.seed_states(rng, lanes=2)
    V = SHAPE["vocabulary"]
    committed = [70, 300]
    rows = [6, 16]
    lanes = [verify.HybridLane(rows[i], committed[i], table_first=i * model.pages_per_lane) for i in range(2)]
    # lane 0's draft continues the target's own choices for three rows and then departs; lane 1's is random
    tokens = rng.integers(0, V, sum(rows)).astype(np.uint32)
    for r in range(1, 4):
        gpu.set_block(lanes, tokens)
        backend.run(gpu.encode(lanes, commit=False))
        tokens[r] = gpu.buffer(verify.LOGITS).download(np.float32, sum(rows) * V).reshape(-1, V)[r - 1].argmax()
    logits, (selected, retained, accepted, masks) = check_step(backend, model, gpu, lanes, tokens)
    assert accepted[0] >= 3 and masks[0] & 0b1111 == 0b1111 and retained[1] >= 1 and masks[1] & 1
    # what the step left: each GDN layer's tape of parity 0 and the cell of parity 1 (the state BEFORE the block)
    before = [[model.read_cell(i, 1, g) for g in range(gpu.gdn_layers)] for i in range(2)]
    # second step: every lane folds the path it retained, at the other parity, after its kept tokens
    lanes2 = [verify.HybridLane(rows2, committed[i] + int(retained[i]), table_first=i * model.pages_per_lane, pending_path=int(masks[i]), parity=1)
              for i, rows2 in enumerate((16, 3))]
    tokens2 = rng.integers(0, V, 19).astype(np.uint32)
    check_step(backend, model, gpu, lanes2, tokens2)
    # the cell the second step wrote holds exactly the accepted rows of the first: the fold of the first step's
    # tape along the retained path, bit for bit (identical arithmetic), and nothing of the rejected rows
    for i in range(2):
        count = bin(int(masks[i])).count("1")
        for g in range(gpu.gdn_layers):
            rc, conv, state = orc.gdn_fold(model.gdn_shape, before[i][g][0], before[i][g][1], model.read_tape(i, 0, g), int(masks[i]), count)
            got_conv, got_state = model.read_cell(i, 0, g)
            assert rc == 0 and np.array_equal(conv, got_conv) and state.tobytes() == got_state.tobytes(), (i, g)


@pytest.mark.parametrize("gated", [False, True])
def test_config5_more_rows_than_one_projection_takes(backend, gated):
    """Five lanes of sixteen rows: the dense projections run in pieces of at most 64 rows, the mixers, the routed
    experts and the acceptance over all 80 at once. Gated: the attention layer's rows carry output gates, as the
    reference's Qwen3.5 attention layers do."""
    print(f"case config 5 hybrid 80 rows gated={gated}", flush=True)
    model = HybridModel(seed=42, gated_attention=gated, **SHAPE)
    gpu = model.build_gpu(backend, max_lanes=5, pages_per_lane=1)
    rng = np.random.default_rng(6)
    model.seed_context(rng)
    model.seed_states(rng, lanes=5)
    lanes = [verify.HybridLane(16, 20 + 30 * i, table_first=i) for i in range(5)]
    check_step(backend, model, gpu, lanes, rng.integers(0, SHAPE["vocabulary"], 80).astype(np.uint32))


@pytest.mark.parametrize("gate", [True, False])
def test_config5_with_a_shared_expert(backend, gate):
    """The reference's Qwen3.5 MoE blocks add a shared expert every row visits (MoE.hpp:50-63), gated by the sigmoid of
    the row's product with the block's scalar gate: two lanes, layer by layer against the oracle."""
    print(f"case config 5 hybrid shared expert gate={gate}", flush=True)
    model = HybridModel(seed=43, shared_slices=1, shared_gate=gate, **SHAPE)
    gpu = model.build_gpu(backend, max_lanes=2, pages_per_lane=1)
    rng = np.random.default_rng(8)
    model.seed_context(rng)
    model.seed_states(rng, lanes=2)
    lanes = [verify.HybridLane(16, 40, table_first=0), verify.HybridLane(9, 100, table_first=1)]
    check_step(backend, model, gpu, lanes, rng.integers(0, SHAPE["vocabulary"], 25).astype(np.uint32))


def test_dense_ffn_under_the_hybrid_mixers(backend):
    """The reference's dense Qwen3.5 targets run the same Gated DeltaNet and attention mixers over a dense SwiGLU
    (QwenTarget.cpp:351-370) instead of a mixture of experts: experts 0 and a dense FFN width, layer by layer against
    the oracle, two lanes, and a second step that folds what the first accepted."""
    print("case hybrid dense FFN", flush=True)
    shape = {**SHAPE, "experts": 0, "top_k": 0, "expert_ffn": 0}
    model = HybridModel(seed=44, dense_ffn=768, **shape)
    gpu = model.build_gpu(backend, max_lanes=2, pages_per_lane=1)
    rng = np.random.default_rng(12)
    model.seed_context(rng)
    model.seed_states(rng, lanes=2)
    lanes = [verify.HybridLane(16, 33, table_first=0), verify.HybridLane(7, 90, table_first=1)]
    _, (selected, retained, accepted, masks) = check_step(backend, model, gpu, lanes, rng.integers(0, SHAPE["vocabulary"], 23).astype(np.uint32))
    following = [verify.HybridLane(16, 33 + int(retained[0]), table_first=0, pending_path=int(masks[0]), parity=1),
                 verify.HybridLane(7, 90 + int(retained[1]), table_first=1, pending_path=int(masks[1]), parity=1)]
    check_step(backend, model, gpu, following, rng.integers(0, SHAPE["vocabulary"], 23).astype(np.uint32))


def test_hidden_rows_are_captured_for_a_draft(backend):
    """After the layers a draft reads, every row's output lies in its slot of the capture buffer: the rows the same layers
    leave when the step runs part by part from the same cells and tapes."""
    print("case hybrid capture", flush=True)
    model = HybridModel(seed=43, **SHAPE)
    gpu = model.build_gpu(backend, max_lanes=2, pages_per_lane=2)
    rng = np.random.default_rng(6)
    model.seed_context(rng)
    model.seed_states(rng, lanes=2)
    H, layers = SHAPE["hidden"], SHAPE["layers"]
    lanes = [verify.HybridLane(5, 40, table_first=0), verify.HybridLane(16, 200, table_first=model.pages_per_lane)]
    rows = 21
    captured = backend.allocate_buffer(2 * 16 * 2 * H * 2)
    picked = [1, layers - 1]
    gpu.set_capture(picked, captured)
    gpu.set_block(lanes, rng.integers(0, SHAPE["vocabulary"], rows).astype(np.uint32))
    backend.run(gpu.encode(lanes, commit=False))
    got = captured.download(np.uint16)[:rows * 2 * H].reshape(rows, 2, H).copy()
    hidden_of = lambda: gpu.buffer(verify.HIDDEN, 0).download(np.uint16, rows * H).reshape(rows, H)
    assert np.array_equal(got[:, 1], hidden_of())          # the last layer's rows are what the step left
    alone = backend.allocate_buffer(2 * 16 * H * 2)
    gpu.set_capture([1], alone)
    backend.run(gpu.encode(lanes, commit=False))
    assert np.array_equal(got[:, 0], alone.download(np.uint16)[:rows * H].reshape(rows, H))
    # part by part a layer's norm is a pass of its own, where the whole step defers it into the projections: the same
    # rows to that rounding
    backend.run(gpu.encode_part(0, 0, lanes))
    for layer in range(2):
        backend.run(gpu.encode_part(1, layer, lanes))
    ok, detail = close_bf16(got[:, 0], hidden_of())
    assert ok, detail
    with pytest.raises(splash_amd.SplashError):
        gpu.set_capture([2, 1], captured)                 # ascending
    with pytest.raises(splash_amd.SplashError):
        gpu.set_capture([0, 1, 2], captured)              # a destination too small for three layers' rows


def test_a_penalized_lane_of_a_hybrid_step(backend):
    """The sampling penalties through the hybrid driver, as through the dense one: the penalized lane's rows of the
    step's logits are the oracle's penalties of the rows the same step leaves without them, its selections their argmax;
    the other lane is untouched; a committing step counts what the lane keeps."""
    print("case hybrid penalized lane", flush=True)
    from splash_amd import ops
    model = HybridModel(seed=47, **SHAPE)
    gpu = model.build_gpu(backend, max_lanes=2, pages_per_lane=2)
    rng = np.random.default_rng(9)
    model.seed_context(rng)
    model.seed_states(rng, lanes=2)
    V = SHAPE["vocabulary"]
    make_lanes = lambda: [verify.HybridLane(7, 40, table_first=0), verify.HybridLane(12, 200, table_first=model.pages_per_lane)]
    lanes, rows = make_lanes(), 19
    tokens = rng.integers(0, V, rows).astype(np.uint32)
    tokens[3] = tokens[2]
    tree = ops.chain_tree_rows([7, 12])
    logits_of = lambda: gpu.buffer(verify.LOGITS).download(np.float32, rows * V).reshape(rows, V)
    gpu.set_block(lanes, tokens)
    backend.run(gpu.encode(lanes, commit=False))
    plain = logits_of()
    favourites = np.argmax(plain[:7], axis=1).astype(np.uint32)
    words = ops.Sampling.rebuild_penalty_words(V, np.concatenate([favourites, favourites[:3]]), 3, pending_token=int(tokens[0]))
    table = gpu.buffer(verify.PENALTY_WORDS)
    table.upload(words)                                          # lane 0's row
    penalties = (1.3, 2.0, 0.5)
    gpu.set_penalties(0, *penalties)
    lanes = make_lanes()
    gpu.set_block(lanes, tokens)
    graph = gpu.encode(lanes, commit=True)
    assert "decode_sample_penalize" in graph.kernels() and "decode_sample_count_tokens" in graph.kernels()
    backend.run(graph)
    seen = logits_of()
    got_tokens, got_retained, _, _ = (np.array(a).copy() for a in gpu.results(lanes))
    want = orc.penalize(plain[:7], words, tokens[:7], tree["ancestors"][:7], *penalties)
    assert seen[:7].tobytes() == want.tobytes() and seen[7:].tobytes() == plain[7:].tobytes()
    selected = np.array([orc.argmax(row) for row in want], np.uint32)
    assert np.any(selected != favourites)
    kept, _, _ = orc.accept_tree(tree[:7], tokens[:7], selected)
    assert got_retained[0] == len(kept) and np.array_equal(got_tokens[:len(kept)], kept)
    want_words = words.copy()
    np.add.at(want_words, kept, 1)
    counted = table.download(np.uint32, 2 * V).reshape(2, V)
    assert np.array_equal(counted[0], want_words) and not counted[1].any()


def test_hybrid_rejects_bad_arguments(backend):
    with pytest.raises(ValueError):
        verify.HybridVerify(backend, **{**SHAPE, "layers": 5})            # not whole groups of four layers
    with pytest.raises(ValueError):
        verify.HybridVerify(backend, **{**SHAPE, "experts": 12})          # the router writes whole column tiles
    with pytest.raises(ValueError):
        verify.HybridVerify(backend, **SHAPE, max_lanes=9)
    gpu = verify.HybridVerify(backend, **SHAPE, max_lanes=1)
    with pytest.raises(ValueError):
        gpu.encode([verify.HybridLane(4, 0), verify.HybridLane(4, 0)])    # more lanes than it was built for


@pytest.mark.parametrize("tokens,file_form", [(100, False), (300, True)])
def test_a_prompt_chunk_through_the_hybrid_layers(backend, tmp_path, tokens, file_form):
    """HybridVerify.encode_prefill: a prompt chunk of one lane, every layer against the oracle from the GPU's own layer
    input -- an attention layer's rows from the history and the chunk's rows up to each (tile by tile as blocks of the
    sequence), a Gated DeltaNet layer's rows and the cell it leaves from orc_gdn_prefill -- and then a verify step of the
    lane from the cell and the pages the chunk left (the other parity, nothing pending), checked as any step is."""
    from tests.hybrid_reference import hybrid_model_file
    print(f"case hybrid prompt chunk tokens={tokens} file_form={file_form}", flush=True)
    model = HybridModel(seed=47, **SHAPE, shared_slices=1, shared_gate=True, gated_attention=file_form, file_form=file_form)
    if file_form:
        gpu = model.build_gpu_from_file(backend, hybrid_model_file(tmp_path / "m.gguf", model), max_lanes=1, pages_per_lane=3, prefill_rows=320)
    else:
        gpu = model.build_gpu(backend, max_lanes=1, pages_per_lane=3, prefill_rows=128)
    rng = np.random.default_rng(12)
    model.seed_context(rng)
    model.seed_states(rng, lanes=1)
    d = model.dims
    H, V, committed = d["hidden"], d["vocabulary"], 200
    prompt = rng.integers(0, V, tokens).astype(np.uint32)
    gpu.set_prefill_block(prompt)
    hidden_of = lambda i=0: gpu.buffer(verify.HIDDEN, i).download(np.uint16, tokens * H).reshape(tokens, H)
    before = model.oracle_embedding(prompt)
    for layer in range(d["layers"]):
        print(f"  layer {layer} ({'attention' if model.attends(layer) else 'GDN'})", flush=True)
        g = gpu.mixer_index(layer)
        if layer:
            before = hidden_of()
        if not model.attends(layer):
            conv_in, state_in = model.read_cell(0, 0, g)
        backend.run(gpu.encode_prefill(0, 0, committed, tokens, parity=0, first_layer=layer, layer_count=1))
        packed = model.oracle_mixer_input(before, layer)
        if model.attends(layer):
            mixed = model.oracle_attention_chunk(packed, layer, 0, committed)
        else:
            w = model.layers[layer]
            want = orc.gdn_prefill(model.gdn_shape, packed, w["conv_w"], w["a_scale"], w["dt_bias"], w["mixer_norm"], conv_in, state_in)
            mixed = want["hidden"]
            conv, state = model.read_cell(0, 1, g)
            # the carry is the chunk's last packed rows, which the GPU's projection and the oracle's exact sums round apart
            # now and then
            ok, detail = close_bf16(conv, want["conv_out"])
            assert ok and (ulps(conv, want["conv_out"]) > 0).mean() < 0.01, (layer, detail)
            assert np.abs(state - want["state_out"]).max() <= 2e-3 * np.abs(want["state_out"]).max(), layer
        ok, detail = close_bf16(hidden_of(1), model.oracle_mixer_output(mixed, before, layer))
        assert ok, ("mixer", layer, detail)
        scores, want = model.oracle_ffn(hidden_of(1), layer)
        sure = sure_routes(scores, d["top_k"])
        assert sure.mean() >= 0.9
        ok, detail = close_bf16(hidden_of()[sure], want[sure])
        assert ok, ("ffn", layer, detail)
    if layer == 0:
        assert np.array_equal(before, model.oracle_embedding(prompt))
    # the chunk in one graph leaves the same pages, cells and rows as its layers one by one
    pools = lambda: np.concatenate([gpu.buffer(verify.KV_POOL, a).download(np.uint8) for a in range(d["layers"] // d["attention_interval"])])
    cells = lambda: gpu.buffer(verify.GDN_STATES).download(np.uint8).copy()
    want_pools, want_cells, want_hidden = pools(), cells(), hidden_of().copy()
    backend.run(gpu.encode_prefill(0, 0, committed, tokens, parity=0))
    assert np.array_equal(pools(), want_pools) and np.array_equal(cells(), want_cells) and np.array_equal(hidden_of(), want_hidden)
    # a verify step of the lane after the chunk
    lanes = [verify.HybridLane(7, committed + tokens, table_first=0, pending_path=0, parity=1)]
    check_step(backend, model, gpu, lanes, rng.integers(0, V, 7).astype(np.uint32))
    with pytest.raises(ValueError):
        gpu.encode_prefill(0, 0, committed, 321 if file_form else 129)
