"""GPU parity of the draft selector's tree growth (draft_select_tree) against the oracle, through the C ABI."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc
from tests.draft_tree_statement import tree as stated_tree
from tests.test_oracle_draft_tree import compare, drawn_lattice

pytestmark = pytest.mark.gpu


def grow(backend, lattices, lanes, chains=None, rates=None):
    """The trees of `lanes` (dicts) over their lattices, as a list of dicts like orc.draft_tree's."""
    n = len(lanes)
    candidates = np.concatenate([l[0] for l in lattices]).astype(np.uint32)
    unary = np.concatenate([l[1] for l in lattices]).astype(np.float32)
    edges = np.concatenate([l[2] for l in lattices]).astype(np.float32)
    chains = np.zeros((n, 15), np.uint32) if chains is None else np.ascontiguousarray(chains, np.uint32)
    rates = np.zeros((n, 15, 4), np.float32) if rates is None else np.ascontiguousarray(rates, np.float32)
    up = backend.from_array
    out = dict(tokens=backend.allocate_buffer(n * 16 * 4), trees=backend.allocate_buffer(n * 16 * 8), scores=backend.allocate_buffer(n * 16 * 8),
               sizes=backend.allocate_buffer(max(n * 4, 16)), draws=backend.allocate_buffer(n * 16 * 4), next=backend.allocate_buffer(n * 16 * 16 * 4),
               caps=backend.allocate_buffer(n * 16 * 4))
    for buffer in out.values():
        buffer.fill(0xEE)
    graph = splash_amd.CommandGraph()
    ops.DraftSelector.add_tree(graph, up(candidates), up(unary), up(edges), up(chains), up(rates), out["tokens"], out["trees"], out["scores"],
                               out["sizes"], out["draws"], out["next"], out["caps"], lanes)
    backend.run(graph)
    sizes = out["sizes"].download(np.uint32)[:n]
    tokens = out["tokens"].download(np.uint32).reshape(n, 16)
    trees = out["trees"].download(np.uint8).view(orc.TREE_DTYPE).reshape(n, 16)
    scores = out["scores"].download(np.float32).reshape(n, 16, 2)
    draws = out["draws"].download(np.uint8).reshape(n, 16, 4)
    nxt = out["next"].download(np.float32).reshape(n, 16, 16)
    caps = out["caps"].download(np.float32).reshape(n, 16)
    return [dict(tokens=tokens[l, :s], tree=trees[l, :s], q=scores[l, :s, 0], estimate=scores[l, :s, 1], draws=draws[l, :s], next=nxt[l, :s],
                 caps=caps[l, :s]) for l, s in enumerate(sizes)]


def oracle_lane(lane):
    return orc.draft_tree_lane(anchor=lane["anchor"], depth=lane["depth"], children=lane["children"], slope=lane.get("slope", 1.0),
                               intercept=lane.get("intercept"), temperature=lane.get("temperature", 0.0), noise=lane.get("noise", 0),
                               chain=lane.get("chain", 0))


def same_tree(got, want):
    """The oracle's own outputs against the GPU's: the structure exactly, floats to the rounding of exp and log."""
    assert len(got["tokens"]) == len(want["tokens"])
    assert np.array_equal(got["tokens"], want["tokens"]) and np.array_equal(got["tree"], want["tree"])
    assert np.array_equal(got["draws"], want["draws"])
    assert np.allclose(got["q"], want["q"], rtol=1e-4, atol=1e-7) and np.allclose(got["estimate"], want["estimate"], rtol=1e-4)
    assert np.allclose(got["caps"], want["caps"], atol=1e-5) and np.allclose(got["next"], want["next"], rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("temperature", [0.0, 0.7, 1.3])
def test_trees_match_the_oracle_and_its_independent_statement(backend, temperature):
    """Batches of up to eight lanes with children 1 to 4 and depths 0 to 15: wherever the independent statement says the
    order of the tree's rows hangs on more than one part in 10^4 (the rounding of exp and log decides nothing), the GPU's
    tree is the oracle's row for row, and both are the statement's."""
    print(f"case draft tree temperature={temperature}", flush=True)
    rng = np.random.default_rng(int(temperature * 10) + 1)
    compared = 0
    for batch in range(12):
        n = int(rng.integers(1, 9))
        lattices = [drawn_lattice(rng) for _ in range(n)]
        lanes = [dict(anchor=int(rng.integers(1000)), depth=int(rng.integers(0, 16)), children=int(rng.integers(1, 5)),
                      slope=float(rng.uniform(0.6, 1.4)), intercept=[float(v) for v in rng.normal(0.5, 0.5, 7)], temperature=temperature,
                      noise=int(rng.integers(1 << 62))) for _ in range(n)]
        trees = grow(backend, lattices, lanes)
        for lattice, lane, got in zip(lattices, lanes, trees):
            want = stated_tree(*lattice, oracle_lane(lane))
            if want is None:
                continue
            compare(got, want)
            same_tree(got, orc.draft_tree(*lattice, oracle_lane(lane)))
            compared += 1
    assert compared >= 30


@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_host_chains_share_the_trees(backend, temperature):
    print(f"case draft tree with host chains temperature={temperature}", flush=True)
    rng = np.random.default_rng(40 + int(temperature * 10))
    compared = 0
    for batch in range(10):
        n = int(rng.integers(1, 9))
        lattices = [drawn_lattice(rng) for _ in range(n)]
        chains = np.zeros((n, 15), np.uint32)
        for l in range(n):
            for d in range(15):
                kind = rng.integers(3)
                c = lattices[l][0]
                chains[l, d] = c[d][0] if d < 7 and kind == 0 else c[d][rng.integers(1, 16)] if d < 7 and kind == 1 else 9000 + d
        rates = rng.uniform(0.2, 0.95, (n, 15, 4)).astype(np.float32)
        lanes = [dict(anchor=3, depth=int(rng.integers(1, 16)), children=int(rng.integers(1, 5)), intercept=[float(v) for v in rng.normal(0, 0.5, 7)],
                      temperature=temperature, noise=int(rng.integers(1 << 62)), chain=int(rng.integers(1, 16))) for _ in range(n)]
        trees = grow(backend, lattices, lanes, chains, rates)
        for l, (lattice, lane, got) in enumerate(zip(lattices, lanes, trees)):
            want = stated_tree(*lattice, oracle_lane(lane), chains[l], rates[l])
            if want is None:
                continue
            compare(got, want)
            same_tree(got, orc.draft_tree(*lattice, oracle_lane(lane), chains[l], rates[l]))
            compared += 1
    assert compared >= 20


def test_candidates_edges_tree_and_rows_in_one_graph(backend):
    """The draft side end to end on the GPU: a draft's logits to candidates and edges, to each lane's tree, to a decode
    step's rows, in one command graph, against the oracle's chain of the same steps."""
    print("case draft side end to end", flush=True)
    rng = np.random.default_rng(9)
    lanes_n, vocabulary, rank = 3, 20000, 256
    logits = rng.normal(0, 2.5, (lanes_n * 8, vocabulary)).astype(np.float32)
    hidden = orc.f32_to_bf16(rng.normal(0, 1, (lanes_n * 8, rank)).astype(np.float32))
    before = orc.f32_to_bf16(rng.normal(0, 0.08, (vocabulary, rank)).astype(np.float32))
    after = orc.f32_to_bf16(rng.normal(0, 0.08, (vocabulary, rank)).astype(np.float32))
    anchors = [11, 12, 13]
    lanes = [dict(anchor=a, depth=15, children=c, intercept=[0.5] * 7) for a, c in zip(anchors, (4, 2, 3))]
    up = backend.from_array
    b = dict(candidates=backend.allocate_buffer(lanes_n * 7 * 16 * 4), unary=backend.allocate_buffer(lanes_n * 7 * 16 * 4),
             edges=backend.allocate_buffer(lanes_n * 7 * 256 * 4), scratch=backend.allocate_buffer(ops.DraftSelector.candidate_scratch_bytes(lanes_n, vocabulary)),
             tokens=backend.allocate_buffer(lanes_n * 64), trees=backend.allocate_buffer(lanes_n * 128), scores=backend.allocate_buffer(lanes_n * 128),
             sizes=backend.allocate_buffer(16), draws=backend.allocate_buffer(lanes_n * 64), next=backend.allocate_buffer(lanes_n * 1024),
             caps=backend.allocate_buffer(lanes_n * 64))
    rows, cap = 30, 16
    step = dict(input=backend.allocate_buffer(rows * 4), tree=backend.allocate_buffer(rows * 8), lane_rows=backend.allocate_buffer(lanes_n * 8),
                sources=backend.allocate_buffer(rows * 4))
    graph = splash_amd.CommandGraph()
    ops.DraftSelector.add_candidates(graph, up(logits), up(hidden), b["scratch"], b["candidates"], b["unary"], b["edges"], up(before), up(after),
                                     vocabulary, vocabulary, vocabulary, anchors)
    ops.DraftSelector.add_tree(graph, b["candidates"], b["unary"], b["edges"], up(np.zeros((lanes_n, 15), np.uint32)),
                               up(np.zeros((lanes_n, 15, 4), np.float32)), b["tokens"], b["trees"], b["scores"], b["sizes"], b["draws"], b["next"],
                               b["caps"], lanes)
    ops.DraftSelector.add_verify_rows(graph, b["tokens"], b["trees"], b["scores"], b["sizes"], step["input"], step["tree"], step["lane_rows"],
                                      step["sources"], lanes_n, rows, cap)
    backend.run(graph)
    candidates, unary = orc.draft_candidates(logits, lanes_n)
    edges = orc.draft_edges(candidates, anchors, vocabulary, hidden, before, after)
    assert np.array_equal(b["candidates"].download(np.uint32).reshape(-1, 16), candidates)
    tokens, trees, scores, sizes = np.zeros((lanes_n, 16), np.uint32), np.zeros((lanes_n, 16), orc.TREE_DTYPE), np.zeros((lanes_n, 16, 2), np.float32), []
    gpu_edges = b["edges"].download(np.float32).reshape(lanes_n, 7, 16, 16)
    for l, lane in enumerate(lanes):
        # the tree over the GPU's own edges (its sums differ from the oracle's in the last bits)
        want = orc.draft_tree(candidates[7 * l:7 * l + 7], unary[7 * l:7 * l + 7], gpu_edges[l], oracle_lane(lane))
        if stated_tree(candidates[7 * l:7 * l + 7], unary[7 * l:7 * l + 7], gpu_edges[l], oracle_lane(lane)) is None:
            pytest.skip("a drawn lattice whose order hangs on the rounding of exp")
        n = len(want["tokens"])
        sizes.append(n)
        tokens[l, :n], trees[l, :n], scores[l, :n, 0], scores[l, :n, 1] = want["tokens"], want["tree"], want["q"], want["estimate"]
    got_sizes = b["sizes"].download(np.uint32)[:lanes_n]
    assert list(got_sizes) == sizes
    got_tokens = b["tokens"].download(np.uint32).reshape(lanes_n, 16)
    for l, n in enumerate(sizes):
        assert np.array_equal(got_tokens[l, :n], tokens[l, :n])
    w_tokens, w_tree, w_lane_rows, w_sources = orc.draft_verify_rows(tokens, trees, b["scores"].download(np.float32).reshape(lanes_n, 16, 2), sizes, rows, cap)
    assert np.array_equal(step["input"].download(np.uint32)[:rows], w_tokens)
    assert np.array_equal(step["tree"].download(np.uint8).view(orc.TREE_DTYPE)[:rows], w_tree)
    assert np.array_equal(step["lane_rows"].download(np.uint32)[:lanes_n * 2].reshape(lanes_n, 2), w_lane_rows)
    assert np.array_equal(step["sources"].download(np.uint32)[:rows], w_sources)


def test_tree_rejects_bad_lanes(backend):
    rng = np.random.default_rng(1)
    lattice = drawn_lattice(rng)
    for bad, message in [(dict(anchor=1, depth=16, children=1), "no deeper"), (dict(anchor=1, depth=3, children=5), "one to four"),
                         (dict(anchor=1, depth=3, children=1, chain=16), "no deeper"),
                         (dict(anchor=1, depth=3, children=1, temperature=-1.0), "invalid draft tree lane")]:
        with pytest.raises(splash_amd.SplashError, match=message):
            grow(backend, [lattice], [bad])


def test_a_tree_feeds_the_step_without_the_host(backend):
    """A sampled lane's tree goes from the draft side's kernels straight into the dense driver's input buffers (tokens,
    tree rows, depths, candidate children), and the step's results are those of the same step with its inputs written by
    the host from the oracle's tree: the draft side and the verify step meet on the device."""
    from splash_amd import verify
    from tests.dense_reference import DenseModel
    print("case tree into the step on the device", flush=True)
    V, rows, context, T = 32000, 16, 300, 0.9
    model = DenseModel(seed=21, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=V, layers=2)
    rng = np.random.default_rng(31)
    gpu = model.build_gpu(backend, max_lanes=1, context_tokens=context + 16)
    model.seed_context(gpu, None, rng)
    # a synthetic draft: logits and selector rows of one lane
    rank = 256
    logits = rng.normal(0, 2.0, (8, V)).astype(np.float32)
    hidden = orc.f32_to_bf16(rng.normal(0, 1, (8, rank)).astype(np.float32))
    before = orc.f32_to_bf16(rng.normal(0, 0.08, (V, rank)).astype(np.float32))
    after = orc.f32_to_bf16(rng.normal(0, 0.08, (V, rank)).astype(np.float32))
    anchor = 777
    draft_lane = dict(anchor=anchor, depth=15, children=3, intercept=[0.3] * 7, temperature=T, noise=12345678901234567)
    up = backend.from_array
    b = dict(candidates=backend.allocate_buffer(7 * 16 * 4), unary=backend.allocate_buffer(7 * 16 * 4), edges=backend.allocate_buffer(7 * 256 * 4),
             scratch=backend.allocate_buffer(ops.DraftSelector.candidate_scratch_bytes(1, V)), tokens=backend.allocate_buffer(64),
             trees=backend.allocate_buffer(128), scores=backend.allocate_buffer(128), sizes=backend.allocate_buffer(16), draws=backend.allocate_buffer(64),
             next=backend.allocate_buffer(1024), caps=backend.allocate_buffer(64), lane_rows=backend.allocate_buffer(16), sources=backend.allocate_buffer(64))
    lane = verify.Lane(rows, context, temperature=T)
    uniforms = rng.random((rows, 2)).astype(np.float32)
    child_uniforms = rng.random((rows, 4)).astype(np.float32)
    # the step's graph exists before its inputs do: its shape is the lane's 16 rows
    gpu.set_block([lane], np.zeros(rows, np.uint32), uniforms=uniforms)
    gpu.set_candidate_children(np.zeros((rows, 16), np.uint32), np.zeros((rows, 16), np.float32), np.full((rows, 4), 0xFF, np.uint8), child_uniforms)
    step = gpu.encode([lane], commit=False)
    assert "decode_sample_draw_children" in step.kernels()
    children = [gpu.buffer(verify.CANDIDATE_CHILDREN, which) for which in range(3)]
    draft = splash_amd.CommandGraph()
    ops.DraftSelector.add_candidates(draft, up(logits), up(hidden), b["scratch"], b["candidates"], b["unary"], b["edges"], up(before), up(after),
                                     V, V, V, [anchor])
    ops.DraftSelector.add_tree(draft, b["candidates"], b["unary"], b["edges"], up(np.zeros((1, 15), np.uint32)), up(np.zeros((1, 15, 4), np.float32)),
                               b["tokens"], b["trees"], b["scores"], b["sizes"], b["draws"], b["next"], b["caps"], [draft_lane])
    ops.DraftSelector.add_verify_rows(draft, b["tokens"], b["trees"], b["scores"], b["sizes"], gpu.buffer(verify.INPUT_TOKENS),
                                      gpu.buffer(verify.TREE_ROWS), b["lane_rows"], b["sources"], 1, rows, rows)
    ops.DraftSelector.add_verify_children(draft, b["sources"], b["lane_rows"], gpu.buffer(verify.TREE_ROWS), b["candidates"], b["next"], b["draws"],
                                          children[0], children[1], children[2], gpu.buffer(verify.DEPTHS), 1, rows)
    backend.run(draft)
    backend.run(step)
    device_results = gpu.results([lane])
    device_logits = gpu.buffer(verify.LOGITS).download(np.float32, rows * V).copy()
    assert b["sizes"].download(np.uint32)[0] == rows and list(b["lane_rows"].download(np.uint32)[:2]) == [0, rows]
    # the same step from the host: the oracle's tree over the GPU's own candidates and edges, laid out and gathered in numpy
    candidates = b["candidates"].download(np.uint32).reshape(7, 16)
    unary, edges = b["unary"].download(np.float32).reshape(7, 16), b["edges"].download(np.float32).reshape(7, 16, 16)
    oracle_lane = orc.draft_tree_lane(anchor=anchor, depth=15, children=3, intercept=[0.3] * 7, temperature=T, noise=draft_lane["noise"])
    if stated_tree(candidates, unary, edges, oracle_lane) is None:
        pytest.skip("a drawn lattice whose order hangs on the rounding of exp")
    grown = orc.draft_tree(candidates, unary, edges, oracle_lane)
    assert len(grown["tokens"]) == rows
    scores = np.stack([grown["q"], grown["estimate"]], axis=1)[None]
    w_tokens, w_tree, w_lane_rows, w_sources = orc.draft_verify_rows(grown["tokens"][None], grown["tree"][None], scores, [rows], rows, rows)
    ids = np.full((rows, 16), 0xFFFFFFFF, np.uint32)
    q = np.zeros((rows, 16), np.float32)
    draws = np.full((rows, 4), 0xFF, np.uint8)
    for r in range(rows):
        depth, source = int(w_tree["depth"][r]), int(w_sources[r])
        if depth < 7:
            ids[r], q[r], draws[r] = candidates[depth], grown["next"][source], grown["draws"][source]
    got_ids = children[0].download(np.uint32)[:rows * 16].reshape(rows, 16)
    got_draws = children[2].download(np.uint8)[:rows * 4].reshape(rows, 4)
    assert np.array_equal(got_ids, ids) and np.array_equal(got_draws, draws)
    assert np.allclose(children[1].download(np.float32)[:rows * 16].reshape(rows, 16), q, rtol=1e-4, atol=1e-7)
    assert np.array_equal(gpu.buffer(verify.INPUT_TOKENS).download(np.uint32)[:rows], w_tokens)
    assert np.array_equal(gpu.buffer(verify.DEPTHS).download(np.uint32)[:rows], w_tree["depth"].astype(np.uint32))
    # ... and run from the host's copies of exactly what the device wrote (its probabilities, to the last bit)
    q_device = children[1].download(np.float32)[:rows * 16].reshape(rows, 16).copy()
    gpu.set_block([lane], w_tokens, tree_rows=w_tree, uniforms=uniforms)
    gpu.set_candidate_children(ids, q_device, draws, child_uniforms)
    backend.run(step)
    assert np.array_equal(gpu.buffer(verify.LOGITS).download(np.float32, rows * V), device_logits)
    for got, want in zip(gpu.results([lane]), device_results):
        assert np.array_equal(got, want)


def test_trees_of_any_size_feed_a_step_recorded_once(backend):
    """Two greedy lanes whose drafts grow trees of different sizes on the device (sixteen rows and a chain of five): the
    rows in slots (spo_draft_add_verify_row_slots) and their depths go straight into the dense driver's input buffers of a
    step recorded, before any of it, for sixteen rows a lane. What each lane keeps, and its own rows' logits, are those
    of the step a host records for the trees' exact sizes from the packed layout of the same trees."""
    from splash_amd import verify
    from tests.dense_reference import DenseModel
    print("case trees of any size into one recorded step", flush=True)
    V, cap, contexts = 32000, 16, (200, 300)
    model = DenseModel(seed=22, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=V, layers=2)
    rng = np.random.default_rng(33)
    gpu = model.build_gpu(backend, max_lanes=2, context_tokens=[c + 16 for c in contexts])
    model.seed_context(gpu, None, rng)
    lanes = [verify.Lane(cap, c, table_first=f) for c, f in zip(contexts, model.table_first)]
    gpu.set_block(lanes, np.zeros(2 * cap, np.uint32))
    step = gpu.encode(lanes, commit=False)             # the step's shape: sixteen rows a lane, whatever the trees will be
    rank = 256
    up = backend.from_array
    logits = rng.normal(0, 2.0, (16, V)).astype(np.float32)
    hidden = orc.f32_to_bf16(rng.normal(0, 1, (16, rank)).astype(np.float32))
    before = orc.f32_to_bf16(rng.normal(0, 0.08, (V, rank)).astype(np.float32))
    after = orc.f32_to_bf16(rng.normal(0, 0.08, (V, rank)).astype(np.float32))
    anchors = [777, 4242]
    draft_lanes = [dict(anchor=anchors[0], depth=15, children=3, intercept=[0.3] * 7), dict(anchor=anchors[1], depth=4, children=1, intercept=[0.3] * 7)]
    b = dict(candidates=backend.allocate_buffer(2 * 7 * 16 * 4), unary=backend.allocate_buffer(2 * 7 * 16 * 4), edges=backend.allocate_buffer(2 * 7 * 256 * 4),
             scratch=backend.allocate_buffer(ops.DraftSelector.candidate_scratch_bytes(2, V)), tokens=backend.allocate_buffer(128),
             trees=backend.allocate_buffer(256), scores=backend.allocate_buffer(256), sizes=backend.allocate_buffer(16), draws=backend.allocate_buffer(128),
             next=backend.allocate_buffer(2048), caps=backend.allocate_buffer(128), lane_rows=backend.allocate_buffer(16), sources=backend.allocate_buffer(128),
             ids=backend.allocate_buffer(32 * 16 * 4), q=backend.allocate_buffer(32 * 16 * 4), drawn=backend.allocate_buffer(32 * 4))
    draft = splash_amd.CommandGraph()
    ops.DraftSelector.add_candidates(draft, up(logits), up(hidden), b["scratch"], b["candidates"], b["unary"], b["edges"], up(before), up(after),
                                     V, V, V, anchors)
    ops.DraftSelector.add_tree(draft, b["candidates"], b["unary"], b["edges"], up(np.zeros((2, 15), np.uint32)), up(np.zeros((2, 15, 4), np.float32)),
                               b["tokens"], b["trees"], b["scores"], b["sizes"], b["draws"], b["next"], b["caps"], draft_lanes)
    ops.DraftSelector.add_verify_row_slots(draft, b["tokens"], b["trees"], b["scores"], b["sizes"], gpu.buffer(verify.INPUT_TOKENS),
                                           gpu.buffer(verify.TREE_ROWS), b["lane_rows"], b["sources"], 2, cap)
    ops.DraftSelector.add_verify_children(draft, b["sources"], b["lane_rows"], gpu.buffer(verify.TREE_ROWS), b["candidates"], b["next"], b["draws"],
                                          b["ids"], b["q"], b["drawn"], gpu.buffer(verify.DEPTHS), 2, 2 * cap)
    backend.run(draft)
    backend.run(step)
    sizes = b["sizes"].download(np.uint32)[:2]
    assert list(sizes) == [16, 5]
    lane_rows = b["lane_rows"].download(np.uint32)[:4].reshape(2, 2)
    assert lane_rows.tolist() == [[0, 16], [16, 5]]
    selected, retained, accepted, masks = (np.array(a).copy() for a in gpu.results(lanes))
    slot_logits = gpu.buffer(verify.LOGITS).download(np.float32, 2 * cap * V).reshape(2 * cap, V).copy()
    # the host's step for the trees' exact sizes, from the packed layout of the device's own trees
    tokens = b["tokens"].download(np.uint32)[:32].reshape(2, 16)
    trees = b["trees"].download(np.uint8)[:256].view(orc.TREE_DTYPE).reshape(2, 16)
    scores = b["scores"].download(np.float32)[:64].reshape(2, 16, 2)
    w_tokens, w_tree, w_lane_rows, _ = orc.draft_verify_rows(tokens, trees, scores, sizes, 21, cap)
    assert w_lane_rows.tolist() == [[0, 16], [16, 5]]
    exact = [verify.Lane(16, contexts[0], table_first=model.table_first[0]), verify.Lane(5, contexts[1], table_first=model.table_first[1])]
    gpu.set_block(exact, w_tokens, tree_rows=w_tree)
    backend.run(gpu.encode(exact, commit=False))
    e_selected, e_retained, e_accepted, e_masks = gpu.results(exact)
    exact_logits = gpu.buffer(verify.LOGITS).download(np.float32, 21 * V).reshape(21, V)
    assert np.array_equal(slot_logits[:21], exact_logits)     # lane 1's five rows follow lane 0's sixteen in both
    assert list(retained) == list(e_retained) and list(accepted) == list(e_accepted) and list(masks) == list(e_masks)
    assert np.array_equal(selected[:retained[0]], np.asarray(e_selected)[:retained[0]])
    assert np.array_equal(selected[cap:cap + retained[1]], np.asarray(e_selected)[16:16 + retained[1]])
    assert all(m >> 5 == 0 for m in [masks[1]])               # nothing past the chain's five rows is ever kept
