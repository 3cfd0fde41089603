"""End-to-end parity of the dense verify step (BASELINE.json config 1) against the oracle, through the C ABI."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops, verify
from tests import oracle as orc
from tests.dense_reference import DenseModel

pytestmark = pytest.mark.gpu


def top2_gap(logits):
    part = np.partition(logits, -2, axis=1)
    return part[:, -1] - part[:, -2]


def close_bf16(got_bits, want_bits):
    """Two bf16 tensors agree: cosine >= 0.9999; every element within max(2e-2, two bf16 steps of it) but for at most
    one in ten thousand, which a stage of several bf16 roundings (a mixer, an FFN) moves further now and then, and none
    further than six steps."""
    g, w = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(want_bits).astype(np.float64)
    cos = (g * w).sum() / np.sqrt((g * g).sum() * (w * w).sum())
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w), 2.0 ** -100))) - 7)     # a bf16 step at a value: 2^(its exponent - 7)
    error = np.abs(g - w)
    beyond = error > np.maximum(2e-2, 2 * step)
    worst = float(np.where(error <= 2e-2, 0, error / step).max())
    return cos >= 0.9999 and beyond.mean() <= 1e-4 and worst <= 6, (cos, error.max(), float(beyond.mean()), worst)


@pytest.mark.parametrize("rows,context", [(16, 512), (5, 37)])
def test_config1_verify_step(backend, rows, context):
    """2-layer dense decoder (hidden 1024, 16 q / 8 kv heads x 64, SwiGLU 3072, vocab 32000), N(0, 0.02)
    weights quantized to Q4_K (Q6_K head), INT8 KV context, a block of uniform-random draft tokens, greedy.
    Layer by layer from the GPU's own layer input: hidden rows within the bf16 tolerance of the oracle's;
    logits from the GPU's final hidden rows within max-abs 2e-2 and cosine >= 0.9999; accepted ids bit-exact.
    The whole chain against the oracle's own chain: cosine >= 0.9999 and max-abs 5e-2 -- a bf16 pipeline is
    chaotic at that level: the oracle with fp32 instead of fp64 projection sums moves its own logits by 2.2e-2."""
    print(f"case config 1 rows={rows} context={context}", flush=True)
    model = DenseModel(seed=11, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=2)
    rng = np.random.default_rng(rows)
    tokens = rng.integers(0, 32000, rows).astype(np.uint32)
    gpu = model.build_gpu(backend, max_lanes=1, context_tokens=context + 16)
    model.seed_context(gpu, context, rng)
    lane = verify.Lane(rows, context)
    gpu.set_block([lane], tokens)
    # the whole step in one command
    backend.run(gpu.encode([lane], commit=True))
    chain_logits = gpu.buffer(verify.LOGITS).download(np.float32, rows * 32000).reshape(rows, 32000)
    selected, retained, accepted, mask = gpu.results([lane])
    # the same step part by part, teacher-forcing the oracle with the GPU's hidden rows
    hidden_of = lambda: gpu.buffer(verify.HIDDEN, 0).download(np.uint16, rows * 1024).reshape(rows, 1024)
    full = gpu.encode([lane], commit=False)      # RoPE tables of the block (first dispatch of a step)
    backend.run(gpu.encode_part(0, 0, [lane]))
    assert np.array_equal(hidden_of(), model.oracle_embedding(tokens))
    for layer in range(2):
        before = hidden_of()
        backend.run(gpu.encode_part(1, layer, [lane]))
        ok, detail = close_bf16(hidden_of(), model.oracle_layer(before, layer, context))
        assert ok, (layer, detail)
    final = hidden_of()
    backend.run(gpu.encode_part(2, 0, [lane]))
    got_logits = gpu.buffer(verify.LOGITS).download(np.float32, rows * 32000).reshape(rows, 32000)
    # A part starts with a norm pass over its input rows; inside the whole step the projection before it wrote
    # that table without the rows' inverse RMS, which the reading projection applies to its sums: one bf16
    # operand rounding apart.
    part_cos = (got_logits.astype(np.float64) * chain_logits).sum() / np.sqrt((got_logits.astype(np.float64) ** 2).sum() * (chain_logits.astype(np.float64) ** 2).sum())
    assert part_cos >= 0.9999 and np.abs(got_logits - chain_logits).max() <= 2e-2, part_cos
    want_logits = model.oracle_head(final)
    cos = (got_logits.astype(np.float64) * want_logits).sum() / np.sqrt((got_logits.astype(np.float64) ** 2).sum() * (want_logits ** 2).sum())
    err = np.abs(got_logits - want_logits).max()
    assert cos >= 0.9999 and err <= 2e-2, (cos, err)
    # greedy acceptance of the GPU's logits is bit-exact
    gpu_argmax = np.array([orc.argmax(got_logits[r]) for r in range(rows)], dtype=np.uint32)
    kept, acc, m = orc.accept_tree(ops.chain_tree_rows([rows]), tokens, gpu_argmax)
    assert retained[0] == len(kept) and accepted[0] == acc and mask[0] == m and np.array_equal(selected[:len(kept)], kept)
    # the whole chain against the oracle's own chain
    model.seed_context(gpu, context, np.random.default_rng(rows + 1000))   # fresh context arrays for the oracle's stores
    del full
    rng = np.random.default_rng(rows); rng.integers(0, 32000, rows)
    model.seed_context(gpu, context, rng)
    want = model.oracle_step(tokens, context)
    cos = (chain_logits.astype(np.float64) * want["logits"]).sum() / np.sqrt((chain_logits.astype(np.float64) ** 2).sum() * (want["logits"] ** 2).sum())
    err = np.abs(chain_logits - want["logits"]).max()
    assert cos >= 0.9999 and err <= 5e-2, (cos, err)
    # Where that difference comes from is not the step's deferred norms: the parts, each after a norm pass that rounds as
    # the oracle's does, lie as far from the oracle's chain (the stages that move are the SwiGLU rows and the attention
    # rows, where a sum taken in fp32 and one taken exactly fall on two sides of a bf16 rounding now and then, and a
    # large activation is worth 3e-2 a step).
    rms = lambda a: float(np.sqrt(((a - want["logits"]) ** 2).mean()))
    print(f"  free-running against the oracle's chain: step max-abs {err:.4f} rms {rms(chain_logits):.5f}; parts max-abs "
          f"{np.abs(got_logits - want['logits']).max():.4f} rms {rms(got_logits):.5f}", flush=True)
    assert rms(chain_logits) <= 1.15 * rms(got_logits)
    sure = top2_gap(want["logits"]) > 1e-1
    assert np.array_equal(gpu_argmax[sure], want["selected"][sure])
    # where the oracle's top two are closer than that, the GPU's choice is still one of the oracle's near-ties
    picked = want["logits"][np.arange(rows), gpu_argmax]
    assert (picked >= want["logits"].max(axis=1) - 1e-1).all()
    if sure.all():
        assert np.array_equal(selected[:retained[0]], want["kept"]) and accepted[0] == want["accepted"] and mask[0] == want["retained_rows"]


def test_config1_accepts_a_self_consistent_draft(backend):
    """A draft block that continues the target's own greedy choices is accepted up to the first planted mismatch."""
    print("case config 1 accepted draft", flush=True)
    rows, context = 8, 100
    model = DenseModel(seed=12, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=2)
    rng = np.random.default_rng(3)
    gpu = model.build_gpu(backend, max_lanes=1, context_tokens=context + 16)
    model.seed_context(gpu, context, rng)
    tokens = np.zeros(rows, dtype=np.uint32)
    tokens[0] = 1234
    lane = verify.Lane(rows, context)
    for r in range(1, rows):     # grow the block row by row with the target's own selection
        gpu.set_block([lane], tokens)
        backend.run(gpu.encode([lane], commit=False))
        tokens[r] = gpu.buffer(verify.LOGITS).download(np.float32, rows * 32000).reshape(rows, 32000)[r - 1].argmax()
    planted = tokens.copy()
    planted[5] = (planted[5] + 1) % 32000
    gpu.set_block([lane], planted)
    backend.run(gpu.encode([lane], commit=True))
    selected, retained, accepted, mask = gpu.results([lane])
    assert accepted[0] == 4 and retained[0] == 5 and mask[0] == 0b11111
    assert np.array_equal(selected[:4], planted[1:5]) and selected[4] == tokens[5]


def test_a_context_built_from_tokens_alone(backend):
    """No seeded KV: from an empty context, three blocks of sixteen prompt tokens run through the step one after the
    other (their rows' keys and values stay in the pages whatever the acceptance says; the caller advances the lane's
    committed tokens itself), then a verify block over the 48-token context the GPU wrote. Against the oracle run the
    same way, storing its own keys and values: logits within the bf16 tolerance of a chain of four steps (cosine >=
    0.999, max-abs 5e-2), and the empty history (committed 0) is a case of its own for the attention's partition."""
    print("case config 1 context from tokens", flush=True)
    model = DenseModel(seed=13, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=2)
    rng = np.random.default_rng(2)
    gpu = model.build_gpu(backend, max_lanes=1, context_tokens=64)
    pages = model.physical_pages
    zero = lambda shape, dtype: np.zeros(shape, dtype=dtype)
    model.context = [[zero((pages, 8, ops.PAGE_TOKENS, 64), np.int8), zero((pages, 8, ops.PAGE_TOKENS), np.float32),
                      zero((pages, 8, ops.PAGE_TOKENS, 64), np.int8), zero((pages, 8, ops.PAGE_TOKENS), np.float32)] for _ in range(2)]
    for layer in range(2):   # the pools start as whatever the allocation held: clear them as the oracle's context is
        gpu.buffer(verify.KV_POOL, layer).fill(0)
    prompt = rng.integers(0, 32000, 48).astype(np.uint32)
    for block in range(3):
        tokens = prompt[16 * block:16 * block + 16]
        lane = verify.Lane(16, 16 * block)
        gpu.set_block([lane], tokens)
        backend.run(gpu.encode([lane], commit=False))
        got = gpu.buffer(verify.LOGITS).download(np.float32, 16 * 32000).reshape(16, 32000)
        want = model.oracle_step(tokens, 16 * block)["logits"]
        cos = (got.astype(np.float64) * want).sum() / np.sqrt((got.astype(np.float64) ** 2).sum() * (want ** 2).sum())
        assert cos >= 0.999 and np.abs(got - want).max() <= 5e-2, (block, cos, np.abs(got - want).max())
    draft = rng.integers(0, 32000, 16).astype(np.uint32)
    lane = verify.Lane(16, 48)
    gpu.set_block([lane], draft)
    backend.run(gpu.encode([lane], commit=True))
    got = gpu.buffer(verify.LOGITS).download(np.float32, 16 * 32000).reshape(16, 32000)
    want = model.oracle_step(draft, 48)
    cos = (got.astype(np.float64) * want["logits"]).sum() / np.sqrt((got.astype(np.float64) ** 2).sum() * (want["logits"] ** 2).sum())
    assert cos >= 0.999 and np.abs(got - want["logits"]).max() <= 5e-2, (cos, np.abs(got - want["logits"]).max())
    selected, retained, accepted, mask = gpu.results([lane])
    picks = np.array([orc.argmax(got[r]) for r in range(16)], dtype=np.uint32)
    kept, acc, m = orc.accept_tree(ops.chain_tree_rows([16]), draft, picks)
    assert retained[0] == len(kept) and accepted[0] == acc and mask[0] == m and np.array_equal(selected[:len(kept)], kept)


def test_a_sampled_tree_block_tests_its_drawn_children(backend):
    """A tree block through the driver with sampled acceptance: every row tests the children its draft drew among its
    sixteen candidates (sampling.metal:697-880), the acceptance walk follows the selected children. The candidates of a
    row are the likeliest tokens of the target itself at that row (found by running the step as the tree grows), so
    children are accepted and rejected; against the oracle's rows over the step's own logits and its walk."""
    print("case config 1 sampled tree block", flush=True)
    V, T, rows = 32000, 0.03, 8          # a peaked target: its likeliest token is accepted, the others seldom
    model = DenseModel(seed=14, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=V, layers=2)
    rng = np.random.default_rng(8)
    context = 200
    gpu = model.build_gpu(backend, max_lanes=1, context_tokens=context + 16)
    model.seed_context(gpu, context, rng)
    parents = [0xFFFF, 0, 0, 1, 1, 2, 3, 3]
    tree = np.zeros(rows, dtype=orc.TREE_DTYPE)
    for r, parent in enumerate(parents):
        tree[r] = ((1 << r) | (0 if r == 0 else int(tree[parent]["ancestors"])), parent, 0 if r == 0 else int(tree[parent]["depth"]) + 1)
    children_of = {r: [c for c in range(rows) if parents[c] == r] for r in range(rows)}
    tokens = np.zeros(rows, dtype=np.uint32)
    tokens[0] = 4321
    ids = np.zeros((rows, 16), np.uint32)
    q = np.zeros((rows, 16), np.float32)
    draws = np.full((rows, 4), 0xFF, np.uint8)
    child_uniforms = rng.random((rows, 4)).astype(np.float32)
    uniforms = rng.random((rows, 2)).astype(np.float32)
    lane = verify.Lane(rows, context, temperature=T)
    logits_of = lambda: gpu.buffer(verify.LOGITS).download(np.float32, rows * V).reshape(rows, V)
    for r in range(rows):       # parents come before children: a row's candidates from the target's own logits at that row
        gpu.set_block([lane], tokens, tree_rows=tree, uniforms=uniforms)
        gpu.set_candidate_children(ids, q, draws, child_uniforms)
        backend.run(gpu.encode([lane], commit=False))
        row_logits = logits_of()[r].astype(np.float64)
        top = np.argsort(-row_logits)[:16]
        ids[r] = rng.permutation(top)
        w = np.exp((row_logits[ids[r]] - row_logits.max()) / (2 * T))        # a flatter draft than the target
        q[r] = (w / w.sum()).astype(np.float32)
        best = int(np.argmax(row_logits[ids[r]]))
        order = ([best] if r % 2 == 0 else []) + [i for i in rng.permutation(16) if i != best]   # even rows draw the likeliest first
        for c, (child, index) in enumerate(zip(children_of[r], order)):
            draws[r, c] = index
            tokens[child] = ids[r, index]
    gpu.set_block([lane], tokens, tree_rows=tree, uniforms=uniforms)
    gpu.set_candidate_children(ids, q, draws, child_uniforms)
    graph = gpu.encode([lane], commit=False)
    assert "decode_sample_draw_children" in graph.kernels()
    backend.run(graph)
    logits = logits_of()
    selected, retained, accepted, mask = gpu.results([lane])
    want_rows, sure = [], True
    for r in range(rows):
        n = int((draws[r] != 0xFF).sum())
        want, close = orc.children_row(logits[r], (T, 0.0, 0, 1.0), ids[r], q[r], list(draws[r, :n]), child_uniforms[r], float(uniforms[r, 0]))
        want_rows.append(want)
        sure &= close > 1e-5
    kept, acc, m = orc.accept_tree(tree, tokens, np.array(want_rows, np.uint32))
    print(f"  oracle rows {want_rows}; kept {list(kept)} accepted {acc} mask {m:#x}; sure {sure}", flush=True)
    if sure:
        assert retained[0] == len(kept) and accepted[0] == acc and mask[0] == m and np.array_equal(selected[:len(kept)], kept)
    assert 1 <= retained[0] <= rows and (not sure or accepted[0] >= 1)


def test_a_penalized_lane_selects_from_its_penalized_rows(backend):
    """SamplingPolicy::penalties through the driver (Sampling.hpp:71, Sampling.cpp:163-194 in the reference): of two lanes
    one takes penalties. Its rows of the step's logits are the oracle's penalties of the rows the same step leaves without
    them, bit for bit, its selections their argmax and its acceptance the walk over those; the other lane's rows and
    results do not change. A step that commits counts the tokens the penalized lane keeps into its row of the table, which
    the next step's penalties then read."""
    print("case config 1 penalized lane", flush=True)
    from splash_amd import ops
    V = 4096
    model = DenseModel(seed=21, hidden=512, q_heads=8, kv_heads=4, head_dim=64, ffn=1024, vocabulary=V, layers=2)
    rng = np.random.default_rng(3)
    context = 70
    gpu = model.build_gpu(backend, max_lanes=2, context_tokens=context + 16)
    make_lanes = lambda: [verify.Lane(6, context, table_first=model.table_first[0]), verify.Lane(9, context, table_first=model.table_first[1])]
    lanes = make_lanes()
    model.seed_context(gpu, None, rng)
    tokens = rng.integers(0, V, 15).astype(np.uint32)
    tokens[10] = tokens[11] = tokens[9]                               # the penalized lane drafts one token three times
    tree = ops.chain_tree_rows([6, 9])
    logits_of = lambda: gpu.buffer(verify.LOGITS).download(np.float32, 15 * V).reshape(15, V)
    gpu.set_block(lanes, tokens, tree_rows=tree)
    backend.run(gpu.encode(lanes, commit=False))
    plain, plain_results = logits_of(), [np.array(a).copy() for a in gpu.results(lanes)]
    # lane 1's history: a prompt that holds the plain step's favourite tokens, outputs that hold some of them again
    favourites = np.argmax(plain[6:], axis=1).astype(np.uint32)
    history = np.concatenate([favourites[:5], rng.integers(0, V, 20).astype(np.uint32), favourites[3:7], favourites[3:4]])
    words = ops.Sampling.rebuild_penalty_words(V, history, 5, pending_token=int(tokens[6]))
    table = gpu.buffer(verify.PENALTY_WORDS)
    table.upload(words, offset_bytes=V * 4)
    penalties = (1.4, 0.9, 0.35)
    gpu.set_penalties(1, *penalties)
    graph = gpu.encode(lanes, commit=False)
    assert "decode_sample_penalize" in graph.kernels() and "decode_sample_count_tokens" not in graph.kernels()
    backend.run(graph)
    seen = logits_of()
    got_tokens, got_retained, got_accepted, got_mask = (np.array(a).copy() for a in gpu.results(lanes))
    want = orc.penalize(plain[6:], words, tokens[6:], tree["ancestors"][6:], *penalties)
    assert seen[:6].tobytes() == plain[:6].tobytes() and seen[6:].tobytes() == want.tobytes()
    assert (got_retained[0], got_accepted[0], got_mask[0]) == (plain_results[1][0], plain_results[2][0], plain_results[3][0])
    assert np.array_equal(got_tokens[:got_retained[0]], plain_results[0][:got_retained[0]])
    selected = np.array([orc.argmax(row) for row in want], np.uint32)
    assert np.any(selected != favourites)                             # the penalties moved a selection
    kept, accepted, mask = orc.accept_tree(tree[6:], tokens[6:], selected)
    assert np.array_equal(got_tokens[6:6 + len(kept)], kept) and (got_retained[1], got_accepted[1], got_mask[1]) == (len(kept), accepted, mask)
    # a committing step counts what the lane keeps; the lane without penalties counts nothing
    graph = gpu.encode(lanes, commit=True)
    assert "decode_sample_count_tokens" in graph.kernels()
    backend.run(graph)
    counted = table.download(np.uint32, 2 * V).reshape(2, V)
    want_words = words.copy()
    np.add.at(want_words, kept, 1)
    assert np.array_equal(counted[1], want_words) and not counted[0].any()
    # a thinking cutoff on the other lane: its rows from depth 2 on select the end, whatever their logits; the acceptance
    # walks those selections
    gpu.set_thinking_cutoff(0, row=2, end=[17, 18, 19])
    lanes = make_lanes()
    gpu.set_block(lanes, tokens, tree_rows=tree)
    graph = gpu.encode(lanes, commit=False)
    assert "decode_sample_end_thinking" in graph.kernels()
    backend.run(graph)
    ended = np.array([orc.argmax(row) for row in plain[:6]], np.uint32)
    ended[2:5] = [17, 18, 19]
    kept0, accepted0, mask0 = orc.accept_tree(tree[:6], tokens[:6], ended)
    got_tokens, got_retained, got_accepted, got_mask = (np.array(a).copy() for a in gpu.results(lanes))
    assert np.array_equal(got_tokens[:len(kept0)], kept0) and (got_retained[0], got_accepted[0], got_mask[0]) == (len(kept0), accepted0, mask0)
    gpu.set_thinking_cutoff(0)
    # penalties off again: the step is the plain one
    gpu.set_penalties(1)
    lanes = make_lanes()
    gpu.set_block(lanes, tokens, tree_rows=tree)
    graph = gpu.encode(lanes, commit=False)
    assert "decode_sample_penalize" not in graph.kernels() and "decode_sample_end_thinking" not in graph.kernels()
    backend.run(graph)
    assert logits_of().tobytes() == plain.tobytes()


def test_admission_and_stop_tokens_through_the_driver(backend):
    """SamplingPolicy::constrained / excludesStopTokens and the step's stop tokens through the driver: a constrained lane
    selects, row by row, the best token its mask row admits; a lane that ignores end-of-sequence never selects a stop
    token; acceptance ends a path at a stop token it accepts; and a thinking end that waits for its mask starts at the
    first row whose mask admits it. Against the oracle's argmax and walk over the plain step's logits."""
    print("case config 1 admission and stop tokens", flush=True)
    from splash_amd import ops
    V = 4096
    model = DenseModel(seed=23, hidden=512, q_heads=8, kv_heads=4, head_dim=64, ffn=1024, vocabulary=V, layers=2)
    rng = np.random.default_rng(4)
    context = 50
    gpu = model.build_gpu(backend, max_lanes=2, context_tokens=context + 16)
    make_lanes = lambda: [verify.Lane(5, context, table_first=model.table_first[0]), verify.Lane(8, context, table_first=model.table_first[1])]
    lanes = make_lanes()
    model.seed_context(gpu, None, rng)
    tokens = rng.integers(0, V, 13).astype(np.uint32)
    tree = ops.chain_tree_rows([5, 8])
    gpu.set_block(lanes, tokens, tree_rows=tree)
    backend.run(gpu.encode(lanes, commit=False))
    plain = gpu.buffer(verify.LOGITS).download(np.float32, 13 * V).reshape(13, V)
    best = np.argmax(plain, axis=1).astype(np.uint32)
    # lane 0 constrained: its masks forbid each row's favourite; lane 1: its favourites of rows 0 and 2 are stop tokens
    words = (V + 31) // 32
    allowed = rng.random((13, V)) < 0.5
    allowed[np.arange(13), best] = False
    end_first = 777
    allowed[:5, end_first] = [False, False, False, True, True]
    mask = np.packbits(allowed.reshape(13, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(13, words)
    gpu.buffer(verify.TOKEN_MASK).upload(mask)
    # lane 1's draft follows its own greedy continuation for three rows, so that the walk reaches a stop token
    for r in range(3):
        tokens[6 + r] = best[5 + r]
        gpu.set_block(lanes, tokens, tree_rows=tree)
        backend.run(gpu.encode(lanes, commit=False))
        plain = gpu.buffer(verify.LOGITS).download(np.float32, 13 * V).reshape(13, V)
        best = np.argmax(plain, axis=1).astype(np.uint32)
    stops = [int(best[7]), 4095]
    gpu.set_admission(0, constrained=True)
    gpu.set_stop_tokens(stops)
    lanes = make_lanes()
    gpu.set_block(lanes, tokens, tree_rows=tree)
    graph = gpu.encode(lanes, commit=False)
    assert "decode_sample_admit" in graph.kernels()
    backend.run(graph)
    got_tokens, got_retained, got_accepted, got_mask = (np.array(a).copy() for a in gpu.results(lanes))
    want0 = np.array([orc.argmax(np.where(allowed[r], plain[r], -np.inf)) for r in range(5)], np.uint32)
    assert np.all(want0 != best[:5])
    kept, accepted, path = orc.accept_tree(tree[:5], tokens[:5], want0, stop_tokens=stops)
    assert np.array_equal(got_tokens[:len(kept)], kept) and (got_retained[0], got_accepted[0], got_mask[0]) == (len(kept), accepted, path)
    # lane 1 does not exclude stop tokens: its walk accepts up to the stop token its row 2 selects and ends there
    kept, accepted, path = orc.accept_tree(tree[5:], tokens[5:], best[5:], stop_tokens=stops)
    assert len(kept) == 3 and kept[-1] == stops[0]
    assert np.array_equal(got_tokens[5:5 + len(kept)], kept) and (got_retained[1], got_accepted[1], got_mask[1]) == (len(kept), accepted, path)
    # excluding them, the lane selects its next best there and walks on
    gpu.set_admission(1, excludes_stop_tokens=True)
    lanes = make_lanes()
    gpu.set_block(lanes, tokens, tree_rows=tree)
    backend.run(gpu.encode(lanes, commit=False))
    got_tokens, got_retained, got_accepted, got_mask = (np.array(a).copy() for a in gpu.results(lanes))
    without = plain[5:].copy()
    without[:, stops] = -np.inf
    want1 = np.array([orc.argmax(row) for row in without], np.uint32)
    kept, accepted, path = orc.accept_tree(tree[5:], tokens[5:], want1, stop_tokens=stops)
    assert stops[0] not in kept
    assert np.array_equal(got_tokens[5:5 + len(kept)], kept) and (got_retained[1], got_accepted[1], got_mask[1]) == (len(kept), accepted, path)
    # the constrained lane's thinking end waits for its mask: rows 3 and 4 admit its first token
    gpu.set_thinking_cutoff(0, row=1, end=[end_first, 778], waits_for_mask=True)
    lanes = make_lanes()
    gpu.set_block(lanes, tokens, tree_rows=tree)
    backend.run(gpu.encode(lanes, commit=False))
    ended = orc.thinking_cutoff(want0, tokens[:5], tree[:5], V, 1, [end_first, 778], admits=allowed[:5, end_first])
    assert list(ended[3:]) == [end_first, 778] and np.array_equal(ended[:3], want0[:3])
    kept, accepted, path = orc.accept_tree(tree[:5], tokens[:5], ended, stop_tokens=stops)
    got_tokens, got_retained, got_accepted, got_mask = (np.array(a).copy() for a in gpu.results(lanes))
    assert np.array_equal(got_tokens[:len(kept)], kept) and (got_retained[0], got_accepted[0], got_mask[0]) == (len(kept), accepted, path)
    gpu.set_admission(0)
    with pytest.raises(ValueError, match="constrained"):
        gpu.encode(make_lanes(), commit=False)                        # an end that waits needs a constrained lane


@pytest.mark.parametrize("lanes_rows", [[16], [7, 16, 3]])
def test_chained_projections_change_nothing(backend, lanes_rows):
    """A step whose layers dispatch their four projections after the attention as one chain (a layer's output, gate/up
    and down projections and the next layer's q|k|v, the LM head after the last) gives the logits, the hidden rows and
    the results of the step that dispatches them one by one, bit for bit, on repeated runs, in far fewer dispatches."""
    print(f"case chained step lanes={lanes_rows}", flush=True)
    model = DenseModel(seed=15, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=4)
    rng = np.random.default_rng(8)
    contexts = [300 + 111 * i for i in range(len(lanes_rows))]
    gpu = model.build_gpu(backend, max_lanes=len(lanes_rows), context_tokens=[c + 16 for c in contexts])
    model.seed_context(gpu, None, rng)
    lanes = [verify.Lane(rows, committed, table_first=first) for rows, committed, first in zip(lanes_rows, contexts, model.table_first)]
    total = sum(lanes_rows)
    gpu.set_block(lanes, rng.integers(0, 32000, total).astype(np.uint32))

    def run(chained):
        gpu.set_chained(chained)
        graph = gpu.encode(lanes, commit=False)
        outcomes = []
        for _ in range(3):
            backend.run(graph)
            assert gpu.chain_status() == 0           # what a reader of the buffers asks before it trusts them
            outcomes.append((gpu.buffer(verify.LOGITS).download(np.float32, total * 32000).copy(),
                             gpu.buffer(verify.HIDDEN, 0).download(np.uint16, total * 1024).copy(), gpu.results(lanes)))
        return len(graph), outcomes
    plain_dispatches, plain = run(False)
    chained_dispatches, chained = run(True)
    assert chained_dispatches == plain_dispatches - 3 * 4   # four projections become one in each of the four layers
    for logits, hidden, results in plain[1:] + chained:
        assert np.array_equal(logits, plain[0][0]) and np.array_equal(hidden, plain[0][1])
        for got, want in zip(results, plain[0][2]):
            assert np.array_equal(got, want)


@pytest.mark.parametrize("lanes_rows", [[16], [7, 16, 3]])
def test_the_fused_prepare_changes_nothing(backend, lanes_rows):
    """A step whose q|k|v projections prepare their attention blocks themselves (off by default) gives the logits, the
    hidden rows, the cache and the results of the step that runs the prepare kernel after each projection, bit for bit,
    with a dispatch a layer fewer."""
    print(f"case fused prepare step lanes={lanes_rows}", flush=True)
    model = DenseModel(seed=16, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=4)
    rng = np.random.default_rng(9)
    contexts = [250 + 111 * i for i in range(len(lanes_rows))]
    gpu = model.build_gpu(backend, max_lanes=len(lanes_rows), context_tokens=[c + 16 for c in contexts])
    model.seed_context(gpu, None, rng)
    lanes = [verify.Lane(rows, committed, table_first=first) for rows, committed, first in zip(lanes_rows, contexts, model.table_first)]
    total = sum(lanes_rows)
    gpu.set_block(lanes, rng.integers(0, 32000, total).astype(np.uint32))

    def run(fused):
        gpu.set_fused_prepare(fused)
        graph = gpu.encode(lanes, commit=False)
        outcomes = []
        for _ in range(2):
            backend.run(graph)
            outcomes.append((gpu.buffer(verify.LOGITS).download(np.float32, total * 32000).copy(),
                             gpu.buffer(verify.HIDDEN, 0).download(np.uint16, total * 1024).copy(),
                             np.concatenate([gpu.buffer(verify.KV_POOL, layer).download(np.uint8) for layer in range(4)]), gpu.results(lanes)))
        return len(graph), outcomes
    fused_dispatches, fused = run(True)
    plain_dispatches, plain = run(False)
    assert fused_dispatches == plain_dispatches - 4
    for logits, hidden, pool, results in plain[1:] + fused:
        assert np.array_equal(logits, plain[0][0]) and np.array_equal(hidden, plain[0][1]) and np.array_equal(pool, plain[0][2])
        for got, want in zip(results, plain[0][3]):
            assert np.array_equal(got, want)


@pytest.mark.parametrize("prompt_tokens", [64, 53, 128])
def test_a_prompt_chunk_in_one_pass_equals_its_blocks_one_by_one(backend, prompt_tokens):
    """Prefill through the path's own kernels: a chunk of up to 128 prompt tokens as blocks of sixteen rows of ONE sequence
    in one pass over the weights (block i's history ends where block i - 1's rows end; its keys and values are in the
    pages before any block attends) leaves the pools and the hidden rows of the same blocks run one step after the
    other, bit for bit."""
    print(f"case prompt chunk tokens={prompt_tokens}", flush=True)
    model = DenseModel(seed=17, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=3)
    rng = np.random.default_rng(4)
    gpu = model.build_gpu(backend, max_lanes=(prompt_tokens + 15) // 16, context_tokens=[prompt_tokens + 300])
    model.seed_context(gpu, None, rng)
    first, committed = model.table_first[0], 250      # the chunk crosses a page
    prompt = rng.integers(0, 32000, prompt_tokens).astype(np.uint32)
    blocks = [(16 * b, min(16, prompt_tokens - 16 * b)) for b in range((prompt_tokens + 15) // 16)]
    pools = lambda: np.concatenate([gpu.buffer(verify.KV_POOL, layer).download(np.uint8) for layer in range(3)])
    start = pools()
    # one step a block
    hidden = []
    for at, rows in blocks:
        lane = verify.Lane(rows, committed + at, table_first=first)
        gpu.set_block([lane], prompt[at:at + rows])
        backend.run(gpu.encode([lane], commit=False))
        hidden.append(gpu.buffer(verify.HIDDEN, 0).download(np.uint16, rows * 1024).copy())
    want_pools, want_hidden = pools(), np.concatenate(hidden)
    assert (want_pools != start).any()
    for layer in range(3):
        gpu.buffer(verify.KV_POOL, layer).upload(start.reshape(3, -1)[layer])
    # the chunk in one pass
    graph = gpu.encode_prefill(first, committed, prompt_tokens)
    gpu.set_prefill_block(prompt)
    backend.run(graph)
    assert np.array_equal(pools(), want_pools)
    assert np.array_equal(gpu.buffer(verify.HIDDEN, 0).download(np.uint16, prompt_tokens * 1024), want_hidden)
    # fewer passes over the weights: a layer's dispatches once, not once a block
    assert len(graph) < len(gpu.encode([verify.Lane(16, committed, table_first=first)], commit=False)) 


@pytest.mark.parametrize("prompt_tokens", [300, 1000])
def test_a_long_prompt_chunk_equals_its_blocks_one_by_one(backend, prompt_tokens):
    """A chunk of more rows than a step's (a driver created with room for them): the projections run in windows of 256
    rows around one chunked attention over all the rows, layer by layer. The pools and the hidden rows are those of
    the sixteen-row blocks run one step after the other, bit for bit."""
    print(f"case long prompt chunk tokens={prompt_tokens}", flush=True)
    model = DenseModel(seed=23, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=3)
    rng = np.random.default_rng(8)
    gpu = model.build_gpu(backend, max_lanes=1, context_tokens=[prompt_tokens + 300], prefill_rows=1024)
    model.seed_context(gpu, None, rng)
    first, committed = model.table_first[0], 250
    prompt = rng.integers(0, 32000, prompt_tokens).astype(np.uint32)
    blocks = [(at, min(16, prompt_tokens - at)) for at in range(0, prompt_tokens, 16)]
    pools = lambda: np.concatenate([gpu.buffer(verify.KV_POOL, layer).download(np.uint8) for layer in range(3)])
    start = pools()
    hidden = []
    for at, rows in blocks:
        lane = verify.Lane(rows, committed + at, table_first=first)
        gpu.set_block([lane], prompt[at:at + rows])
        backend.run(gpu.encode([lane], commit=False))
        hidden.append(gpu.buffer(verify.HIDDEN, 0).download(np.uint16, rows * 1024).copy())
    want_pools, want_hidden = pools(), np.concatenate(hidden)
    for layer in range(3):
        gpu.buffer(verify.KV_POOL, layer).upload(start.reshape(3, -1)[layer])
    graph = gpu.encode_prefill(first, committed, prompt_tokens)
    gpu.set_prefill_block(prompt)
    backend.run(graph)
    assert np.array_equal(pools(), want_pools)
    assert np.array_equal(gpu.buffer(verify.HIDDEN, 0).download(np.uint16, prompt_tokens * 1024), want_hidden)
    with pytest.raises(ValueError):
        gpu.encode_prefill(first, committed, 1025)


def test_a_staged_prompt_chunk_is_the_exact_one_to_the_staged_rules_rounding(backend):
    """The same chunk through the prefill tile (DenseVerify::setStagedPrefill: every weight rounded once to half, as the
    reference's prompt chunks run): the hidden rows agree with the exact chunk's as two bf16 tensors of several stages do,
    the keys and values it stored are the exact chunk's codes but for a step here and there, and a verify step on top of
    the context it built selects the tokens the exact context's step selects wherever the logits' margin exceeds their
    difference."""
    print("case staged prompt chunk", flush=True)
    prompt_tokens, V = 600, 32000
    model = DenseModel(seed=29, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=V, layers=3)
    rng = np.random.default_rng(9)
    gpu = model.build_gpu(backend, max_lanes=1, context_tokens=[prompt_tokens + 300], prefill_rows=1024)
    model.seed_context(gpu, None, rng)
    first, committed = model.table_first[0], 250
    prompt = rng.integers(0, V, prompt_tokens).astype(np.uint32)
    block = rng.integers(0, V, 16).astype(np.uint32)
    pools = lambda: np.concatenate([gpu.buffer(verify.KV_POOL, layer).download(np.uint8) for layer in range(3)])
    start = pools()
    seen = {}
    for staged in (False, True):
        gpu.set_staged_prefill(staged)
        for layer in range(3):
            gpu.buffer(verify.KV_POOL, layer).upload(start.reshape(3, -1)[layer])
        graph = gpu.encode_prefill(first, committed, prompt_tokens)
        gpu.set_prefill_block(prompt)
        backend.run(graph)
        hidden = gpu.buffer(verify.HIDDEN, 0).download(np.uint16, prompt_tokens * 1024).copy()
        stored = pools()
        lane = verify.Lane(16, committed + prompt_tokens, table_first=first)
        gpu.set_block([lane], block)
        backend.run(gpu.encode([lane], commit=False))
        logits = gpu.buffer(verify.LOGITS).download(np.float32, 16 * V).reshape(16, V).copy()
        seen[staged] = (hidden, stored, logits, len(graph.kernels()))
    gpu.set_staged_prefill(False)
    (h0, p0, l0, d0), (h1, p1, l1, d1) = seen[False], seen[True]
    print(f"  dispatches: {d0} in windows of the step's kernels, {d1} through the prefill tile", flush=True)
    # Two rules, not two roundings of one: every weight is rounded to half before it multiplies, in every projection of
    # every layer. The reference holds such rows to cosine 0.9999 and max-abs 2e-2 a stage; over three layers' stages:
    a, b = orc.bf16_to_f32(h0).astype(np.float64), orc.bf16_to_f32(h1).astype(np.float64)
    hidden_cosine, error = float((a * b).sum() / np.sqrt((a * a).sum() * (b * b).sum())), np.abs(a - b)
    print(f"  hidden rows: cosine {hidden_cosine:.6f}, largest difference {error.max():.4f} of magnitudes up to {np.abs(a).max():.2f}, "
          f"{(error > 2e-2).mean():.5f} of them past 2e-2", flush=True)
    assert hidden_cosine >= 0.9999 and error.max() <= 6e-2 and (error > 2e-2).mean() <= 2e-3
    # the keys and values the chunk stored: the same values to a couple of INT8 steps
    helper = ops.KvPages.__new__(ops.KvPages)
    helper.kv_heads, helper.head_dim, helper.page_bytes = 8, 64, gpu.page_bytes
    assert (p0 != p1).any()
    for layer in range(3):
        kc0, ks0, vc0, vs0 = helper.unpack_pages(p0.reshape(3, -1, gpu.page_bytes)[layer])
        kc1, ks1, vc1, vs1 = helper.unpack_pages(p1.reshape(3, -1, gpu.page_bytes)[layer])
        for c0, s0, c1, s1 in ((kc0, ks0, kc1, ks1), (vc0, vs0, vc1, vs1)):
            apart = np.abs(c0.astype(np.float64) * s0[..., None] - c1.astype(np.float64) * s1[..., None]) / np.maximum(s0[..., None], 1e-30)
            assert np.percentile(apart, 99.9) <= 2.5 and apart.max() <= 8, (layer, float(np.percentile(apart, 99.9)), float(apart.max()))
    cosine = float((l0.astype(np.float64) * l1).sum() / np.sqrt((l0.astype(np.float64) ** 2).sum() * (l1.astype(np.float64) ** 2).sum()))
    top = np.sort(l0, axis=1)
    clear = top[:, -1] - top[:, -2] > 2 * np.abs(l0 - l1).max()
    print(f"  logits cosine {cosine:.6f}, largest difference {np.abs(l0 - l1).max():.4f}, rows with a clear margin {int(clear.sum())}/16", flush=True)
    assert cosine >= 0.9999 and np.array_equal(l0.argmax(axis=1)[clear], l1.argmax(axis=1)[clear])


def test_eight_lanes_equal_each_lane_alone(backend):
    """The driver's most lanes: eight lanes of unequal blocks and histories in one step give, lane by lane, the logits,
    selections and acceptance each lane gives alone, bit for bit."""
    print("case eight lanes", flush=True)
    model = DenseModel(seed=19, hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=2)
    rng = np.random.default_rng(6)
    rows = [16, 3, 9, 16, 1, 12, 16, 7]
    contexts = [100 + 97 * i for i in range(8)]
    gpu = model.build_gpu(backend, max_lanes=8, context_tokens=[c + 16 for c in contexts])
    model.seed_context(gpu, None, rng)
    lanes = [verify.Lane(r, c, table_first=f) for r, c, f in zip(rows, contexts, model.table_first)]
    tokens = rng.integers(0, 32000, sum(rows)).astype(np.uint32)
    gpu.set_block(lanes, tokens)
    backend.run(gpu.encode(lanes, commit=False))
    logits = gpu.buffer(verify.LOGITS).download(np.float32, sum(rows) * 32000).reshape(-1, 32000).copy()
    selected, retained, accepted, mask = (np.array(a).copy() for a in gpu.results(lanes))
    first = 0
    for i, lane in enumerate(lanes):
        gpu.set_block([lane], tokens[first:first + lane.rows])
        backend.run(gpu.encode([lane], commit=False))
        alone = gpu.buffer(verify.LOGITS).download(np.float32, lane.rows * 32000).reshape(-1, 32000)
        assert np.array_equal(alone, logits[first:first + lane.rows]), i
        s1, r1, a1, m1 = gpu.results([lane])
        assert r1[0] == retained[i] and a1[0] == accepted[i] and m1[0] == mask[i], i
        assert np.array_equal(np.asarray(s1)[:r1[0]], selected[first:first + r1[0]]), i
        first += lane.rows
