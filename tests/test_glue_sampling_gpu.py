"""GPU parity of the glue kernels and the acceptance kernels against the oracle, through the C ABI."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,width", [(1, 1024), (16, 5120), (33, 2048)])
def test_rms_norm_and_its_activation_table(backend, rows, width):
    """normalization.metal:59-99; the fused table equals gguf_prepare_table of the normalized rows bit for bit."""
    print(f"case norm rows={rows} width={width}", flush=True)
    rng = np.random.default_rng(rows)
    x = orc.f32_to_bf16((rng.standard_normal((rows, width)) * 3).astype(np.float32))
    w = orc.f32_to_bf16((1 + 0.2 * rng.standard_normal(width)).astype(np.float32))
    xb, wb = backend.from_array(x), backend.from_array(w)
    plain, fused = backend.allocate_buffer(rows * width * 2), backend.allocate_buffer(rows * width * 2)
    nbytes = ops.gguf_table_bytes(width, rows)
    table, table2 = backend.allocate_buffer(nbytes), backend.allocate_buffer(nbytes)
    g = splash_amd.CommandGraph()
    ops.Normalization.add_rms(g, xb, wb, plain, width, rows)
    ops.Normalization.add_rms_table(g, xb, wb, fused, table, width, rows)
    import ctypes

    class Prepare(ctypes.Structure):
        _fields_ = [("input_size", ctypes.c_uint32), ("rows", ctypes.c_uint32), ("tiles", ctypes.c_uint32), ("row_stride", ctypes.c_uint32)]
    tiles = (rows + 15) // 16
    g.add("gguf_prepare_table", [plain, table2], Prepare(width, rows, tiles, width), (width // 32, tiles, 1), (64, 1, 1))
    backend.run(g)
    got = plain.download(np.uint16).reshape(rows, width)
    want = orc.rms_norm(x, w)
    assert np.array_equal(fused.download(np.uint16).reshape(rows, width), got)
    # the reduction tree of a 64-lane wavefront differs from the oracle's 32-lane one: bf16 ulp at most
    diff = np.abs(got.astype(np.int32) - want.astype(np.int32))
    assert diff.max() <= 1 and (diff > 0).mean() < 0.01, (diff.max(), (diff > 0).mean())
    assert np.array_equal(table.download(), table2.download())


@pytest.mark.parametrize("rows,n,k,bf16_weights", [(130, 128, 2048, False), (1, 7, 8, False), (33, 64, 2048, True), (16, 250, 1000, False)])
def test_float_projection_equals_the_oracle(backend, rows, n, k, bf16_weights):
    """kernels/shared/gguf_float.metal: the fp32 projection of weights kept as rows, bit for bit the oracle's fixed
    order; a row alone gives its bits of the batch; the bf16 destination is the fp32 result rounded once, written at
    its columns of a wider row that it otherwise leaves alone (the GDN alpha/beta columns of a packed row)."""
    print(f"case float projection rows={rows} n={n} k={k} bf16={bf16_weights}", flush=True)
    rng = np.random.default_rng(rows + n)
    x = orc.f32_to_bf16((rng.standard_normal((rows, k)) * 2).astype(np.float32))
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    weights = orc.f32_to_bf16(w) if bf16_weights else w
    want = orc.float_projection(x, weights)
    xb, wb = backend.from_array(x), backend.from_array(weights)
    out = backend.allocate_buffer(rows * n * 4)
    stride, offset = n + 24, 16
    before = orc.f32_to_bf16(rng.standard_normal((rows, stride)).astype(np.float32))
    packed = backend.from_array(before)
    alone = backend.allocate_buffer(n * 4)
    g = splash_amd.CommandGraph()
    ops.FloatProjection.add(g, xb, wb, n, k, out, rows, bf16_weights=bf16_weights)
    ops.FloatProjection.add(g, xb, wb, n, k, packed, rows, out_stride=stride, out_offset=offset, bf16_weights=bf16_weights, float32_output=False)
    ops.FloatProjection.add(g, backend.from_array(x[rows - 1:]), wb, n, k, alone, 1, bf16_weights=bf16_weights)
    backend.run(g)
    got = out.download(np.float32).reshape(rows, n)
    assert got.tobytes() == want.tobytes()
    assert alone.download(np.float32).tobytes() == want[rows - 1].tobytes()
    rows_out = packed.download(np.uint16).reshape(rows, stride)
    assert np.array_equal(rows_out[:, offset:offset + n], orc.f32_to_bf16(want))
    assert np.array_equal(rows_out[:, :offset], before[:, :offset]) and np.array_equal(rows_out[:, offset + n:], before[:, offset + n:])
    with pytest.raises(ValueError):
        ops.FloatProjection.add(splash_amd.CommandGraph(), xb, wb, n, k, packed, rows, out_stride=n, out_offset=8, float32_output=False)


@pytest.mark.parametrize("fmt", ops.FORMATS)
def test_embedding_gathers_native_rows(backend, fmt):
    """embedding.metal:10-18: bf16(decode(row)); a token past the vocabulary gives zeros."""
    vocab, hidden = 500, 1024
    native = orc.make_native(fmt, vocab, hidden, 3)
    tokens = np.array([0, 499, 17, 500, 4_000_000_000, 17], dtype=np.uint32)
    out = backend.allocate_buffer(len(tokens) * hidden * 2)
    g = splash_amd.CommandGraph()
    ops.Embedding.add(g, fmt, backend.from_array(native), vocab, hidden, backend.from_array(tokens), out, len(tokens))
    backend.run(g)
    assert np.array_equal(out.download(np.uint16).reshape(len(tokens), hidden), orc.embed(fmt, native, vocab, hidden, tokens))


def test_rope_tree_tables(backend):
    """rope.metal:51-80: cos/sin of (anchor + depth) * inverse frequency per packed row."""
    pairs = 64
    inv = (1e6 ** (-np.arange(pairs) / pairs)).astype(np.float32)
    depth = np.array([0, 1, 2, 2, 3, 0, 1], dtype=np.uint32)
    seqs = [(0, 5, 32752), (5, 2, 7)]
    cos, sin = backend.allocate_buffer(7 * pairs * 4), backend.allocate_buffer(7 * pairs * 4)
    g = splash_amd.CommandGraph()
    ops.RoPE.add_tree_tables(g, backend.from_array(inv), backend.from_array(depth), cos, sin, pairs, seqs)
    backend.run(g)
    pos = np.array([32752 + d for d in depth[:5]] + [7 + d for d in depth[5:]], dtype=np.float32)
    angle = (pos[:, None] * inv[None, :]).astype(np.float32).astype(np.float64)
    assert np.abs(cos.download(np.float32).reshape(7, pairs) - np.cos(angle)).max() < 2e-6
    assert np.abs(sin.download(np.float32).reshape(7, pairs) - np.sin(angle)).max() < 2e-6


def test_row_copy(backend):
    """RowCopy.hpp:17-28: a capture copies a layer's output rows into its slot of wider rows."""
    rng = np.random.default_rng(5)
    source = rng.integers(0, 65536, (20, 96), dtype=np.uint16)
    before = rng.integers(0, 65536, (24, 300), dtype=np.uint16)
    destination = backend.from_array(before)
    g = splash_amd.CommandGraph()
    ops.RowCopy.add(g, backend.from_array(source), (3, 96, 16), destination, (5, 300, 100), 16, 64)
    backend.run(g)
    want = before.copy()
    want[5:21, 100:164] = source[3:19, 16:80]
    assert np.array_equal(destination.download(np.uint16).reshape(24, 300), want)
    for bad in (((3, 96, 40), (5, 300, 100), 16, 64), ((3, 96, 16), (5, 300, 250), 16, 64), ((5, 96, 16), (5, 300, 100), 16, 64)):
        with pytest.raises(ValueError):
            ops.RowCopy.add(splash_amd.CommandGraph(), backend.from_array(source), bad[0], destination, bad[1], bad[2], bad[3])


def sampling_buffers(backend, rows, V, logits, draft=None, uniforms=None, tokens=None, tree=None):
    sizes = ops.Sampling.workspace(rows)
    b = dict(logits=backend.from_array(logits.astype(np.float32)), tokens=backend.allocate_buffer(rows * 4),
             partial_values=backend.allocate_buffer(sizes[0]), partial_indices=backend.allocate_buffer(sizes[1]),
             draft_probabilities=backend.from_array(draft.astype(np.float32)) if draft is not None else None,
             uniforms=backend.from_array(uniforms.astype(np.float32)) if uniforms is not None else None,
             masses=backend.allocate_buffer(sizes[2]), ranges=backend.allocate_buffer(sizes[3]),
             decisions=backend.allocate_buffer(sizes[4]),
             input_tokens=backend.from_array(tokens) if tokens is not None else None,
             tree_rows=backend.from_array(tree) if tree is not None else None)
    return b


def test_greedy_argmax_ties_sentinel_and_large_vocabulary(backend):
    """sampling.metal:1896-1997: ties to the lowest id, NaN/-inf skipped, no selectable logit -> sentinel."""
    print("case argmax", flush=True)
    rng = np.random.default_rng(5)
    rows, V = 16, 151936
    logits = rng.standard_normal((rows, V)).astype(np.float32)
    logits[1, [7, 90000, 151935]] = 9.0                      # a three-way tie
    logits[2, :] = -np.inf
    logits[3, :] = np.nan
    logits[4, 151935] = 50.0                                 # the last token
    logits[5, rng.random(V) < 0.5] = np.nan
    logits[6, :] = 1.0                                       # all equal: id 0
    b = sampling_buffers(backend, rows, V, logits)
    g = splash_amd.CommandGraph()
    ops.Sampling.add_verify(g, b, V, V, [(0, rows)], [0.0])
    backend.run(g)
    got = b["tokens"].download(np.uint32)
    want = np.array([orc.argmax(logits[r]) for r in range(rows)], dtype=np.uint32)
    assert np.array_equal(got, want)
    assert got[1] == 7 and got[2] == ops.NO_TOKEN and got[3] == ops.NO_TOKEN and got[4] == 151935 and got[6] == 0


def test_acceptance_walk_matches_oracle_on_trees(backend):
    """sampling.metal:2044-2083 decode_accept_tree over chains and trees, several lanes, caps and stop tokens."""
    print("case accept tree", flush=True)
    from tests.test_oracle_sampling import random_tree
    rng = np.random.default_rng(6)
    for trial in range(20):
        lanes, first = [], 0
        trees, toks, sels = [], [], []
        for _ in range(int(rng.integers(1, 5))):
            rows = int(rng.integers(1, 17))
            lanes.append((first, rows)); first += rows
            trees.append(random_tree(rng, rows) if trial % 2 else ops.chain_tree_rows([rows]))
            toks.append(rng.integers(0, 3, rows).astype(np.uint32)); sels.append(rng.integers(0, 3, rows).astype(np.uint32))
        tree, tokens, selected = np.concatenate(trees), np.concatenate(toks), np.concatenate(sels)
        remaining = [int(rng.integers(1, 20)) for _ in lanes]
        stops = (2, ops.NO_TOKEN, ops.NO_TOKEN, ops.NO_TOKEN) if trial % 3 == 0 else (ops.NO_TOKEN,) * 4
        tb = backend.from_array(selected)
        ret, acc, mask = (backend.allocate_buffer(len(lanes) * 4) for _ in range(3))
        g = splash_amd.CommandGraph()
        ops.Sampling.add_acceptance(g, backend.from_array(tokens), backend.from_array(tree), tb, ret, acc, mask, lanes, remaining, stops)
        backend.run(g)
        out, retained, accepted, masks = tb.download(np.uint32), ret.download(np.uint32), acc.download(np.uint32), mask.download(np.uint32)
        for i, (f, rows) in enumerate(lanes):
            kept, a, m = orc.accept_tree(tree[f:f + rows], tokens[f:f + rows], selected[f:f + rows], remaining[i],
                                         [s for s in stops if s != ops.NO_TOKEN])
            assert retained[i] == len(kept) and accepted[i] == a and masks[i] == m
            assert np.array_equal(out[f:f + len(kept)], kept)


def test_rejection_sampling_rows_match_oracle(backend):
    """sampling.metal:713-885 at a full-vocabulary draft distribution: the drafted child is accepted iff
    u q < p, else the row draws from max(p - q, 0); ids equal the oracle's except where a comparison
    lies within 1e-5 of its threshold (target_sampling_metal_test.mm:2645-2709)."""
    print("case rejection sampling", flush=True)
    rng = np.random.default_rng(7)
    rows, V, T = 16, 32000, 0.7
    logits = (rng.standard_normal((rows, V)) * 2.5).astype(np.float32)
    logits[3, rng.random(V) < 0.01] = -np.inf
    dl = rng.standard_normal((rows, V)) * 2
    draft = np.exp(dl - dl.max(axis=1, keepdims=True)); draft = (draft / draft.sum(axis=1, keepdims=True)).astype(np.float32)
    p = np.exp((logits.astype(np.float64) - np.nanmax(np.where(np.isfinite(logits), logits, -1e30), axis=1, keepdims=True)) / T)
    p = np.where(np.isfinite(logits), p, 0); p /= p.sum(axis=1, keepdims=True)
    tokens = np.zeros(rows, dtype=np.uint32)
    for r in range(1, rows):   # row r's token is the child drawn at row r - 1: mix likely-accepted and likely-rejected ones
        tokens[r] = int(np.argmax(p[r - 1])) if r % 2 else int(rng.choice(V, p=draft[r - 1].astype(np.float64) / draft[r - 1].sum()))
    uniforms = rng.random((rows, 2)).astype(np.float32)
    tree = ops.chain_tree_rows([rows])
    b = sampling_buffers(backend, rows, V, logits, draft, uniforms, tokens, tree)
    g = splash_amd.CommandGraph()
    ops.Sampling.add_verify(g, b, V, V, [(0, rows)], [T])
    backend.run(g)
    got = b["tokens"].download(np.uint32)
    checked = accepted_rows = 0
    for r in range(rows):
        child = int(tokens[r + 1]) if r + 1 < rows else orc.NO_TOKEN
        want, accepted, close = orc.rejection_row(logits[r], T, draft[r] if child != orc.NO_TOKEN else None, child,
                                                  float(uniforms[r, 1]), float(uniforms[r, 0]))
        if close > 1e-5:
            assert got[r] == want, (r, got[r], want, accepted)
            checked += 1
            accepted_rows += accepted
    assert checked >= rows - 2 and 0 < accepted_rows < rows
    # a greedy lane beside a sampled one keeps its argmax
    g = splash_amd.CommandGraph()
    ops.Sampling.add_verify(g, b, V, V, [(0, 8), (8, 8)], [0.0, T])
    backend.run(g)
    mixed = b["tokens"].download(np.uint32)
    assert all(mixed[r] == orc.argmax(logits[r]) for r in range(8))


@pytest.mark.parametrize("V,policy", [(151936, (0.7, 0.0, 0, 1.0)), (32000, (0.9, 0.0, 40, 0.95))])
def test_tree_rows_test_their_drawn_children(backend, V, policy):
    """sampling.metal:697-880 (vocabulary_draw with children): every sampled row of a tree block tests the children its
    draft drew among sixteen candidates, one to four of them or none, then draws from the last residual: among the
    candidates or, past them, outside them. Token for token the oracle's, except where one of its comparisons lies within
    1e-5 of its threshold (target_sampling_metal_test.mm:2645-2709); a greedy lane beside keeps its argmax."""
    print(f"case children rows V={V}", flush=True)
    rng = np.random.default_rng(V)
    rows, K = 16, 16
    logits = (rng.standard_normal((rows, V)) * 2.5).astype(np.float32)
    logits[2, rng.random(V) < 0.02] = -np.inf
    for r in (1, 4, 6, 9):                                 # peaked rows: a child that is the likeliest token is accepted
        logits[r, rng.integers(0, V, 2)] += np.float32(14.0)
    T = policy[0]
    ids = np.zeros((rows, K), np.uint32)
    q = np.zeros((rows, K), np.float32)
    draws = np.full((rows, 4), 0xFF, np.uint8)
    for r in range(rows):
        # the candidates: the row's likeliest tokens mixed with random ones, so that children are accepted and rejected
        top = np.argsort(-logits[r])[:8]
        ids[r] = rng.permutation(np.concatenate([top, rng.choice(V, 8, replace=False)]))[:K]
        if r == 5:
            ids[r, 12:] = 0xFFFFFFFF                    # a draft row of fewer comparable logits
        weights = -np.log(0.5 * (rng.random(K) + 1.0))
        weights[ids[r] >= V] = 0
        if r % 3 == 0:
            weights[rng.integers(0, K, 3)] = 0
        q[r] = (weights / weights.sum()).astype(np.float32)
        count = r % 5                                   # 0 .. 4 children
        keys = sorted(((np.log(q[r, i]) - np.log(-np.log(rng.random() + 1e-300)), i) for i in range(K) if q[r, i] > 0), reverse=True)
        for c, (_, i) in enumerate(keys[:count]):
            draws[r, c] = i
    if True:   # a row whose candidates hold none of its mass and whose children are all rejected: the draw lands outside them
        ids[7] = rng.choice(np.where(logits[7] < -3)[0], K, replace=False)
        draws[7] = [0, 1, 2, 3]
    child_uniforms = rng.random((rows, 4)).astype(np.float32)
    uniforms = rng.random((rows, 2)).astype(np.float32)
    tokens = rng.integers(0, V, rows).astype(np.uint32)
    tree = ops.chain_tree_rows([rows])
    b = sampling_buffers(backend, rows, V, logits, None, uniforms, tokens, tree)
    b.update(candidate_ids=backend.from_array(ids), candidate_probabilities=backend.from_array(q), candidate_draws=backend.from_array(draws),
             child_uniforms=backend.from_array(child_uniforms))
    g = splash_amd.CommandGraph()
    ops.Sampling.add_verify(g, b, V, V, [(0, 12), (12, 4)], [policy, 0.0])
    assert "decode_sample_draw_children" in g.kernels() and "decode_sample_draw" not in g.kernels()
    backend.run(g)
    got = b["tokens"].download(np.uint32)
    checked = children_selected = outside = 0
    for r in range(12):
        n = int((draws[r] != 0xFF).sum())
        want, close = orc.children_row(logits[r], policy, ids[r], q[r], list(draws[r, :n]), child_uniforms[r], float(uniforms[r, 0]))
        if close > 1e-5:
            assert got[r] == want, (r, n, got[r], want)
            checked += 1
            children_selected += int(n and got[r] in ids[r, draws[r, :n]])
            outside += int(got[r] not in ids[r])
    assert checked >= 9 and children_selected >= 1 and outside >= 1
    assert all(got[r] == orc.argmax(logits[r]) for r in range(12, 16))
    # the buffers are checked before anything is added
    short = dict(b, candidate_draws=backend.allocate_buffer(16))
    with pytest.raises(ValueError, match="drawn children"):
        ops.Sampling.add_verify(splash_amd.CommandGraph(), short, V, V, [(0, 12), (12, 4)], [policy, 0.0])


@pytest.mark.parametrize("ties", [False, True])
def test_truncated_distributions_match_oracle(backend, ties):
    """min_p, top_k and top_p (distribution_end, sampling.metal:603-670): the end of every row's distribution -- the
    last kept token's key and id, the kept count -- equals the oracle's sort, the kept mass to fp32 summation order,
    and the rows' selections the oracle's over the cut distribution, except where a comparison lies within 1e-5 of its
    threshold. With ties: logits on a grid of halves, so that top_k and the nucleus end inside runs of equal logits."""
    print(f"case truncated sampling ties={ties}", flush=True)
    rng = np.random.default_rng(11 + ties)
    V = 151936 if not ties else 40000
    lanes = [(0, 3), (3, 3), (6, 3), (9, 3), (12, 2), (14, 1), (15, 1)]
    policies = [(0.7, 0.0, 50, 1.0), (0.7, 0.0, 0, 0.9), (1.2, 0.02, 0, 1.0), (0.5, 0.001, 1000, 0.95), (0.7, 0.0, V + 1, 1.0), (0.9, 0.0, 2, 0.5),
                (0.0, 0.0, 0, 1.0)]
    rows = 16
    logits = (rng.standard_normal((rows, V)) * 2.5).astype(np.float32)
    if ties:
        logits = (np.round(logits * 2) / 2).astype(np.float32)
    logits[4, rng.random(V) < 0.01] = -np.inf
    dl = rng.standard_normal((rows, V)) * 2
    draft = np.exp(dl - dl.max(axis=1, keepdims=True)); draft = (draft / draft.sum(axis=1, keepdims=True)).astype(np.float32)
    tokens = np.zeros(rows, dtype=np.uint32)
    tree = ops.chain_tree_rows([n for _, n in lanes])
    for first, n in lanes:        # a lane's row r + 1 carries the child drawn at its row r: a likely token, or a draft draw
        for r in range(first + 1, first + n):
            d64 = draft[r - 1].astype(np.float64)
            tokens[r] = int(np.argmax(logits[r - 1])) if r % 2 else int(rng.choice(V, p=d64 / d64.sum()))
    uniforms = rng.random((rows, 2)).astype(np.float32)
    b = sampling_buffers(backend, rows, V, logits, draft, uniforms, tokens, tree)
    g = splash_amd.CommandGraph()
    ops.Sampling.add_verify(g, b, V, V, lanes, policies)
    backend.run(g)
    got = b["tokens"].download(np.uint32)
    words = b["decisions"].download(np.uint32).reshape(rows, 8)
    checked = 0
    for (first, n), policy in zip(lanes, policies):
        T, min_p, top_k, top_p = policy
        for r in range(first, first + n):
            if T == 0.0:
                assert got[r] == orc.argmax(logits[r])
                continue
            cuts = min_p > 0 or (top_k and top_k < V) or top_p < 1
            key, last, mass, count, close_end = orc.distribution_end(logits[r], T, min_p, top_k, top_p)
            if cuts and close_end > 1e-5:
                assert (words[r, 2], words[r, 3], words[r, 5]) == (key, last, count), (r, policy)
                assert abs(words[r, 4:5].view(np.float32)[0] - mass) <= 1e-5 * mass
            child = int(tokens[r + 1]) if r + 1 < first + n else orc.NO_TOKEN
            want, accepted, close = orc.rejection_row_policy(logits[r], policy, draft[r] if child != orc.NO_TOKEN else None, child,
                                                             float(uniforms[r, 1]), float(uniforms[r, 0]))
            if close > 1e-5:
                assert got[r] == want, (r, policy, got[r], want, accepted)
                checked += 1
    assert checked >= 12


def test_constraint_masks_and_stop_exclusion(backend):
    """TargetRow::admits (sampling.metal:42-46): a constrained lane's rows select only tokens of their mask rows, a lane
    that ignores end-of-sequence never a stop token, greedy or sampled; the other lanes' rows are untouched. The
    oracle sees the same rows with -infinity at the tokens a lane does not admit."""
    print("case sampling admits", flush=True)
    rng = np.random.default_rng(21)
    rows, V, words = 12, 5000, (5000 + 31) // 32
    lanes = [(0, 3), (3, 3), (6, 3), (9, 3)]
    # greedy constrained; sampled constrained + stop-excluding with a nucleus; greedy stop-excluding; plain sampled
    policies = [(0.0, 0.0, 0, 1.0, 1, 0), (0.8, 0.0, 0, 0.9, 1, 1), (0.0, 0.0, 0, 1.0, 0, 1), (0.7, 0.0, 0, 1.0, 0, 0)]
    logits = (rng.standard_normal((rows, V)) * 2.5).astype(np.float32)
    stops = [int(np.argmax(logits[6])), int(np.argmax(logits[4])), 17]
    allowed = rng.random((rows, V)) < 0.3
    allowed[:, 0] = True
    allowed[1] = False                              # a row that admits nothing selects the sentinel
    bits = np.zeros((rows, words * 32), dtype=np.uint8)
    bits[:, :V] = allowed
    mask = np.packbits(bits.reshape(rows, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(rows, words)
    dl = rng.standard_normal((rows, V)) * 2
    draft = np.exp(dl - dl.max(axis=1, keepdims=True)); draft = (draft / draft.sum(axis=1, keepdims=True)).astype(np.float32)
    tokens = rng.integers(0, V, rows).astype(np.uint32)
    uniforms = rng.random((rows, 2)).astype(np.float32)
    tree = ops.chain_tree_rows([n for _, n in lanes])
    b = sampling_buffers(backend, rows, V, logits, draft, uniforms, tokens, tree)
    b["token_mask"], b["mask_words"] = backend.from_array(mask), words
    g = splash_amd.CommandGraph()
    ops.Sampling.add_verify(g, b, V, V, lanes, policies, stop_tokens=stops)
    backend.run(g)
    got = b["tokens"].download(np.uint32)
    seen = b["logits"].download(np.float32).reshape(rows, V)
    for (first, n), policy in zip(lanes, policies):
        for r in range(first, first + n):
            x = logits[r].copy()
            if policy[4]:
                x[~allowed[r]] = -np.inf
            if policy[5]:
                x[stops] = -np.inf
            assert np.array_equal(seen[r], x)
            if policy[0] == 0.0:
                assert got[r] == orc.argmax(x), r
                continue
            child = int(tokens[r + 1]) if r + 1 < first + n else orc.NO_TOKEN
            want, _, close = orc.rejection_row_policy(x, policy[:4], draft[r] if child != orc.NO_TOKEN else None, child,
                                                      float(uniforms[r, 1]), float(uniforms[r, 0]))
            if close > 1e-5:
                assert got[r] == want, (r, got[r], want)
            assert got[r] == orc.NO_TOKEN or np.isfinite(x[got[r]])
    assert got[1] == orc.NO_TOKEN and got[6] != stops[0] and got[4] != stops[1]
    with pytest.raises(ValueError, match="constraint"):
        ops.Sampling.add_verify(splash_amd.CommandGraph(), {**b, "token_mask": None}, V, V, lanes, policies)


def test_penalties_rewrite_the_rows_and_count_what_a_step_keeps(backend):
    """Sampling::addPenalties and the device's count of a step's tokens: the logits rows of the penalized lanes are the
    oracle's bit for bit (chain and tree blocks, a stride wider than the vocabulary, NaN and -infinity among the logits,
    tokens drafted several times), the other lanes' rows are untouched, greedy rows then select the argmax of the
    penalized rows, and the tokens each penalized lane retains are counted into its row of the table, twice if kept
    twice, so that a second step's penalties see them."""
    from tests.test_oracle_sampling import random_tree
    print("case sampling penalties", flush=True)
    rng = np.random.default_rng(77)
    V, stride = 5003, 5008
    lanes = [(0, 5), (5, 16), (21, 1), (22, 9)]
    rows = 31
    # lane 0: defaults (left alone); lane 1: a tree, all three penalties; lane 2: one row, repetition; lane 3: a chain, presence / frequency
    penalties = [(1.0, 0.0, 0.0, 3), (1.25, 0.4, 0.15, 2), (0.8, 0.0, 0.0, 0), (1.0, 1.5, 0.3, 1)]
    logits = np.zeros((rows, stride), np.float32)
    logits[:, :V] = (rng.standard_normal((rows, V)) * 3).astype(np.float32)
    logits[6, rng.integers(0, V, 40)] = -np.inf
    logits[7, rng.integers(0, V, 40)] = np.nan
    logits[:, V:] = 123.0                                            # the padding of a row is never touched
    tree = np.concatenate([ops.chain_tree_rows([5]), random_tree(rng, 16), ops.chain_tree_rows([1]), ops.chain_tree_rows([9])])
    tokens = rng.integers(0, 40, rows).astype(np.uint32)              # few distinct tokens: drafts repeat and hit the table
    # a row whose best token its own context drafted and whose second best nothing penalizes: the selection moves
    logits[24, tokens[23]], logits[24, 4000] = 20.0, 19.0
    table = np.zeros((4, V), np.uint32)
    for row in range(4):
        hit = rng.integers(0, 60, 30)
        table[row, hit] = rng.integers(0, 4, 30).astype(np.uint32) | (rng.integers(0, 2, 30).astype(np.uint32) << 31)
    words = backend.from_array(table)
    b = sampling_buffers(backend, rows, V, logits, tokens=tokens, tree=tree)
    g = splash_amd.CommandGraph()
    ops.Sampling.add_penalties(g, b["logits"], words, b["input_tokens"], b["tree_rows"], V, stride, lanes, penalties)
    ops.Sampling.add_verify(g, b, V, stride, lanes, [0.0] * 4)
    backend.run(g)
    seen = b["logits"].download(np.float32).reshape(rows, stride)
    selected = b["tokens"].download(np.uint32)
    for (first, n), (repetition, presence, frequency, row) in zip(lanes, penalties):
        want = orc.penalize(logits[first:first + n, :V], table[row], tokens[first:first + n], tree["ancestors"][first:first + n],
                            repetition, presence, frequency)
        assert seen[first:first + n, :V].tobytes() == want.tobytes(), first
        assert np.all(seen[first:first + n, V:] == 123.0)
        for r in range(n):
            assert selected[first + r] == orc.argmax(want[r])
    assert seen[:5].tobytes() == logits[:5].tobytes()
    assert orc.argmax(logits[24, :V]) == tokens[23] and selected[24] == 4000
    # the acceptance, then the count of what each penalized lane retained
    print("case sampling penalty count", flush=True)
    retained, accepted, mask = (backend.allocate_buffer(len(lanes) * 4) for _ in range(3))
    kept_tokens = backend.from_array(selected.copy())
    g = splash_amd.CommandGraph()
    ops.Sampling.add_acceptance(g, b["input_tokens"], b["tree_rows"], kept_tokens, retained, accepted, mask, lanes, [16] * 4)
    ops.Sampling.add_penalty_count(g, words, kept_tokens, retained, V, lanes, penalties)
    backend.run(g)
    counts, kept = retained.download(np.uint32), kept_tokens.download(np.uint32)
    want_table = table.copy()
    for (first, n), (_, _, _, row), count in zip(lanes[1:], penalties[1:], counts[1:]):
        assert 1 <= count <= n
        np.add.at(want_table[row], kept[first:first + count], 1)
    assert np.array_equal(words.download(np.uint32).reshape(4, V), want_table)
    assert np.array_equal(want_table[3], table[3])                    # the lane without penalties counts nothing
    # a token kept twice in one step is counted twice
    twice = backend.from_array(np.array([11, 11, 11], np.uint32))
    g = splash_amd.CommandGraph()
    ops.Sampling.add_penalty_count(g, words, twice, backend.from_array(np.array([3], np.uint32)), V, [(0, 3)], [(1.1, 0.0, 0.0, 3)])
    backend.run(g)
    assert words.download(np.uint32).reshape(4, V)[3, 11] == want_table[3, 11] + 3
    with pytest.raises(ValueError, match="repetition"):
        ops.Sampling.add_penalties(splash_amd.CommandGraph(), b["logits"], words, b["input_tokens"], b["tree_rows"], V, stride, lanes,
                                   [(0.0, 0.0, 0.0, 0)] * 4)
    with pytest.raises(ValueError, match="penalty words"):
        ops.Sampling.add_penalties(splash_amd.CommandGraph(), b["logits"], words, b["input_tokens"], b["tree_rows"], V, stride, lanes,
                                   [(1.5, 0.0, 0.0, 4)] * 4)


def test_thinking_cutoffs_rewrite_the_selections(backend):
    """decode_sample_end_thinking against the oracle over random chains and trees: lanes with and without a cutoff, ends
    longer than the block, cutoffs below the block, close and also-ends tokens among the drafts (few distinct tokens, so
    they occur), sentinels among the selections, and ends that wait for their masks. Then through add_verify, whose last
    dispatch it is: greedy rows select the argmax, the cutoff's rows the end."""
    from tests.test_oracle_sampling import random_tree
    print("case sampling thinking cutoff", flush=True)
    rng = np.random.default_rng(91)
    V, words = 300, (300 + 31) // 32
    for trial in range(30):
        lanes, first, trees = [], 0, []
        for _ in range(int(rng.integers(1, 9))):
            n = int(rng.integers(1, 17))
            lanes.append((first, n)); first += n
            trees.append(random_tree(rng, n) if trial % 2 else ops.chain_tree_rows([n]))
        rows = first
        tree = np.concatenate(trees)
        drafts = rng.integers(0, 6, rows).astype(np.uint32)
        picked = rng.integers(100, 200, rows).astype(np.uint32)
        picked[rng.random(rows) < 0.1] = ops.NO_TOKEN
        allowed = rng.random((rows, V)) < 0.4
        bits = np.zeros((rows, words * 32), dtype=np.uint8)
        bits[:, :V] = allowed
        mask = np.packbits(bits.reshape(rows, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(rows, words)
        cutoffs, specs = [], []
        for f, n in lanes:
            if rng.random() < 0.25:
                cutoffs.append(None); specs.append(None)
                continue
            spec = dict(row=int(rng.integers(0, 18)), end=[int(t) for t in rng.integers(0, 8, int(rng.integers(1, 17)))],
                        also_ends=int(rng.integers(0, 8)) if rng.random() < 0.5 else ops.NO_TOKEN, waits_for_mask=bool(rng.random() < 0.4))
            specs.append(spec)
            cutoffs.append(ops.Sampling.thinking_cutoff(**spec))
        tokens = backend.from_array(picked.copy())
        g = splash_amd.CommandGraph()
        ops.Sampling.add_thinking_cutoff(g, backend.from_array(drafts), backend.from_array(tree), tokens, V, lanes, cutoffs,
                                         token_mask=backend.from_array(mask), mask_words=words)
        backend.run(g)
        got = tokens.download(np.uint32)
        for (f, n), spec in zip(lanes, specs):
            want = picked[f:f + n]
            if spec is not None:
                admits = allowed[f:f + n, spec["end"][0]] if spec["waits_for_mask"] else None
                want = orc.thinking_cutoff(picked[f:f + n], drafts[f:f + n], tree[f:f + n], V, spec["row"], spec["end"], spec["also_ends"],
                                           admits=admits)
            assert np.array_equal(got[f:f + n], want), (trial, f, spec)
    # through add_verify: a greedy lane whose rows from depth 2 on end thinking
    rows, V = 6, 5000
    logits = (rng.standard_normal((rows, V)) * 2).astype(np.float32)
    chain = ops.chain_tree_rows([rows])
    b = sampling_buffers(backend, rows, V, logits, tokens=np.arange(rows, dtype=np.uint32) + 3000, tree=chain)
    g = splash_amd.CommandGraph()
    ops.Sampling.add_verify(g, b, V, V, [(0, rows)], [0.0])
    ops.Sampling.add_thinking_cutoff(g, b["input_tokens"], b["tree_rows"], b["tokens"], V, [(0, rows)],
                                     [ops.Sampling.thinking_cutoff(2, [11, 12])])
    backend.run(g)
    best = [orc.argmax(row) for row in logits]
    assert list(b["tokens"].download(np.uint32)) == best[:2] + [11, 12] + best[4:]
    with pytest.raises(ValueError, match="has an end"):
        ops.Sampling.add_thinking_cutoff(splash_amd.CommandGraph(), b["input_tokens"], b["tree_rows"], b["tokens"], V, [(0, rows)],
                                         [ops.Sampling.thinking_cutoff(2, [])])
    with pytest.raises(ValueError, match="constraint"):
        ops.Sampling.add_thinking_cutoff(splash_amd.CommandGraph(), b["input_tokens"], b["tree_rows"], b["tokens"], V, [(0, rows)],
                                         [ops.Sampling.thinking_cutoff(2, [5], waits_for_mask=True)])


def test_verify_rows_are_laid_out_from_the_trees(backend):
    """draft_verify_rows (sampling.metal:1799-1895) against the oracle, bit for bit: tokens, tree rows, lane rows and
    sources over random trees, caps, floors and tied estimates; and its outputs are what the acceptance walk reads."""
    print("case draft verify rows", flush=True)
    from tests.draft_case import grown_trees
    rng = np.random.default_rng(37)
    for trial in range(40):
        lanes = int(rng.integers(1, 9))
        tokens, trees, scores, sizes = grown_trees(rng, lanes, ties=trial % 3 == 0)
        lane_cap = int(rng.integers(1, 17))
        rows = int(rng.integers(lanes, lanes * lane_cap + 1))
        floor = float(rng.choice([0.0, 0.3, 0.7]))
        out = [backend.from_array(np.full(rows, 0xA5A5A5A5, np.uint32)), backend.from_array(np.zeros(rows, dtype=orc.TREE_DTYPE)),
               backend.from_array(np.zeros((lanes, 2), np.uint32)), backend.from_array(np.full(rows, 0xA5A5A5A5, np.uint32))]
        graph = splash_amd.CommandGraph()
        ops.DraftSelector.add_verify_rows(graph, backend.from_array(tokens), backend.from_array(trees), backend.from_array(scores),
                                          backend.from_array(sizes), *out, lanes, rows, lane_cap, floor)
        backend.run(graph)
        want = orc.draft_verify_rows(tokens, trees, scores, sizes, rows, lane_cap, floor)
        got = (out[0].download(np.uint32), out[1].download(np.uint8).view(orc.TREE_DTYPE), out[2].download(np.uint32).reshape(lanes, 2),
               out[3].download(np.uint32))
        for g, w in zip(got, want):
            assert np.array_equal(g, w), (trial, lanes, rows, lane_cap, floor)
    # the step's rows feed the acceptance walk as they are: every lane accepts the path its selections name
    lane_list = [(int(f), int(n)) for f, n in got[2]]
    selected = rng.integers(0, 50000, rows).astype(np.uint32)
    tb, ret, acc, mask = (backend.from_array(selected), backend.allocate_buffer(lanes * 4), backend.allocate_buffer(lanes * 4),
                          backend.allocate_buffer(lanes * 4))
    graph = splash_amd.CommandGraph()
    ops.Sampling.add_acceptance(graph, out[0], out[1], tb, ret, acc, mask, lane_list, [0xFFFFFFFF] * lanes, [0xFFFFFFFF] * 4)
    backend.run(graph)
    for i, (f, n) in enumerate(lane_list):
        kept, a, m = orc.accept_tree(got[1][f:f + n], got[0][f:f + n], selected[f:f + n])
        assert ret.download(np.uint32)[i] == len(kept) and acc.download(np.uint32)[i] == a and mask.download(np.uint32)[i] == m
    with pytest.raises(splash_amd.SplashError):
        ops.DraftSelector.add_verify_rows(graph, backend.from_array(tokens), backend.from_array(trees), backend.from_array(scores),
                                          backend.from_array(sizes), *out, lanes, lanes * lane_cap + 1, lane_cap, 0.0)


def test_verify_rows_in_slots(backend):
    """The slots layout against the oracle, bit for bit, and what makes it useful: the acceptance walk over a lane's whole
    slot (the shape a step is recorded for) keeps what the walk over the lane's own rows keeps."""
    print("case draft verify row slots", flush=True)
    from tests.draft_case import grown_trees
    rng = np.random.default_rng(38)
    for trial in range(30):
        lanes = int(rng.integers(1, 9))
        tokens, trees, scores, sizes = grown_trees(rng, lanes, ties=trial % 3 == 0)
        cap = int(rng.integers(1, 17))
        rows = lanes * cap
        floor = float(rng.choice([0.0, 0.3, 0.7]))
        out = [backend.from_array(np.full(rows, 0xA5A5A5A5, np.uint32)), backend.from_array(np.zeros(rows, dtype=orc.TREE_DTYPE)),
               backend.from_array(np.zeros((lanes, 2), np.uint32)), backend.from_array(np.full(rows, 0xA5A5A5A5, np.uint32))]
        graph = splash_amd.CommandGraph()
        ops.DraftSelector.add_verify_row_slots(graph, backend.from_array(tokens), backend.from_array(trees), backend.from_array(scores),
                                               backend.from_array(sizes), *out, lanes, cap, floor)
        backend.run(graph)
        want = orc.draft_verify_row_slots(tokens, trees, scores, sizes, cap, floor)
        got = (out[0].download(np.uint32), out[1].download(np.uint8).view(orc.TREE_DTYPE), out[2].download(np.uint32).reshape(lanes, 2),
               out[3].download(np.uint32))
        for g, w in zip(got, want):
            assert np.array_equal(g, w), (trial, lanes, cap, floor)
        selected = rng.integers(0, 40, rows).astype(np.uint32)
        tb, ret, acc, mask = (backend.from_array(selected), backend.allocate_buffer(lanes * 4), backend.allocate_buffer(lanes * 4),
                              backend.allocate_buffer(lanes * 4))
        graph = splash_amd.CommandGraph()
        ops.Sampling.add_acceptance(graph, out[0], out[1], tb, ret, acc, mask, [(l * cap, cap) for l in range(lanes)], [0xFFFFFFFF] * lanes,
                                    [0xFFFFFFFF] * 4)
        backend.run(graph)
        for lane in range(lanes):
            first, mine = int(got[2][lane][0]), int(got[2][lane][1])
            kept, a, m = orc.accept_tree(got[1][first:first + mine], got[0][first:first + mine], selected[first:first + mine])
            assert ret.download(np.uint32)[lane] == len(kept) and acc.download(np.uint32)[lane] == a and mask.download(np.uint32)[lane] == m
            assert np.array_equal(tb.download(np.uint32)[first:first + len(kept)], kept)


def test_draft_candidates_and_edges(backend):
    """draft_select_top16_sharded and draft_select_edges (sampling.metal:1099-1356) against the oracle: candidates and
    their logits bit for bit (ties, signed zeros, short rows, rows of few finite columns, a draft vocabulary that skips a
    range, a vocabulary of several shards with a ragged last one); edge scores to the fp32 rounding of a 256-term sum,
    2^-20 of the terms' largest magnitude times 256, the order of the sum being the kernel's own."""
    print("case draft candidates and edges", flush=True)
    from tests.draft_case import bf16_bits, bf16_values, proposal_logits
    rng = np.random.default_rng(73)
    cases = [("plain", 151936, 151936, 151936, 1), ("plain", 32000, 20000, 139936, 8), ("tied", 20000, 8000, 9000, 3),
             ("sparse", 40000, 40000, 40000, 2), ("plain", 9, 4, 10, 2), ("tied", 8193, 8193, 8193, 1), ("sparse", 300000, 300000, 300000, 1)]
    for kind, columns, leading, trailing, lanes in cases:
        print("  ", kind, columns, lanes, flush=True)
        vocabulary = columns - leading + trailing
        logits = proposal_logits(rng, lanes, columns, kind)
        codebook_rows = min(vocabulary, 4096)      # random rows, repeated up to the vocabulary
        hidden, before, after = (bf16_bits(rng.standard_normal(shape)) for shape in
                                 ((lanes * 8, 256), (codebook_rows, 256), (codebook_rows, 256)))
        anchors = rng.integers(0, vocabulary, lanes).astype(np.uint32)
        out = [backend.from_array(np.full((lanes * 7, 16), 0xA5A5A5A5, np.uint32)), backend.from_array(np.zeros((lanes * 7, 16), np.float32)),
               backend.from_array(np.zeros((lanes * 7, 16, 16), np.float32))]
        scratch = backend.allocate_buffer(ops.DraftSelector.candidate_scratch_bytes(lanes, columns))
        graph = splash_amd.CommandGraph()
        ops.DraftSelector.add_candidates(graph, backend.from_array(logits), backend.from_array(hidden), scratch, *out,
                                         backend.from_array(_padded(before, vocabulary)), backend.from_array(_padded(after, vocabulary)),
                                         leading, trailing, vocabulary, list(anchors))
        backend.run(graph)
        candidates, unary = out[0].download(np.uint32).reshape(-1, 16), out[1].download(np.float32).reshape(-1, 16)
        want = orc.draft_candidates(logits, lanes, leading, trailing)
        assert np.array_equal(candidates, want[0]), (kind, columns)
        assert np.array_equal(unary.view(np.uint32), want[1].view(np.uint32)), (kind, columns)
        edges = out[2].download(np.float32).reshape(-1, 16, 16)
        want_edges = orc.draft_edges(want[0], anchors, vocabulary, hidden, _padded(before, vocabulary), _padded(after, vocabulary))
        scale = np.abs(bf16_values(hidden)).max() * np.abs(bf16_values(before)).max() * np.abs(bf16_values(after)).max() * 256
        assert np.abs(edges - want_edges).max() <= 2.0 ** -20 * scale, (kind, columns)
        assert np.abs(want_edges).max() > 10
    with pytest.raises(splash_amd.SplashError):      # a draft's tokens lie in its vocabulary
        ops.DraftSelector.add_candidates(graph, backend.from_array(logits), backend.from_array(hidden), scratch, *out,
                                         backend.from_array(before), backend.from_array(after), 10, 5, 8193, [0])
    with pytest.raises(splash_amd.SplashError):      # more columns than the selector's shards hold
        ops.DraftSelector.add_candidates(graph, backend.from_array(logits), backend.from_array(hidden), scratch, *out,
                                         backend.from_array(before), backend.from_array(after), 600000, 600000, 600000, [0])


def _padded(codebook, vocabulary):
    """A codebook of `vocabulary` rows whose rows past the given ones repeat them."""
    rows = codebook.shape[0]
    return codebook if rows == vocabulary else codebook[np.arange(vocabulary) % rows]
