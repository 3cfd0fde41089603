"""The oracle's acceptance functions against brute force, the enumerated selection law and statistics (CPU)."""
import numpy as np
import pytest

from tests import oracle as orc


def test_argmax_brute_force_ties_and_unselectable():
    rng = np.random.default_rng(0)
    for _ in range(200):
        n = int(rng.integers(1, 40))
        x = rng.integers(-3, 4, n).astype(np.float32)           # many ties
        x[rng.random(n) < 0.2] = -np.inf
        x[rng.random(n) < 0.1] = np.nan
        ok = np.isfinite(x)
        want = orc.NO_TOKEN if not ok.any() else int(np.flatnonzero(ok & (x == x[ok].max()))[0])   # lowest id of the max
        assert orc.argmax(x) == want
    assert orc.argmax(np.array([np.inf, 1.0], dtype=np.float32)) == 0    # +inf is selectable


def walk(tree, tokens, selected, remaining, stops):
    """An independent restatement of the acceptance walk (sampling.metal:2044-2083), recursive on children."""
    rows = len(tree)
    path = [0]
    while True:
        row = path[-1]
        nxt = [c for c in range(row + 1, rows) if tree[c]["parent"] == row and tokens[c] == selected[row]]
        if not nxt:
            break
        path.append(nxt[0])
    accepted = len(path) - 1
    kept = min(accepted + 1, max(remaining, 1))
    out = []
    for i in range(kept):
        out.append(int(selected[path[i]]))
        if out[-1] in stops:
            kept = i + 1
            break
    return out[:kept], min(accepted, kept), int(tree[path[kept - 1]]["ancestors"])


def random_tree(rng, rows):
    tree = np.zeros(rows, dtype=np.dtype([("ancestors", "<u4"), ("parent", "<u2"), ("depth", "<u2")]))
    tree[0] = (1, 0xFFFF, 0)
    for r in range(1, rows):
        parent = int(rng.integers(0, r))
        tree[r] = (int(tree[parent]["ancestors"]) | (1 << r), parent, int(tree[parent]["depth"]) + 1)
    return tree


def test_accept_tree_fuzz_against_independent_walk():
    rng = np.random.default_rng(1)
    for _ in range(500):
        rows = int(rng.integers(1, 17))
        tree = random_tree(rng, rows)
        tokens = rng.integers(0, 4, rows).astype(np.uint32)
        selected = rng.integers(0, 4, rows).astype(np.uint32)
        remaining = int(rng.integers(1, 20))
        stops = [3] if rng.random() < 0.3 else []
        got = orc.accept_tree(tree, tokens, selected, remaining, stops)
        want = walk(tree, tokens, selected, remaining, stops)
        assert list(got[0]) == want[0] and got[1] == want[1] and got[2] == want[2]


def test_chain_acceptance_closed_form():
    """A chain keeps the longest prefix whose drafted tokens equal the selections, plus the bonus token."""
    rows = 16
    tree = np.zeros(rows, dtype=np.dtype([("ancestors", "<u4"), ("parent", "<u2"), ("depth", "<u2")]))
    for r in range(rows):
        tree[r] = ((2 << r) - 1, r - 1 if r else 0xFFFF, r)
    selected = np.arange(100, 100 + rows, dtype=np.uint32)
    for match in range(rows):
        tokens = np.zeros(rows, dtype=np.uint32)
        tokens[1:match + 1] = selected[:match]          # rows 1..match were drafted right
        tokens[match + 1:] = 7
        kept, accepted, mask = orc.accept_tree(tree, tokens, selected)
        assert accepted == match and list(kept) == list(selected[:match + 1]) and mask == (2 << match) - 1


def test_rejection_rule_enumerated_law_equals_target():
    """target_sampling_metal_test.mm:2602-2631: the selection law of test-then-residual equals softmax(logits / T)."""
    rng = np.random.default_rng(2)
    for V in (3, 17, 300):
        x = (rng.standard_normal(V) * 3).astype(np.float32)
        x[rng.random(V) < 0.1] = -np.inf
        if not np.isfinite(x).any():
            x[0] = 0
        q = np.exp(rng.standard_normal(V) * 2); q = (q / q.sum()).astype(np.float32)
        T = float(np.float32(0.7))    # the temperature the fp32 interface carries
        p = np.where(np.isfinite(x), np.exp((x.astype(np.float64) - x[np.isfinite(x)].max()) / T), 0); p /= p.sum()
        law = orc.rejection_law(x, T, q)
        assert np.abs(law - p).max() < 1e-12 and abs(law.sum() - 1) < 1e-9


def test_rejection_row_follows_the_target_distribution():
    """target_sampling_metal_test.mm:3019 followsDistribution: chi-square of the row's selections over seeds."""
    rng = np.random.default_rng(3)
    V, T, draws = 12, 0.7, 20000
    x = (rng.standard_normal(V) * 2).astype(np.float32)
    q = np.exp(rng.standard_normal(V)); q = (q / q.sum()).astype(np.float32)
    p = np.exp((x.astype(np.float64) - x.max()) / T); p /= p.sum()
    counts = np.zeros(V)
    children = rng.choice(V, size=draws, p=q / q.sum())
    u = rng.random((draws, 2)).astype(np.float32)
    for i in range(draws):
        tok, accepted, _ = orc.rejection_row(x, T, q, int(children[i]), float(u[i, 0]), float(u[i, 1]))
        counts[tok] += 1
    chi2 = ((counts - draws * p) ** 2 / (draws * p)).sum()
    assert chi2 < 40, chi2      # 11 degrees of freedom: P(chi2 > 40) < 1e-4
    # without a child the row is a plain draw from p
    counts = np.zeros(V)
    for i in range(draws):
        tok, _, _ = orc.rejection_row(x, T, None, orc.NO_TOKEN, 0.0, float(u[i, 1]))
        counts[tok] += 1
    assert ((counts - draws * p) ** 2 / (draws * p)).sum() < 40


def test_rejection_row_accepts_iff_uq_below_p():
    x = np.array([0.0, 1.0, 2.0, -1.0], dtype=np.float32)
    q = np.array([0.1, 0.2, 0.3, 0.4], dtype=np.float32)
    p = np.exp(x.astype(np.float64) / 0.7); p /= p.sum()
    for child in range(4):
        for u in (0.01, 0.3, 0.6, 0.99):
            tok, accepted, close = orc.rejection_row(x, 0.7, q, child, u, 0.5)
            if close > 1e-5:
                assert accepted == (u * q[child] < p[child])
                assert (tok == child) if accepted else (p[tok] > q[tok])   # a redraw comes from max(p - q, 0)


def brute_force_end(x, T, min_p, top_k, top_p):
    """distribution_end (sampling.metal:603-670) from its description alone, in fp64: the kept token ids, in order."""
    finite = np.isfinite(x) | (x == np.inf)
    ids = np.nonzero(finite)[0]
    keys = orc.logit_key(x[ids]).astype(np.int64)
    order = ids[np.lexsort((ids, -keys))]
    mx = x[order[0]]
    w = np.exp((x[order].astype(np.float64) - float(mx)) / T)
    keep = len(order)
    if min_p > 0:
        threshold = np.float32(min(np.float32(mx) + np.float32(T) * np.float32(np.log(np.float32(min_p))), np.float32(mx)))
        keep = int((orc.logit_key(x[order]) >= orc.logit_key(np.array([threshold], np.float32))[0]).sum())
    if top_k and top_k < keep:
        keep = top_k
    mass = w[:keep].sum()
    margin = 1.0
    if top_p < 1:
        cumulative = np.cumsum(w[:keep])
        target = float(np.float32(top_p) * np.float32(mass))
        crossing = np.nonzero(cumulative > target)[0]
        if len(crossing):
            keep = int(crossing[0]) + 1
            margin = min(abs(cumulative[keep - 1] - target), abs(cumulative[keep - 2] - target) if keep > 1 else 1.0) / target
    return order[:keep], margin


@pytest.mark.parametrize("seed", range(6))
def test_distribution_end_against_a_sort(seed):
    """min_p, then top_k, then top_p, in the order of the logits with ties to the smaller id: the oracle's end keeps
    exactly the tokens a sort keeps, also where whole runs of tokens share a logit."""
    rng = np.random.default_rng(100 + seed)
    V = int(rng.integers(5, 3000))
    x = (rng.standard_normal(V) * 2.5).astype(np.float32)
    if seed % 2:
        x = (np.round(x * 2) / 2).astype(np.float32)      # many ties
    x[rng.random(V) < 0.05] = -np.inf
    x[0] = max(x[0], np.float32(0))
    T = float(np.float32(rng.uniform(0.3, 1.5)))
    for min_p, top_k, top_p in [(0.0, 0, 1.0), (0.05, 0, 1.0), (0.0, 7, 1.0), (0.0, 0, 0.9), (0.02, 40, 0.8), (0.0, V + 5, 0.5), (0.3, 2, 0.99)]:
        min_p, top_p = float(np.float32(min_p)), float(np.float32(top_p))
        kept, margin = brute_force_end(x, T, min_p, top_k, top_p)
        key, last, mass, count, closeness = orc.distribution_end(x, T, min_p, top_k, top_p)
        if margin < 1e-6:
            continue
        assert count == len(kept), (min_p, top_k, top_p)
        keys, ids = orc.logit_key(x), np.arange(V)
        stays = np.isfinite(x) & ((keys > key) | ((keys == key) & (ids <= last)))
        assert np.array_equal(np.sort(kept), np.nonzero(stays)[0])
        w = np.exp((x[kept].astype(np.float64) - float(x[kept[0]])) / T)
        assert abs(mass - w.sum()) <= 1e-5 * w.sum()


def test_truncated_rejection_law_is_the_renormalized_kept_distribution():
    """The selection law of test-then-residual over a cut distribution is that distribution renormalized, whatever the
    draft proposes (also tokens outside it), and a row's draw never leaves it."""
    rng = np.random.default_rng(7)
    for V, policy in ((14, (0.7, 0.0, 5, 1.0)), (40, (1.1, 0.05, 0, 0.9)), (300, (0.7, 0.01, 50, 0.7))):
        x = (rng.standard_normal(V) * 3).astype(np.float32)
        q = np.exp(rng.standard_normal(V) * 2); q = (q / q.sum()).astype(np.float32)
        T = float(np.float32(policy[0]))
        kept, _ = brute_force_end(x, T, float(np.float32(policy[1])), policy[2], float(np.float32(policy[3])))
        p = np.zeros(V)
        p[kept] = np.exp((x[kept].astype(np.float64) - float(x.max())) / T)
        p /= p.sum()
        law = orc.rejection_law_policy(x, policy, q)
        assert np.abs(law - p).max() < 1e-12
        for _ in range(200):
            child = int(rng.integers(0, V))
            tok, accepted, _ = orc.rejection_row_policy(x, policy, q, child, float(rng.random()), float(rng.random()))
            assert p[tok] > 0 and (not accepted or tok == child)


def test_verify_rows_layout_against_a_sort_and_a_recursive_preorder():
    from tests.draft_case import grown_trees, layout_by_sorting
    rng = np.random.default_rng(29)
    for trial in range(200):
        lanes = int(rng.integers(1, 9))
        tokens, trees, scores, sizes = grown_trees(rng, lanes, ties=trial % 3 == 0)
        lane_cap = int(rng.integers(1, 17))
        rows = int(rng.integers(lanes, lanes * lane_cap + 1))
        floor = float(rng.choice([0.0, 0.3, 0.7]))
        got = orc.draft_verify_rows(tokens, trees, scores, sizes, rows, lane_cap, floor)
        want = layout_by_sorting(tokens, trees, scores, sizes, rows, lane_cap, floor)
        for g, w in zip(got, want):
            assert np.array_equal(g, w), (trial, lanes, rows, lane_cap, floor)
        # what the verify path relies on: a lane's first row is its anchor, parents precede children, a row's ancestors
        # are its parent's and itself, and the rows of no lane are on no path
        _, tree, lane_rows, sources = got
        for first, count in lane_rows:
            assert count >= 1 and int(tree[first]["ancestors"]) == 1 and int(tree[first]["parent"]) == 0xFFFF
            for at in range(1, count):
                up = int(tree[first + at]["parent"])
                assert up < at and int(tree[first + at]["ancestors"]) == int(tree[first + up]["ancestors"]) | (1 << at)
                assert int(tree[first + at]["depth"]) == int(tree[first + up]["depth"]) + 1
        used = int(lane_rows[-1][0] + lane_rows[-1][1])
        assert np.all(sources[used:] == orc.NO_TOKEN) and np.all(tree[used:]["ancestors"] == 0)


def test_verify_rows_in_slots_are_the_packed_rows_moved_and_inert_rows():
    """The slots layout against the packed one (pinned above) of the same trees with every lane free to take its cap:
    a lane's rows moved to its slot as they are, and the rest of the slot rows that the step cannot mistake for drafted
    ones -- the acceptance walk never follows them whatever the target selects, and they lie on no other row's path."""
    from tests.draft_case import grown_trees
    rng = np.random.default_rng(30)
    for trial in range(100):
        lanes = int(rng.integers(1, 9))
        tokens, trees, scores, sizes = grown_trees(rng, lanes, ties=trial % 3 == 0)
        cap = int(rng.integers(1, 17))
        floor = float(rng.choice([0.0, 0.3, 0.7]))
        got_tokens, got_tree, got_lanes, got_sources = orc.draft_verify_row_slots(tokens, trees, scores, sizes, cap, floor)
        p_tokens, p_tree, p_lanes, p_sources = orc.draft_verify_rows(tokens, trees, scores, sizes, lanes * cap, cap, floor)
        for lane in range(lanes):
            first, mine = lane * cap, int(p_lanes[lane][1])
            assert list(got_lanes[lane]) == [first, mine]
            at = int(p_lanes[lane][0])
            assert np.array_equal(got_tokens[first:first + mine], p_tokens[at:at + mine])
            assert np.array_equal(got_tree[first:first + mine], p_tree[at:at + mine]) and np.array_equal(got_sources[first:first + mine], p_sources[at:at + mine])
            pad = slice(first + mine, first + cap)
            assert np.all(got_tokens[pad] == orc.NO_TOKEN) and np.all(got_sources[pad] == orc.NO_TOKEN)
            assert np.all(got_tree[pad]["ancestors"] == (1 << np.arange(mine, cap)).astype(np.uint32))
            # no drafted row's path names an inert row
            assert not np.any(got_tree[first:first + mine]["ancestors"] >> mine)
            # the walk over the whole slot keeps what the walk over the lane's own rows keeps, whatever is selected
            selected = rng.integers(0, 50, cap).astype(np.uint32)
            own = orc.accept_tree(got_tree[first:first + mine], got_tokens[first:first + mine], selected[:mine])
            whole = orc.accept_tree(got_tree[first:first + cap], got_tokens[first:first + cap], selected)
            assert np.array_equal(own[0], whole[0]) and own[1:] == whole[1:]


def test_draft_candidates_are_the_sorted_heads_of_the_rows():
    """orc_draft_candidates against a lexicographic sort (logit descending, column ascending): plain rows, rows of few
    distinct values with signed zeros, rows with fewer finite columns than candidates, fewer columns than candidates, and a
    draft vocabulary that skips a range of the target's tokens."""
    from tests.draft_case import candidates_by_sorting, proposal_logits
    rng = np.random.default_rng(71)
    for kind, columns, leading, trailing in [("plain", 5000, 5000, 5000), ("tied", 3000, 1000, 4000), ("sparse", 20000, 12000, 13000),
                                             ("plain", 9, 4, 10), ("tied", 40, 0, 7)]:
        lanes = int(rng.integers(1, 4))
        logits = proposal_logits(rng, lanes, columns, kind)
        got = orc.draft_candidates(logits, lanes, leading, trailing)
        want = candidates_by_sorting(logits, lanes, leading, trailing)
        assert np.array_equal(got[0], want[0]), kind
        assert np.array_equal(got[1].view(np.uint32), want[1].view(np.uint32)), kind   # signed zeros as the row holds them


def test_draft_edges_are_the_trilinear_sums():
    """orc_draft_edges against the fp64 einsum of the decoded factors: each of the 256 products is rounded to fp32 once or
    twice (2^-23 relative each), so the sums agree to 2^-22 of the sum of the products' magnitudes; position 0 scores its
    anchor alone and a token past the vocabulary reads its last row."""
    from tests.draft_case import bf16_bits, bf16_values, edges_by_einsum
    rng = np.random.default_rng(72)
    lanes, vocabulary = 2, 300
    hidden, before, after = (bf16_bits(rng.standard_normal(shape)) for shape in ((lanes * 8, 256), (vocabulary, 256), (vocabulary, 256)))
    candidates = rng.integers(0, vocabulary, (lanes * 7, 16)).astype(np.uint32)
    candidates[3, 5] = 0xFFFFFFFF
    anchors = np.array([7, 299], np.uint32)
    got = orc.draft_edges(candidates, anchors, vocabulary, hidden, before, after)
    want = edges_by_einsum(candidates, anchors, vocabulary, hidden, before, after)
    written = ~np.isnan(want)
    assert written.sum() == lanes * (16 + 6 * 256) and not got[~written].any()
    scale = np.abs(bf16_values(hidden)).max() * np.abs(bf16_values(before)).max() * np.abs(bf16_values(after)).max() * 256
    assert np.abs(got[written] - want[written]).max() <= 2.0 ** -22 * scale
    assert np.abs(want[written]).max() > 10      # the scores are far from zero: a dropped factor would show


# ------------------------------------------------------------------ a tree block's sampled rows (sampling.metal:697-880)
def _dirichlet(rng, n, zeros):
    v = -np.log(0.5 * (rng.random(n) + 1.0) + 1e-9)
    v[rng.integers(0, n, zeros)] = 0.0
    return v / v.sum()


def test_children_law_is_the_target_distribution_whatever_the_draft():
    """The proof harness of the reference (target_sampling_metal_test.mm:2602-2631): over 300 random targets and drafts of
    one to four children, some candidates outside the target's support and some of its mass outside the candidates, the
    enumerated law of the selection is the target's to 1e-12. A wrong residual, a missing renormalization of p or of
    the draft's rest, or a draw past the candidates that forgets their mass all break it."""
    rng = np.random.default_rng(0x7272)
    worst = 0.0
    for trial in range(300):
        p = _dirichlet(rng, 24, trial % 5)
        ids = rng.permutation(24)[:16].astype(np.uint32)
        q = _dirichlet(rng, 16, trial % 7)
        law = orc.children_law(p, ids, q, 1 + trial % 4)
        worst = max(worst, float(np.abs(law - p).max()))
    assert worst < 1e-12, worst
    # candidates past the vocabulary (a draft row of fewer comparable logits lists 0xffffffff) weigh nothing
    p = _dirichlet(rng, 10, 0)
    ids = np.concatenate([rng.permutation(10)[:6], np.full(10, 0xFFFFFFFF)]).astype(np.uint32)
    q = np.concatenate([_dirichlet(rng, 6, 0), np.zeros(10)])
    assert np.abs(orc.children_law(p, ids, q, 3) - p).max() < 1e-12


def _gumbel_draws(rng, q, count):
    keys = [(np.log(q[i]) - np.log(-np.log(rng.random() + 1e-300)), i) for i in range(len(q)) if q[i] > 0]
    return [i for _, i in sorted(keys, reverse=True)[:count]]


def test_children_row_follows_the_target_distribution():
    """The row itself over many seeds (the reference's followsDistribution, target_sampling_metal_test.mm:3019): children
    drawn without replacement from q, uniform tests and draws; the selected tokens' frequencies are the target's."""
    rng = np.random.default_rng(9)
    V, T, N = 40, 0.8, 30000
    logits = (rng.standard_normal(V) * 1.5).astype(np.float32)
    logits[[3, 17]] = -np.inf
    p = np.where(np.isfinite(logits), np.exp((logits.astype(np.float64) - logits[np.isfinite(logits)].max()) / T), 0)
    p /= p.sum()
    ids = rng.permutation(V)[:16].astype(np.uint32)
    q = _dirichlet(rng, 16, 2).astype(np.float32)
    for draws_n in (1, 4):
        counts = np.zeros(V)
        for _ in range(N):
            draws = _gumbel_draws(rng, q.astype(np.float64), draws_n)
            token, _ = orc.children_row(logits, (T, 0.0, 0, 1.0), ids, q, draws, rng.random(4).astype(np.float32), float(rng.random()))
            counts[token] += 1
        freq = counts / N
        assert np.all(np.abs(freq - p) <= 4 * np.sqrt(p * (1 - p) / N) + 5e-4), (draws_n, np.abs(freq - p).max())
        assert counts[3] == 0 and counts[17] == 0


def test_children_row_decisions_at_their_thresholds():
    rng = np.random.default_rng(10)
    V, T = 64, 0.7
    logits = (rng.standard_normal(V) * 2).astype(np.float32)
    w = np.exp((logits.astype(np.float64) - logits.max()) / T)
    p = w / w.sum()
    ids = np.arange(8, 24).astype(np.uint32)
    q = np.full(16, 1 / 16, np.float32)
    policy = (T, 0.0, 0, 1.0)
    # a child is selected iff u q < p: just below and just above the threshold p / q
    c = 5
    threshold = p[ids[c]] / q[c]
    if threshold < 1:
        assert orc.children_row(logits, policy, ids, q, [c], [np.float32(threshold * 0.999)], 0.5)[0] == ids[c]
        assert orc.children_row(logits, policy, ids, q, [c], [np.float32(min(threshold * 1.001, 0.99999))], 0.5)[0] != ids[c] or threshold * 1.001 >= 1
    assert orc.children_row(logits, policy, ids, q, [c], [0.0], 0.5)[0] == ids[c]                 # u = 0 always accepts a possible child
    # a second child is tested after the first is rejected, against the residual: with q concentrated on the first child
    # (q0 = 1 - eps), its rejection leaves p almost untouched elsewhere and the draft's rest uniform over the others
    q2 = np.full(16, 1e-3 / 15, np.float32); q2[0] = 1 - 1e-3
    token, _ = orc.children_row(logits, policy, ids, q2, [0, 7], [0.999999, 0.0], 0.5)
    assert token == ids[7]
    # no children: the row draws from its whole distribution, exactly as the one-child rule's row without a child does
    for u in (0.0, 0.3, 0.77, 0.999):
        assert orc.children_row(logits, policy, ids, q, [], [], u)[0] == orc.rejection_row(logits, T, None, orc.NO_TOKEN, 0.0, u)[0]
    # every child rejected and all of the target's mass on the candidates' complement: the draw lands outside them
    far = np.full(V, -np.inf, np.float32); far[[40, 50]] = [0.0, 1.0]
    token, _ = orc.children_row(far, policy, ids, q, [1, 2, 3, 4], [0.5] * 4, 0.99)
    assert token in (40, 50)
    # the draw over the candidates walks them in index order: with the mass on candidates only, u_row picks by cumulative p
    only = np.full(V, -np.inf, np.float32); only[ids[2]] = 0.0; only[ids[9]] = 0.0
    qz = np.zeros(16, np.float32); qz[0] = 1.0                                      # the drawn child has no target mass: rejected
    assert orc.children_row(only, policy, ids, qz, [0], [0.5], 0.25)[0] == ids[2]
    assert orc.children_row(only, policy, ids, qz, [0], [0.5], 0.75)[0] == ids[9]


def test_penalties_closed_forms():
    """orc_penalize against what the definition fixes (PenaltyReference.hpp:27-40; sampling.metal:1008-1050), case by
    case in float32 arithmetic: untouched tokens bitwise, a prompt token's single product, a count's single difference,
    saturation instead of infinity, unselectable logits, and which rows of a chain and of a forked tree count a draft
    token. Each case would fail for a dropped term, a swapped multiply / divide, a row counting its siblings or the
    anchor counted twice."""
    f32 = np.float32
    V = 64
    rng = np.random.default_rng(31)
    base = (rng.standard_normal((4, V)) * 3).astype(np.float32)
    chain = np.array([(2 << r) - 1 for r in range(4)], np.uint32)
    tokens = np.array([5, 9, 9, 12], np.uint32)            # the anchor 5, then drafts 9, 9, 12
    words = np.zeros(V, np.uint32)
    # defaults change nothing, whatever the table holds
    words[[3, 5, 7]] = [0x80000000, 2, 0x80000001]
    assert orc.penalize(base, words, tokens, chain).tobytes() == base.tobytes()
    # repetition alone: prompt-only token 3, output token 5 (count 2), both (7), and drafted tokens by row
    rep = f32(1.3)
    out = orc.penalize(base, words, tokens, chain, repetition=rep)
    scaled = lambda x: x * (f32(1.0) / rep) if x > 0 else x * rep
    for r in range(4):
        for t in (3, 5, 7):
            assert out[r, t] == scaled(base[r, t])
        # row r's context holds drafts 1..r: token 9 from row 1 on, token 12 at row 3 only
        assert out[r, 9] == (scaled(base[r, 9]) if r >= 1 else base[r, 9])
        assert out[r, 12] == (scaled(base[r, 12]) if r >= 3 else base[r, 12])
        untouched = np.setdiff1d(np.arange(V), [3, 5, 7, 9, 12])
        assert out[r, untouched].tobytes() == base[r, untouched].tobytes()
    # the sign decides divide or multiply: a positive logit shrinks, a negative one grows in magnitude, zero stays zero
    probe = np.zeros((1, V), np.float32); probe[0, 3] = 2.0; probe[0, 7] = -2.0
    out = orc.penalize(probe, words, tokens[:1], chain[:1], repetition=2.0)
    assert (out[0, 3], out[0, 7], out[0, 5]) == (1.0, -4.0, 0.0)
    # presence and frequency: only counted tokens (the prompt-only token 3 is not), by presence + frequency * count
    presence, frequency = f32(0.7), f32(0.25)
    out = orc.penalize(base, words, tokens, chain, presence=presence, frequency=frequency)
    for r in range(4):
        assert out[r, 3] == base[r, 3]
        assert out[r, 5] == base[r, 5] - (frequency * f32(2) + presence)       # the anchor is in the table, never added again
        assert out[r, 7] == base[r, 7] - (frequency * f32(1) + presence)
        drafted9 = min(r, 2)                                                   # rows 1 and 2 both hold token 9
        assert out[r, 9] == (base[r, 9] - (frequency * f32(drafted9) + presence) if drafted9 else base[r, 9])
    # all three at once: scale first, then subtract
    out = orc.penalize(base, words, tokens, chain, repetition=rep, presence=presence, frequency=frequency)
    assert out[2, 7] == scaled(base[2, 7]) - (frequency * f32(1) + presence)
    # a forked tree: rows 1 and 2 are siblings under the anchor, row 3 under row 2: a row counts its own path only
    tree = np.array([0b0001, 0b0011, 0b0101, 0b1101], np.uint32)
    forked = np.array([5, 20, 21, 20], np.uint32)
    out = orc.penalize(base, np.zeros(V, np.uint32), forked, tree, presence=1.0)
    assert [out[r, 20] == base[r, 20] - f32(1) for r in range(4)] == [False, True, False, True]
    assert [out[r, 21] == base[r, 21] - f32(1) for r in range(4)] == [False, False, True, True]
    assert [out[r, 20] == base[r, 20] for r in range(4)] == [True, False, True, False]
    # the anchor's own token drafted again further down counts there
    again = np.array([5, 5], np.uint32)
    out = orc.penalize(base[:2], np.zeros(V, np.uint32), again, chain[:2], presence=1.0)
    assert out[0, 5] == base[0, 5] and out[1, 5] == base[1, 5] - f32(1)
    # saturation and the unselectable
    big = np.zeros((1, V), np.float32)
    big[0, 3] = np.finfo(np.float32).max; big[0, 7] = -np.finfo(np.float32).max; big[0, 5] = np.inf
    edge_words = np.zeros(V, np.uint32); edge_words[[3, 5, 7, 8, 9]] = [0x80000000, 1, 1, 1, 1]
    big[0, 8] = -np.inf; big[0, 9] = np.nan
    out = orc.penalize(big, edge_words, tokens[:1], chain[:1], repetition=0.5, presence=1.0)
    assert out[0, 3] == np.finfo(np.float32).max          # max / 0.5 saturates
    assert out[0, 7] == -np.finfo(np.float32).max * f32(0.5) - f32(1)
    assert out[0, 5] == np.finfo(np.float32).max          # +infinity becomes the largest float: still selectable, never infinite
    assert out[0, 8] == -np.inf and np.isnan(out[0, 9])
    # a repetition so small that its inverse overflows: the inverse saturates, the product does too
    out = orc.penalize(probe, words, tokens[:1], chain[:1], repetition=1e-39)
    assert out[0, 3] == np.finfo(np.float32).max


def tree_of(parents):
    tree = np.zeros(len(parents), dtype=orc.TREE_DTYPE)
    for r, parent in enumerate(parents):
        tree[r] = ((1 << r) | (0 if parent is None else int(tree[parent]["ancestors"])), 0xFFFF if parent is None else parent,
                   0 if parent is None else int(tree[parent]["depth"]) + 1)
    return tree


def test_thinking_cutoff_hand_worked():
    """orc_thinking_cutoff against cases worked by hand from its definition (ThinkingCutoffParams, abi/Sampling.h:147-175
    in the reference): which rows take which end token, the rows past the end, an end that a draft token on the row's own
    path already made (at or above the cut, never the anchor's, never a sibling's), the sentinel, and the later start of an
    end that waits for its mask. Each would fail for an off-by-one in the cut, the depth or the count."""
    V = 1000
    chain = tree_of([None, 0, 1, 2, 3, 4])
    drafts = np.array([50, 51, 52, 53, 54, 55], np.uint32)
    picked = np.array([100, 101, 102, 103, 104, 105], np.uint32)
    cut = lambda **kw: list(orc.thinking_cutoff(picked, kw.pop("drafts", drafts), kw.pop("tree", chain), V, **kw))
    assert cut(row=2, end=[7, 8, 9]) == [100, 101, 7, 8, 9, 105]
    assert cut(row=0, end=[7]) == [7, 101, 102, 103, 104, 105]
    assert cut(row=4, end=[7, 8, 9, 10, 11, 12]) == [100, 101, 102, 103, 7, 8]           # as many as the block holds
    assert cut(row=6, end=[7]) == list(picked) and cut(row=40, end=[7]) == list(picked)  # a cutoff below the block
    # thinking that the draft ended at or above the cut stays ended: the close token (the end's last) or also_ends
    with_close = lambda at: np.array([9 if i == at else d for i, d in enumerate(drafts)], np.uint32)
    assert cut(row=2, end=[7, 8, 9], drafts=with_close(1)) == list(picked)
    assert cut(row=2, end=[7, 8, 9], drafts=with_close(2)) == list(picked)               # at the cut counts
    assert cut(row=2, end=[7, 8, 9], drafts=with_close(3)) == [100, 101, 7, 8, 9, 105]   # below the cut does not
    assert cut(row=2, end=[7, 8, 9], drafts=with_close(0)) == [100, 101, 7, 8, 9, 105]   # the anchor is no draft token
    assert cut(row=2, end=[7, 8, 9], also_ends=51) == list(picked)
    assert cut(row=2, end=[7, 8, 9], also_ends=54) == [100, 101, 7, 8, 9, 105]
    middle = np.array([50, 51, 8, 53, 54, 55], np.uint32)                                # the end's middle token closes nothing
    assert cut(row=2, end=[7, 8, 9], drafts=middle) == [100, 101, 7, 8, 9, 105]
    # a row with no selectable logit keeps its sentinel; a token outside the vocabulary likewise
    holes = np.array([100, 101, 102, orc.NO_TOKEN, V, 105], np.uint32)
    assert list(orc.thinking_cutoff(holes, drafts, chain, V, 2, [7, 8, 9])) == [100, 101, 7, orc.NO_TOKEN, V, 105]
    # a tree: depths 0 1 1 2 2 2 3; every path is cut on its own
    tree = tree_of([None, 0, 0, 1, 2, 2, 4])
    seven = np.arange(100, 107).astype(np.uint32)
    tdrafts = np.array([50, 51, 52, 53, 54, 55, 56], np.uint32)
    assert list(orc.thinking_cutoff(seven, tdrafts, tree, V, 1, [7, 8])) == [100, 7, 7, 8, 8, 8, 106]
    closed = tdrafts.copy(); closed[1] = 8                                               # row 1 drafted the close token
    assert list(orc.thinking_cutoff(seven, closed, tree, V, 1, [7, 8])) == [100, 101, 7, 103, 8, 8, 106]
    closed = tdrafts.copy(); closed[4] = 8                                               # depth 2 is below the cut at depth 1
    assert list(orc.thinking_cutoff(seven, closed, tree, V, 1, [7, 8])) == [100, 7, 7, 8, 8, 8, 106]
    assert list(orc.thinking_cutoff(seven, closed, tree, V, 2, [7, 8])) == [100, 101, 102, 7, 104, 7, 106]   # rows 4 and 6 hold it at the cut
    # an end that waits for its mask starts at the first row from depth `row` on that admits end[0]
    five, fdrafts = np.arange(100, 105).astype(np.uint32), np.arange(50, 55).astype(np.uint32)
    short = tree_of([None, 0, 1, 2, 3])
    waits = lambda admits, row=1: list(orc.thinking_cutoff(five, fdrafts, short, V, row, [7, 8, 9], admits=admits))
    assert waits([0, 0, 0, 1, 1]) == [100, 101, 102, 7, 8]
    assert waits([1, 0, 0, 1, 0]) == [100, 101, 102, 7, 8]                               # a row above `row` does not start it
    assert waits([0, 1, 0, 0, 0]) == [100, 7, 8, 9, 104]
    assert waits([0, 0, 0, 0, 0]) == list(five)
    assert waits([1, 1, 1, 1, 1], row=0) == [7, 8, 9, 103, 104]
    # a draft token ends thinking up to the later cut too
    late = fdrafts.copy(); late[2] = 9
    assert list(orc.thinking_cutoff(five, late, short, V, 1, [7, 8, 9], admits=[0, 0, 0, 1, 1])) == list(five)          # depth 2 <= cut 3
    assert list(orc.thinking_cutoff(five, late, short, V, 1, [7, 8, 9], admits=[0, 1, 1, 1, 1])) == [100, 7, 8, 9, 104]  # depth 2 > cut 1
