"""CPU tests that pin the oracle's tree growth (orc_draft_tree) by an independent statement, invariants and frequencies."""
import numpy as np
import pytest

from tests import oracle as orc
from tests.draft_tree_statement import tree as stated_tree


def drawn_lattice(rng, spread=2.0, vocabulary=5000):
    candidates = np.stack([rng.choice(vocabulary, 16, replace=False) for _ in range(7)]).astype(np.uint32)
    unary = np.sort(rng.normal(0, spread, (7, 16)).astype(np.float32), axis=1)[:, ::-1].copy()   # the larger logit first
    edges = rng.normal(0, 1.0, (7, 16, 16)).astype(np.float32)
    return candidates, unary, edges


def compare(got, want):
    assert len(got["tokens"]) == len(want)
    for r, row in enumerate(want):
        if r:
            assert got["tokens"][r] == row["path"][-1], r
            assert got["tree"]["parent"][r] == row["parent"] and got["tree"]["depth"][r] == len(row["path"]), r
            assert got["tree"]["ancestors"][r] == got["tree"]["ancestors"][row["parent"]] | 1 << r, r
            if row["q"] < 0:
                assert got["q"][r] == -1.0
            else:
                assert abs(got["q"][r] - row["q"]) <= 1e-4 * row["q"] + 1e-7, r
            assert abs(got["estimate"][r] - row["estimate"]) <= 1e-4 * row["estimate"], r
            assert abs(got["caps"][r] - row["cap"]) <= 1e-5, r
        draws = [d for d in got["draws"][r] if d != 0xFF]
        assert draws == list(row["draws"]), (r, draws, row["draws"])
        if row["next"] is not None:
            assert np.allclose(got["next"][r], row["next"], rtol=1e-4, atol=1e-7), r
        else:
            assert not got["next"][r].any()


@pytest.mark.parametrize("temperature", [0.0, 0.7, 1.0])
@pytest.mark.parametrize("children,depth", [(1, 7), (2, 7), (4, 15), (4, 3), (3, 0)])
def test_trees_equal_the_independent_statement(temperature, children, depth):
    rng = np.random.default_rng(int(temperature * 10) + children * 100 + depth)
    compared = 0
    for trial in range(12):
        candidates, unary, edges = drawn_lattice(rng)
        lane = orc.draft_tree_lane(anchor=7, depth=depth, children=children, slope=float(rng.uniform(0.6, 1.4)),
                                   intercept=list(rng.normal(0.5, 0.5, 7)), temperature=temperature, noise=int(rng.integers(1 << 62)))
        want = stated_tree(candidates, unary, edges, lane)
        if want is None:
            continue
        compare(orc.draft_tree(candidates, unary, edges, lane), want)
        compared += 1
    assert compared >= 5


@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_a_host_chain_shares_the_tree(temperature):
    """A lane's host chain: its tokens join the tree at their rates, a draft step to a chain token is the chain's child
    (its cap what the others left, its estimate the more of its own and the rate), and a chain that leaves the draft's
    candidates goes on alone."""
    rng = np.random.default_rng(5 + int(temperature * 10))
    compared = 0
    for trial in range(24):
        candidates, unary, edges = drawn_lattice(rng)
        chain = np.zeros(15, np.uint32)
        for d in range(15):      # the draft's top candidate, another of its candidates, or a token of neither
            kind = rng.integers(3)
            chain[d] = candidates[d][0] if d < 7 and kind == 0 else candidates[d][rng.integers(1, 16)] if d < 7 and kind == 1 else 9000 + d
        rates = rng.uniform(0.2, 0.95, (15, 4)).astype(np.float32)
        lane = orc.draft_tree_lane(anchor=3, depth=int(rng.integers(1, 16)), children=int(rng.integers(1, 5)), slope=1.0,
                                   intercept=list(rng.normal(0, 0.5, 7)), temperature=temperature, noise=int(rng.integers(1 << 62)),
                                   chain=int(rng.integers(1, 16)))
        want = stated_tree(candidates, unary, edges, lane, chain, rates)
        if want is None:
            continue
        compare(orc.draft_tree(candidates, unary, edges, lane, chain, rates), want)
        compared += 1
    assert compared >= 8


def test_estimates_never_exceed_what_the_parent_has():
    """A row's children's estimates sum to at most its own (the target selects one token after it), a row's estimate is
    at most its parent's, a row's parent comes before it, and no tree outgrows its depth + 1 rows."""
    rng = np.random.default_rng(17)
    for trial in range(200):
        candidates, unary, edges = drawn_lattice(rng, spread=float(rng.uniform(0.5, 4)))
        chain = rng.choice(candidates[:, :3].ravel(), 15).astype(np.uint32)
        rates = rng.uniform(0, 1, (15, 4)).astype(np.float32)
        depth = int(rng.integers(0, 16))
        lane = orc.draft_tree_lane(anchor=1, depth=depth, children=int(rng.integers(1, 5)), slope=float(rng.uniform(0.5, 2)),
                                   intercept=list(rng.normal(0, 1, 7)), temperature=float(rng.choice([0.0, 0.5, 1.0])),
                                   noise=int(rng.integers(1 << 62)), chain=int(rng.integers(0, 16)))
        got = orc.draft_tree(candidates, unary, edges, lane, chain, rates)
        n = len(got["tokens"])
        assert 1 <= n <= min(16, depth + 1)
        sums = np.zeros(n)
        for r in range(1, n):
            parent = got["tree"]["parent"][r]
            assert parent < r and got["estimate"][r] <= got["estimate"][parent] * (1 + 1e-6)
            assert got["tree"]["depth"][r] == got["tree"]["depth"][parent] + 1 <= depth
            sums[parent] += got["estimate"][r]
        assert (sums <= got["estimate"] * (1 + 1e-5) + 1e-7).all(), (sums, got["estimate"])
        assert len({(got["tree"]["parent"][r], got["tokens"][r]) for r in range(1, n)}) == n - 1     # one row a token path


def test_a_sampled_row_draws_from_its_tempered_distribution():
    """The anchor's first drawn child over many seeds follows q_T, the candidates' probabilities at the lane's temperature
    (a Gumbel-top-1 draw is a draw from the distribution), and its draws are distinct."""
    rng = np.random.default_rng(23)
    candidates, unary, edges = drawn_lattice(rng, spread=1.0)
    T = 0.7
    score = (unary[0] + edges[0][0]).astype(np.float64)
    q = np.exp(score - score.max())
    q /= q.sum()
    w = np.exp((np.log(q) - np.log(q.max())) / T)
    q_t = w / w.sum()
    counts, trials = np.zeros(16), 4000
    for seed in range(trials):
        lane = orc.draft_tree_lane(anchor=1, depth=1, children=4, temperature=T, noise=seed * 7919 + 1)
        got = orc.draft_tree(candidates, unary, edges, lane)
        draws = got["draws"][0]
        assert len(set(draws)) == 4 and 0xFF not in draws
        counts[draws[0]] += 1
        assert np.allclose(got["next"][0], q_t, rtol=1e-4)
    sigma = np.sqrt(trials * q_t * (1 - q_t))
    assert (np.abs(counts - trials * q_t) <= 4.5 * sigma + 1).all(), (counts, trials * q_t)
