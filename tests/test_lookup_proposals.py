"""Prompt lookup (host code): the index's match after every token against the definition searched by brute force."""
import numpy as np
import pytest

from splash_amd import lookup


def brute_force(tokens, minimum=3, longest=64):
    """The definition (LookupProposals.hpp:17-24 in the reference): the longest suffix of the tokens, counted up to
    `longest`, that also ends at an earlier token, none shorter than `minimum`; of its earlier ends the most recent."""
    n = len(tokens)
    last = n - 1
    for length in range(min(longest, last), minimum - 1, -1):
        suffix = tokens[n - length:]
        for end in range(last - 1, length - 2, -1):
            if tokens[end - length + 1:end + 1] == suffix:
                return length, end
    return 0, 0


@pytest.mark.parametrize("alphabet,count,seed", [(2, 400, 1), (3, 600, 2), (5, 500, 3), (50, 300, 4)])
def test_the_match_after_every_token_is_the_definitions(alphabet, count, seed):
    rng = np.random.default_rng(seed)
    tokens = [int(t) for t in rng.integers(0, alphabet, count)]
    # stretches copied from earlier and runs of one token, as prompts with repeated files and padding have them
    for _ in range(6):
        at, n, to = (int(v) for v in (rng.integers(0, count // 2), rng.integers(5, 120), rng.integers(count // 2, count)))
        tokens[to:to + n] = tokens[at:at + n]
    tokens = tokens[:count]
    tokens[count // 3:count // 3 + 90] = [7] * 90
    index = lookup.LookupIndex()
    for i, token in enumerate(tokens):
        index.append([token])
        want = brute_force(tokens[:i + 1])
        got = index.match()
        assert (got if got[0] else (0, 0)) == want, (i, got, want)
        length, end = got
        proposals = list(index.proposals(7))
        assert proposals == (tokens[end + 1:min(end + 8, i + 1)] if length else [])


def test_appending_in_pieces_is_appending_at_once_and_long_runs_stay_cheap():
    rng = np.random.default_rng(9)
    tokens = rng.integers(0, 4, 3000).astype(np.uint32)
    whole, pieces = lookup.LookupIndex(tokens), lookup.LookupIndex()
    for part in np.array_split(tokens, 17):
        pieces.append(part)
    assert whole.match() == pieces.match() == brute_force([int(t) for t in tokens])
    # a hundred thousand of one token: the match is the 64 tokens that end one before
    run = lookup.LookupIndex(np.full(100_000, 5, np.uint32))
    assert run.match() == (64, 99_998) and list(run.proposals(4)) == [5]
    assert lookup.LookupIndex([1, 2, 3]).match() == (0, 0) and list(lookup.LookupIndex([1, 2]).proposals(3)) == []
    # the shortest match: three tokens; two are none
    assert lookup.LookupIndex([1, 2, 3, 9, 1, 2, 3]).match() == (3, 2)
    assert lookup.LookupIndex([1, 2, 3, 9, 8, 2, 3]).match() == (0, 0)
    assert list(lookup.LookupIndex([1, 2, 3, 4, 5, 9, 1, 2, 3]).proposals(8)) == [4, 5, 9, 1, 2, 3]


def test_a_lookup_tokens_agreement_with_the_drafts_candidates():
    candidates = np.arange(7 * 16).reshape(7, 16)
    assert lookup.agreement(0, 0, candidates) == lookup.AGREEMENT_TOP
    assert lookup.agreement(5, 0, candidates) == lookup.AGREEMENT_CANDIDATE
    assert lookup.agreement(16, 0, candidates) == lookup.AGREEMENT_ABSENT
    assert lookup.agreement(16, 1, candidates) == lookup.AGREEMENT_TOP
    assert lookup.agreement(16, 7, candidates) == lookup.AGREEMENT_UNKNOWN      # the draft proposes seven positions
