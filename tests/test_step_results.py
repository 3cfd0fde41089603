"""The checks a completed step's results pass before a caller commits them (Runtime::finalizeDecode,
runtime/model/Runtime.cpp:2943-2972; invalidSelection, :1559-1582), on host arrays: no GPU."""
import numpy as np
import pytest

import splash_amd
from splash_amd import verify

V = 1000


def check(lanes, tokens, retained, accepted, masks, remaining=None, step_rows=None):
    verify.check_results(lanes, tokens, retained, accepted, masks, V, remaining, step_rows)


def test_valid_results_pass():
    tokens = np.arange(24, dtype=np.uint32)
    # a chain that kept its first three rows; a tree lane that kept rows 0, 2 and 5; a lane that kept its anchor only
    check([(0, 16), (16, 6), (22, 2)], tokens, [3, 3, 1], [2, 2, 0], [0b111, 0b100101, 0b1])
    check([(0, 16)], tokens[:16], [16], [15], [0xFFFF])                      # every row kept: the last token is the bonus
    check([(0, 5)], tokens[:5], [2], [1], [0b11], remaining=[2])               # cut by what the lane may still keep
    check([(4, 3)], tokens, [1], [0], [1], step_rows=24)                        # a lane that does not start the step


@pytest.mark.parametrize("what,args", [
    ("nothing retained", dict(retained=[0], accepted=[0], masks=[0])),
    ("more than its rows", dict(retained=[5], accepted=[3], masks=[0b11111])),
    ("mask and count disagree", dict(retained=[3], accepted=[2], masks=[0b11])),
    ("the anchor is not on the path", dict(retained=[2], accepted=[1], masks=[0b110])),
    ("a row past the lane's", dict(retained=[2], accepted=[1], masks=[0b10001])),
    ("accepted every row", dict(retained=[4], accepted=[4], masks=[0b1111])),
    ("accepted more than retained", dict(retained=[2], accepted=[3], masks=[0b11])),
    ("past what the lane may keep", dict(retained=[3], accepted=[2], masks=[0b111], remaining=[2])),
])
def test_invalid_results_are_backend_errors(what, args):
    tokens = np.arange(4, dtype=np.uint32)
    with pytest.raises(splash_amd.SplashError) as e:
        check([(0, 4)], tokens, args["retained"], args["accepted"], args["masks"], args.get("remaining"))
    assert not isinstance(e.value, ValueError), what       # SP_BACKEND_ERROR, not an argument error
    assert "lane 0" in str(e.value)


def test_a_sentinel_token_names_its_row():
    tokens = np.array([5, 0xFFFFFFFF, 7, 8], np.uint32)      # row 1 had no selectable logit
    with pytest.raises(splash_amd.SplashError, match="retained token 1"):
        check([(0, 4)], tokens, [3], [2], [0b111])
    check([(0, 4)], tokens, [1], [0], [1])                   # the sentinel is past what the lane retained
    with pytest.raises(splash_amd.SplashError, match="retained token 0"):
        check([(0, 4)], np.array([V, 1, 2, 3], np.uint32), [1], [0], [1])   # the first id past the vocabulary


def test_lanes_outside_the_step_and_missing_arrays():
    tokens = np.arange(8, dtype=np.uint32)
    with pytest.raises(splash_amd.SplashError, match="rows of the step"):
        check([(0, 4), (6, 4)], tokens, [1, 1], [0, 0], [1, 1])
    with pytest.raises(splash_amd.SplashError, match="rows of the step"):
        check([(0, 17)], np.arange(17, dtype=np.uint32), [1], [0], [1])


def test_penalty_words_are_rebuilt_from_a_history():
    """Sampling::rebuildPenaltyWords (Sampling.cpp:91-114 in the reference): the prompt's tokens carry the prompt bit when
    asked, the outputs and the pending anchor are counted, everything else is zero; a history without a prompt and a
    token past the vocabulary are refused."""
    from splash_amd import ops
    V = 50
    prompt, outputs = [3, 7, 7, 9], [7, 11, 11, 11]
    words = ops.Sampling.rebuild_penalty_words(V, prompt + outputs, len(outputs), pending_token=9)
    want = np.zeros(V, np.uint32)
    want[[3, 7, 9]] = ops.Sampling.PENALTY_PROMPT
    want[7] |= 1
    want[11] = 3
    want[9] |= 1
    assert np.array_equal(words, want)
    unmarked = ops.Sampling.rebuild_penalty_words(V, prompt + outputs, len(outputs), mark_prompt=False)
    assert np.array_equal(unmarked, np.bincount(outputs, minlength=V).astype(np.uint32))
    only_prompt = ops.Sampling.rebuild_penalty_words(V, prompt, 0)
    assert np.array_equal(only_prompt, np.where(np.isin(np.arange(V), prompt), ops.Sampling.PENALTY_PROMPT, 0).astype(np.uint32))
    with pytest.raises(splash_amd.SplashError):
        ops.Sampling.rebuild_penalty_words(V, outputs, len(outputs))          # no prompt
    with pytest.raises(ValueError):
        ops.Sampling.rebuild_penalty_words(V, [3, V], 0)
    with pytest.raises(ValueError):
        ops.Sampling.rebuild_penalty_words(V, [3], 0, pending_token=V)
