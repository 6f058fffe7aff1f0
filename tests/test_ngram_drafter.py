"""The oracle's n-gram drafter (src/engine/session.c:437-513 of the reference) against worked
examples and an independent enumeration. The reference holds no test of this function; what
pins the restatement is its documented rule -- longest suffix of history + [seed] (at most
min(max_suffix, 8)) that occurs earlier, the occurrence with the most following tokens up to
k_max - 1, the most recent among equals -- enumerated here over every (length, position)."""
import numpy as np
import pytest


def enumerate_drafts(hist, seed, k_max, max_suffix):
    """All (length, position) pairs, ranked by the documented rule; no early exits."""
    hist = [int(t) for t in hist]
    n = len(hist)
    if k_max <= 1 or n == 0:
        return [seed], 0
    text = hist + [seed]
    cands = []
    for length in range(1, min(max_suffix, 8) + 1):
        if length > n + 1:
            continue
        suffix = text[len(text) - length:]
        for p in range(0, n - length + 1):
            if hist[p:p + length] != suffix:
                continue
            follow = n - (p + length)
            if follow <= 0:
                continue
            cands.append((length, min(follow, k_max - 1), p))
    if not cands:
        return [seed], 0
    length, take, p = max(cands)
    return [seed] + hist[p + length:p + length + take], length


def test_worked_examples(oracle):
    # history: a b c d a b c e ; seed continues "a b" -> after the earlier "a b c"? worked by hand:
    h = [1, 2, 3, 4, 1, 2, 3, 5]
    # suffix (3, 5, seed=1)? no earlier "5 1"; longest match is the seed alone: "1" occurs at 0
    # and 4. After position 4 three tokens follow (2 3 5), after position 0 seven; with k_max = 4
    # both offer 3 drafts, so the more recent one (4) wins.
    assert oracle.propose_drafts_ngram(h, 1, 4, 4) == ([1, 2, 3, 5], 1)
    # with k_max = 6 position 4 offers only 3, position 0 offers 5: more following tokens win
    assert oracle.propose_drafts_ngram(h, 1, 6, 4) == ([1, 2, 3, 4, 1, 2], 1)
    # history ends "... 1 2", seed 3: suffix "1 2 3" occurs at 0 (and "2 3" at 1): length 3 wins
    h = [1, 2, 3, 9, 8, 1, 2]
    assert oracle.propose_drafts_ngram(h, 3, 3, 4) == ([3, 9, 8], 3)
    # max_suffix 2 limits the reported length, the same occurrence is found
    assert oracle.propose_drafts_ngram(h, 3, 3, 2) == ([3, 9, 8], 2)
    # a match at the very end has nothing after it and is not a candidate
    assert oracle.propose_drafts_ngram([4, 5, 6], 6, 4, 4) == ([6], 0)
    # no match, k_max <= 1, empty history, max_suffix 0
    assert oracle.propose_drafts_ngram([4, 5, 6], 7, 4, 4) == ([7], 0)
    assert oracle.propose_drafts_ngram([7, 5, 6], 7, 1, 4) == ([7], 0)
    assert oracle.propose_drafts_ngram([], 7, 4, 4) == ([7], 0)
    assert oracle.propose_drafts_ngram([7, 5, 6], 7, 4, 0) == ([7], 0)
    # periodic text: "1 2 1 2 1 2", seed 1: suffix of 4 = "2 1 2 1"? history+seed = 1 2 1 2 1 2 1,
    # last four "2 1 2 1" occurs at position 1 (followed by 2 at index 5): one draft
    assert oracle.propose_drafts_ngram([1, 2, 1, 2, 1, 2], 1, 8, 4) == ([1, 2], 4)
    # max_suffix beyond 8 is capped at 8
    h = list(range(20)) + list(range(20))
    assert oracle.propose_drafts_ngram(h[:-1], 19, 5, 100)[1] == 8


@pytest.mark.parametrize("seed", range(4))
def test_oracle_matches_enumeration(oracle, seed):
    g = np.random.default_rng(seed)
    for _ in range(1500):
        n = int(g.integers(0, 40))
        alphabet = int(g.choice([2, 3, 5, 50]))
        hist = g.integers(0, alphabet, n).astype(np.int32)
        sd = int(g.integers(0, alphabet))
        k_max = int(g.integers(1, 17))
        ms = int(g.integers(0, 12))
        assert oracle.propose_drafts_ngram(hist, sd, k_max, ms) == \
            enumerate_drafts(hist, sd, k_max, ms), (hist.tolist(), sd, k_max, ms)
