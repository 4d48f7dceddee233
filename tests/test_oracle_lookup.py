"""Prompt-lookup draft (PromptLookupDraft, neural/neuraldecode.pas:7742-7765): the oracle against hand-derived cases and against
the definition restated over ALL start positions, then the library's host-side function against the oracle."""
import itertools

import numpy as np
import pytest

from helpers import oracle_lib as O


def by_definition(ctx, m, k):
    """every start p (0-based) of an occurrence strictly before the suffix; the latest one wins; what follows it, cut to k"""
    n = len(ctx)
    if m < 1 or k < 1 or n < m + 1:
        return []
    suffix = ctx[n - m:]
    starts = [p for p in range(0, n - m) if ctx[p:p + m] == suffix]
    if not starts:
        return []
    p = max(starts)
    return ctx[p + m:p + m + k]


HAND = [
    # 'abcabc', suffix 'bc' occurs earlier at 1..2, followed by 'abc'
    (([0, 1, 2, 0, 1, 2], 2, 3), [0, 1, 2]),
    (([0, 1, 2, 0, 1, 2], 2, 2), [0, 1]),
    # the most recent earlier occurrence wins: 'a x a y a' with suffix 'a' -> the one before 'y'
    (([0, 7, 0, 8, 0], 1, 2), [8, 0]),
    # overlapping occurrence: 'aaa', suffix 'aa' also starts at 0, one token follows it
    (([5, 5, 5], 2, 4), [5]),
    # no earlier occurrence
    (([1, 2, 3, 4], 2, 3), []),
    # context shorter than match_len + 1 (the reference's no-match test: MatchLen 64 on a 2-token prompt)
    (([0, 1], 64, 4), []),
    (([3], 1, 1), []),
    # degenerate arguments
    (([1, 1, 1], 0, 3), []),
    (([1, 1, 1], 1, 0), []),
]


@pytest.mark.parametrize("args,want", HAND)
def test_hand_cases(args, want):
    ctx, m, k = args
    assert O.prompt_lookup_draft(ctx, m, k) == want
    assert by_definition(ctx, m, k) == want


def test_oracle_equals_the_definition_on_every_short_context():
    n_checked = 0
    for alphabet, max_len in ((2, 10), (3, 7)):
        for n in range(1, max_len + 1):
            for ctx in itertools.product(range(alphabet), repeat=n):
                ctx = list(ctx)
                for m in (1, 2, 3):
                    for k in (1, 2, 4):
                        assert O.prompt_lookup_draft(ctx, m, k) == by_definition(ctx, m, k), (ctx, m, k)
                        n_checked += 1
    assert n_checked > 40000


def test_library_host_function_equals_the_oracle():
    import importlib
    cai = importlib.import_module("neural-api_amd.caihip")
    rng = np.random.default_rng(77)
    for args, want in HAND:
        assert cai.prompt_lookup_draft(*args) == want
    for _ in range(3000):
        n = int(rng.integers(1, 60)); alphabet = int(rng.integers(2, 6))
        ctx = rng.integers(0, alphabet, n).tolist()
        m = int(rng.integers(1, 5)); k = int(rng.integers(1, 8))
        assert cai.prompt_lookup_draft(ctx, m, k) == O.prompt_lookup_draft(ctx, m, k), (ctx, m, k)
