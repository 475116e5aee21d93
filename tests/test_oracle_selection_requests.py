"""The oracle's selection-request resolver against what the reference's own test states in closed
form (append, truncate to the window, deduplicate), and against the compiled reference where it built."""
import numpy as np
import pytest

from selection_cases import expected_unique, malformed_rows, random_cases, raw_row, reference_cases

VOCAB, TOP_K = 1000, 8


def check(gfo, ref, base, suffix, limit):
    raw = raw_row(gfo, base, suffix, limit)
    got, status = gfo.selection_request(raw, VOCAB, TOP_K)
    want = expected_unique(base, suffix, limit)
    assert status == 0
    assert got["top_k"] == TOP_K and got["history_count"] == len(want)
    assert got["base_candidate_count"] == TOP_K + len(want)
    assert got["history_token_ids"][:len(want)].tolist() == want
    assert not got["history_token_ids"][len(want):].any()
    if ref is not None:
        theirs = gfo.ref_selection_request(raw, TOP_K)
        assert theirs is not None
        for field in ("top_k", "base_candidate_count", "history_count"):
            assert theirs[field] == got[field]
        assert (theirs["history_token_ids"] == got["history_token_ids"]).all()


def test_the_reference_sweep_of_base_and_suffix_lengths(gfo, ref):
    cases = list(reference_cases())
    assert len(cases) == 120
    for base, suffix in cases:
        check(gfo, ref, base, suffix, 64)


def test_wrapped_heads_and_short_windows(gfo, ref):
    for base, suffix, limit in random_cases(5, 400, VOCAB):
        check(gfo, ref, base, suffix, limit)


def test_a_zero_window_keeps_nothing(gfo):
    got, status = gfo.selection_request(raw_row(gfo, [1, 2, 1], [1, 2, 1], limit=0), VOCAB, TOP_K)
    assert status == 0 and got["history_count"] == 0 and got["base_candidate_count"] == TOP_K


def test_without_a_penalty_the_history_is_not_listed(gfo, ref):
    raw = raw_row(gfo, [5, 6, 5], [7])
    got, status = gfo.selection_request(raw, VOCAB, TOP_K, repetition_enabled=False)
    assert status == 0 and got["history_count"] == 0 and got["base_candidate_count"] == TOP_K
    if ref is not None:
        theirs = gfo.ref_selection_request(raw, TOP_K, repetition_enabled=False)
        assert theirs["history_count"] == 0 and theirs["base_candidate_count"] == TOP_K


def test_malformed_rows_raise_bit_two_where_the_reference_throws(gfo, ref):
    for what, raw in malformed_rows(gfo):
        got, status = gfo.selection_request(raw, VOCAB, TOP_K)
        assert status == 2, what
        assert got["history_count"] == 0 and got["base_candidate_count"] == TOP_K, what
        if ref is not None:
            assert gfo.ref_selection_request(raw, TOP_K) is None, what


def test_tokens_outside_the_vocabulary_raise_bit_four_and_are_skipped(gfo):
    got, status = gfo.selection_request(raw_row(gfo, [3, VOCAB, 4], [VOCAB + 7, 3, 9]), VOCAB, TOP_K)
    assert status == 4
    assert got["history_token_ids"][:got["history_count"]].tolist() == [3, 4, 9]
    # also when the bad token has already left the window, and when the window is zero
    base = [VOCAB] + list(range(64))
    raw = raw_row(gfo, base[:64], [64])
    assert gfo.selection_request(raw, VOCAB, TOP_K)[1] == 4
    assert gfo.selection_request(raw_row(gfo, [], [VOCAB], limit=0), VOCAB, TOP_K)[1] == 4
