"""guffin_hip_selection_requests against the oracle on the reference's cases (wrapped heads, full
windows, suffix overflow), bit for bit, and the candidate selection that consumes the resolved rows."""
import numpy as np
import pytest

from selection_cases import malformed_rows, random_cases, raw_row, reference_cases

pytestmark = pytest.mark.gpu
VOCAB, TOP_K = 1000, 8


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def resolve(hip, rows, vocab=VOCAB, top_k=TOP_K, repetition=True):
    resolved, histories, status = hip.selection_requests(np.stack(rows), vocab, top_k, repetition)
    return (resolved.cpu().numpy().view(hip.resolved_row_dtype), histories.cpu().numpy().view(np.uint32),
            int(status.item()), resolved)


def same(gfo, got, histories, raw, vocab=VOCAB, top_k=TOP_K, repetition=True):
    want, status = gfo.selection_request(raw, vocab, top_k, repetition)
    for field in ("top_k", "base_candidate_count", "history_count", "reserved"):
        assert got[field] == want[field], field
    assert np.array_equal(got["history_token_ids"], want["history_token_ids"])
    assert np.array_equal(histories, want["history_token_ids"])
    return status


def test_the_reference_sweep_in_one_launch(hip, gfo):
    rows = [raw_row(gfo, base, suffix) for base, suffix in reference_cases()]
    got, histories, status, _ = resolve(hip, rows)
    assert status == 0 and got.size == 120
    for i, raw in enumerate(rows):
        assert same(gfo, got[i], histories[i], raw) == 0


def test_wrapped_heads_short_windows_and_no_penalty(hip, gfo):
    rows = [raw_row(gfo, base, suffix, limit) for base, suffix, limit in random_cases(11, 500, VOCAB)]
    assert any(int(r["history_head"]) > 0 for r in rows)
    for repetition in (True, False):
        got, histories, status, _ = resolve(hip, rows, repetition=repetition)
        assert status == 0
        for i, raw in enumerate(rows):
            same(gfo, got[i], histories[i], raw, repetition=repetition)
        if not repetition:
            assert not got["history_count"].any() and (got["base_candidate_count"] == TOP_K).all()


def test_status_bits_are_the_references(hip, gfo):
    for what, raw in malformed_rows(gfo):
        got, histories, status, _ = resolve(hip, [raw])
        assert status == 2, what
        assert same(gfo, got[0], histories[0], raw) == 2
    bad = raw_row(gfo, [3, VOCAB, 4], [VOCAB + 7, 3, 9])
    got, histories, status, _ = resolve(hip, [bad])
    assert status == 4 and same(gfo, got[0], histories[0], bad) == 4
    assert got[0]["history_token_ids"][:3].tolist() == [3, 4, 9] and got[0]["history_count"] == 3
    # a malformed row and a bad token in one launch leave both bits; good rows are untouched by either
    good = raw_row(gfo, [1, 2, 1], [5])
    got, histories, status, _ = resolve(hip, [malformed_rows(gfo)[0][1], good, bad])
    assert status == 6 and same(gfo, got[1], histories[1], good) == 0


def test_candidates_of_resolved_rows_keep_each_rows_own_count(hip, gfo):
    """Row r keeps top_k + its own distinct-history count best logits, then its history's logits:
    the reference's candidate kernels read base_candidate_count per row (metal_kernels.mm:3821-3840)."""
    import torch
    vocab, top_k = 50000, 40
    rng = np.random.default_rng(3)
    logits = rng.normal(0, 3, (3, vocab)).astype(np.float32)
    rows = [raw_row(gfo, [], []), raw_row(gfo, [7, 9, 7, 11], [9, 13]),
            raw_row(gfo, rng.integers(0, vocab, 90).tolist(), rng.integers(0, vocab, 5).tolist())]
    got, _, status, resolved = resolve(hip, rows, vocab=vocab, top_k=top_k)
    assert status == 0 and got["history_count"].tolist()[:2] == [0, 4]
    res, st = hip.select_candidates_resolved(torch.from_numpy(logits).cuda(), top_k + 64, resolved)
    c = hip.candidates_to_numpy(res)
    for r in range(3):
        hist = got[r]["history_token_ids"][:got[r]["history_count"]]
        want = gfo.select_candidates(logits[r], int(got[r]["base_candidate_count"]), hist)
        assert int(st[r]) == 0 and c[r]["count"] == want.size
        assert np.array_equal(c[r]["values"]["token"][:want.size], want["token"])
        assert np.array_equal(c[r]["values"]["logit"][:want.size].view(np.uint32), want["logit"].view(np.uint32))


def test_input_validation_flags_a_foreign_or_changed_token(hip):
    """verifier_input_validate_u32_kernel (metal_kernels.mm:2323-2334): bit 1 when a row's id is outside
    the vocabulary or is not the id the host planned."""
    import torch
    def run(actual, expected, vocab=100):
        status = torch.zeros(1, dtype=torch.int32, device="cuda")
        hip.input_validation(torch.tensor(actual, dtype=torch.int32).cuda(), torch.tensor(expected, dtype=torch.int32).cuda(),
                             vocab, status)
        return int(status.item())
    assert run([1, 2, 99], [1, 2, 99]) == 0
    assert run([1, 2, 3], [1, 5, 3]) == 1
    assert run([1, 100], [1, 100]) == 1
    assert run(list(range(90)) + [7], list(range(90)) + [8]) == 1
