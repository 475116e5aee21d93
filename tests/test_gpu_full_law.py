"""Full-vocabulary proposal law on the device against the oracle's table, bit for bit
(src/engine/gemma3_draft.mm:295-395, dispatch :1040-1166; gather :1528-1581)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

VOCAB = 262144
TOTAL = 1 << 32


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as h
    h.init()
    return h


@pytest.fixture(scope="module")
def gfo():
    from oracle import gfo as g
    return g


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def opts(mod, t=1.0, k=64, p=0.95, m=0.0):
    return mod.SamplerOptions(t, k, p, m, 1.0)


def draws_for(hip, word):
    d = np.zeros(1, hip.draws_dtype)
    d["word"] = word
    d["u_accept"], d["u_residual"], d["u_next"] = 0.5, 0.5, 0.5
    return dev(d.view(np.uint8))


def full_law(hip, logits, o, word):
    law, cdf, proposal, status = hip.draft_law_any(dev(logits), o, draws=draws_for(hip, word))
    head = law.cpu().numpy().view(hip.law_dtype)[0]
    return head, cdf.cpu().numpy().view(np.uint64), int(proposal[0]) & 0xFFFFFFFF, int(status[0])


def check_full(hip, gfo, logits, t, k, p, m, word):
    head, cdf, proposal, status = full_law(hip, logits, opts(hip, t, k, p, m), word)
    rc, want = gfo.draft_law_full(logits, opts(gfo, t, k, p, m))
    assert rc == 0 and status == 0
    assert head["count"] == 0xFFFFFFFF
    assert np.array_equal(cdf, want)
    assert proposal == gfo.draft_select_full(want, word)
    return cdf


def test_wide_top_k_takes_the_full_path_bit_exact(hip, gfo):
    rng = np.random.default_rng(11)
    for trial in range(6):
        logits = rng.normal(0, 2, VOCAB).astype(np.float32)
        k = int(rng.choice([65, 128, 256]))
        t = float(rng.choice([0.7, 1.0, 1.3]))
        p = float(rng.choice([0.5, 0.9, 1.0]))
        m = float(rng.choice([0.0, 0.02]))
        cdf = check_full(hip, gfo, logits, t, k, p, m, int(rng.integers(0, 2 ** 32)))
        assert int(cdf[-1]) == TOTAL and np.count_nonzero(np.diff(cdf.astype(np.int64))) <= k


def test_small_and_ragged_vocabularies(hip, gfo):
    rng = np.random.default_rng(12)
    for vocab in (256, 768, 2048, 4096, 6400):   # below, at and between the 2048-token sort tiles
        logits = rng.normal(0, 2, vocab).astype(np.float32)
        check_full(hip, gfo, logits, 0.9, 100, 0.9, 0.0, int(rng.integers(0, 2 ** 32)))
    with pytest.raises(Exception):
        hip.draft_law_any(dev(np.zeros(1000, np.float32)), opts(hip, 1.0, 100))


def test_reference_uniform_and_nucleus_cases(hip, gfo):
    """tests/engine/gemma3_draft_tests.cpp:285-307: 262144 tied logits overflow the compact support."""
    logits = np.zeros(VOCAB, np.float32)
    cdf = check_full(hip, gfo, logits, 1.0, 1, 1.0, 0.0, 0xFFFFFFFF)
    assert np.all(np.diff(cdf.astype(np.int64)) == 16384)
    cdf = check_full(hip, gfo, logits, 1.0, 1, 0.5, 0.0, 0)
    d = np.diff(cdf.astype(np.int64))
    assert d[0] == 32768 and d[-1] == 0
    tiny = float(np.float32(1.401298464324817e-45))
    cdf = check_full(hip, gfo, logits, 1.0, 1, tiny, 0.0, 0xFFFFFFFF)
    assert int(cdf[1]) == TOTAL


def test_tie_overflow_hands_over_and_compact_stays_compact(hip, gfo):
    """:392-403: 256 ties stay compact, 257 fall back to the full table, 64 compact again."""
    for count in (256, 257, 64):
        logits = np.full(VOCAB, -100.0, np.float32)
        logits[:count] = 0.0
        head, cdf, proposal, status = full_law(hip, logits, opts(hip, 1.0, 1, 1.0, 0.0), 0xFFFFFFFF)
        assert status == 0 and proposal == count - 1
        if count == 257:
            rc, want = gfo.draft_law_full(logits, opts(gfo, 1.0, 1, 1.0, 0.0))
            assert rc == 0 and head["count"] == 0xFFFFFFFF and np.array_equal(cdf, want)
            assert abs((int(cdf[count]) - int(cdf[count - 1])) / TOTAL - 1.0 / count) < 1e-6
        else:
            rc, want = gfo.draft_law_compact(logits, opts(gfo, 1.0, 1, 1.0, 0.0))
            assert rc == 0 and head["count"] == count
            assert list(head["cdf"][:count + 1]) == [want.cdf[i] for i in range(count + 1)]


def test_greedy_drafting_is_a_step_at_the_lowest_argmax(hip, gfo):
    rng = np.random.default_rng(13)
    logits = rng.normal(0, 2, VOCAB).astype(np.float32)
    logits[[200000, 4242, 77777]] = 11.0
    cdf = check_full(hip, gfo, logits, 0.0, 1, 1.0, 0.0, 123456)
    assert int(cdf[4242]) == 0 and int(cdf[4243]) == TOTAL


def test_non_finite_logits_poison_the_law(hip):
    bad = np.zeros(VOCAB, np.float32)
    bad[5] = np.inf
    _, cdf, proposal, status = full_law(hip, bad, opts(hip, 1.0, 100, 1.0, 0.0), 7)
    assert status & 16 and status & 2 and proposal == 0xFFFFFFFF and not cdf.any()


def test_accept_gathers_from_the_full_table(hip, gfo):
    """Accept / residual decisions with q read from the table equal the oracle's, draws injected."""
    import torch
    rng = np.random.default_rng(14)
    p_logits = rng.normal(0, 3, (2, VOCAB)).astype(np.float32)
    q_logits = (p_logits[0] + rng.normal(0, 1.0, VOCAB)).astype(np.float32)
    o_gpu, o_cpu = opts(hip, 1.0, 128, 0.95, 0.0), opts(gfo, 1.0, 128, 0.95, 0.0)
    res, _ = hip.select_candidates(dev(p_logits), 128)
    rows = [gfo.select_candidates(p_logits[r], 128) for r in range(2)]
    rc, want_cdf = gfo.draft_law_full(q_logits, o_cpu)
    assert rc == 0
    accepted = 0
    for step in range(200):
        word, ua, ur, un = gfo.step_draws(21, step)
        law, cdf, proposal, status = hip.draft_law_any(dev(q_logits), o_gpu, seed=21, step=step)
        out = hip.spec_accept_law(res, law, cdf, proposal, o_gpu, seed=21, step=step, status=status)
        got = out.cpu().numpy().view(hip.result_dtype)[0]
        prop = gfo.draft_select_full(want_cdf, word)
        rc, want = gfo.spec_accept_full(rows[0], rows[1], want_cdf, prop, o_cpu, ua, ur, un)
        assert int(status[0]) == 0 and got["proposal"] == prop
        if rc != 0:   # a proposal outside p's support with no residual is refused by both
            assert got["status"] == -rc
            continue
        assert (got["accepted"], got["token"], got["next_root"]) == (want.accepted, want.token, want.next_root), step
        accepted += want.accepted
    assert 0 < accepted < 200


def test_device_laws_against_the_double_restatement(hip):
    """Both law paths on the device against the rule restated in double precision (tests/law_brute.py), not
    against the oracle: same supports, masses within 1e-6, on cases whose membership decisions are not
    within 1e-5 of their edge."""
    from law_brute import law, random_case
    rng = np.random.default_rng(909)
    compact = full = 0
    while compact < 8 or full < 8:
        logits, T, k, p, m = random_case(rng, 32768)
        wide = bool(rng.integers(0, 2))
        if wide:
            k = int(rng.choice([100, 256]))
        want, margin = law(logits, T, k, p, m)
        if margin < 1e-5:
            continue
        head, cdf, proposal, status = full_law(hip, logits, opts(hip, T, k, p, m), int(rng.integers(0, 2 ** 32)))
        assert status == 0
        if head["count"] == 0xFFFFFFFF:
            bins = np.diff(cdf.astype(np.int64))
            got = {int(t): bins[t] / TOTAL for t in np.nonzero(bins)[0]}
            tiny, full = 1e-6, full + 1
        else:
            n = int(head["count"])
            got = {int(head["ids"][i]): (int(head["cdf"][i + 1]) - int(head["cdf"][i])) / TOTAL for i in range(n)}
            got = {t: v for t, v in got.items() if v > 0}
            tiny, compact = 2.0 ** -31, compact + 1
        assert proposal in got
        for token, mass in want.items():
            if mass > tiny:
                assert token in got, (T, k, p, m, token, mass)
        for token, mass in got.items():
            assert token in want and abs(mass - want[token]) <= 1e-6, (T, k, p, m, token, mass)


def test_full_law_behind_a_vocabulary_map_is_the_oracles_table(hip, gfo):
    """guffin_hip_draft_law_any_mapped: the table, the proposal in both id spaces and the greedy case, bit for
    bit against the oracle's mapped full law; acceptance gathers q through the inverse map from the full table."""
    import torch
    vocab = 32768
    rng = np.random.default_rng(21)
    d2t = rng.permutation(vocab).astype(np.int32)
    d2t[rng.choice(vocab, 2000, replace=False)] = -1
    t2d = np.full(vocab, -1, np.int32)
    t2d[d2t[d2t >= 0]] = np.nonzero(d2t >= 0)[0].astype(np.int32)
    logits = rng.normal(0, 2, vocab).astype(np.float32)
    logits[np.nonzero(d2t < 0)[0][:4]] = 40.0
    for t, k, p, m in ((1.0, 128, 0.9, 0.0), (0.8, 256, 1.0, 0.02), (0.0, 1, 1.0, 0.0)):
        word = int(rng.integers(0, 2 ** 32))
        law, cdf, draft, target, status = hip.draft_law_any_mapped(dev(logits), dev(d2t), opts(hip, t, k, p, m),
                                                                   draws=draws_for(hip, word))
        rc, want = gfo.draft_law_full_mapped(logits, opts(gfo, t, k, p, m), d2t)
        assert rc == 0 and int(status[0]) == 0
        assert law.cpu().numpy().view(hip.law_dtype)[0]["count"] == 0xFFFFFFFF
        assert np.array_equal(cdf.cpu().numpy().view(np.uint64), want)
        pick = gfo.draft_select_full(want, word)
        assert int(draft[0]) == pick and int(target[0]) == d2t[pick] and d2t[pick] >= 0
        if t > 0:
            # acceptance with this table: the target's candidates are in its ids, q comes through the inverse map
            p_logits = rng.normal(0, 3, (2, vocab)).astype(np.float32)
            p_logits[0, d2t[pick]] += 6.0          # the proposal sits in the target's support
            cands, _ = hip.select_candidates(dev(p_logits), 64)
            o_gpu, o_cpu = opts(hip, t, 64, p, m), opts(gfo, t, 64, p, m)
            out = hip.spec_accept_mapped(cands, law, dev(t2d), target, o_gpu, seed=5, step=3, full_cdf=cdf, vocab=vocab)
            got = out.cpu().numpy().view(hip.result_dtype)[0]
            _, ua, ur, un = gfo.step_draws(5, 3)
            rc, ref = gfo.spec_accept_full_mapped(gfo.select_candidates(p_logits[0], 64), gfo.select_candidates(p_logits[1], 64),
                                                  want, t2d, int(d2t[pick]), o_cpu, ua, ur, un)
            assert rc == 0 and got["status"] == 0
            assert (got["accepted"], got["token"], got["next_root"]) == (ref.accepted, ref.token, ref.next_root)
            assert abs(got["acceptance_probability"] - ref.acceptance_probability) <= 1e-14
    # an unmapped token's NaN still poisons the law
    broken = logits.copy()
    broken[np.nonzero(d2t < 0)[0][0]] = np.nan
    *_, status = hip.draft_law_any_mapped(dev(broken), dev(d2t), opts(hip, 1.0, 128, 0.9, 0.0))
    assert int(status[0]) != 0
