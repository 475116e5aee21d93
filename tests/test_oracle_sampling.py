"""Pins the oracle's sampling laws (CPU only).

Exact fixtures restate tests/engine/sampling_tests.cpp:34-76, 181-228 and
tests/engine/lossless_sampling_tests.cpp:69-168 (data only); random cases are compared
bit for bit with the compiled reference sampling.cpp where oracle/_ref is built.
"""
import ctypes as C
import math

import numpy as np
import pytest

TOTAL = 1 << 32


def opts(gfo, t=1.0, k=64, p=0.95, m=0.0, r=1.0):
    return gfo.SamplerOptions(t, k, p, m, r)


def cands(gfo, pairs):
    return np.array(pairs, gfo.token_logit)


def law_from(gfo, pairs):
    """Compact law from (token, mass) pairs given in ascending token order."""
    law = gfo.DraftLaw()
    law.count = len(pairs)
    acc = 0
    for i, (tok, mass) in enumerate(pairs):
        law.ids[i] = tok
        law.cdf[i] = acc
        acc += mass
    law.cdf[len(pairs)] = acc
    return law


def prepared_from(gfo, pairs):
    p = gfo.Prepared()
    p.count = len(pairs)
    p.total_sampling_weight = 1.0
    for i, (tok, prob) in enumerate(pairs):
        p.token[i], p.probability[i], p.sampling_weight[i] = tok, prob, prob
    return p


def spec(gfo, prepared, law, proposal, ua, ur):
    out = gfo.SpecResult()
    rc = gfo.lib().gfo_spec_from_prepared(C.byref(prepared), C.byref(law), proposal,
                                          C.c_double(ua), C.c_double(ur), C.byref(out))
    return rc, out


def test_ties_and_repetition_penalty(gfo):
    c = cands(gfo, [(2, 3.0), (1, 3.0), (0, 2.9), (3, -1.0)])
    rc, p = gfo.prepare(c, opts(gfo, t=0.0, k=4))
    assert rc == 0 and p.count == 1 and p.token[0] == 1
    rc, p = gfo.prepare(c, opts(gfo, t=0.0, k=4, r=2.0), history=[2, 1])
    assert rc == 0 and p.token[0] == 0
    neg = cands(gfo, [(0, -1.0), (1, -1.1), (2, -2.0)])
    rc, p = gfo.prepare(neg, opts(gfo, t=0.0, k=3, r=2.0), history=[0])
    assert rc == 0 and p.token[0] == 1


def test_top_p_filters_before_temperature_and_min_p(gfo):
    c = cands(gfo, [(0, 0.0), (1, -1.0), (2, -4.0), (3, -8.0)])
    rc, p = gfo.prepare(c, opts(gfo, t=2.0, k=4, p=0.7, m=0.05, r=1.1), history=[3])
    assert rc == 0 and p.count == 1 and p.token[0] == 0 and p.probability[0] == 1.0


def test_prepared_probabilities_fixture(gfo):
    c = cands(gfo, [(3, 0.0), (1, 2.0), (2, 1.0), (1, 2.0), (4, -4.0)])
    rc, p = gfo.prepare(c, opts(gfo, t=1.0, k=4, p=1.0, m=0.0, r=2.0), history=[1])
    assert rc == 0 and p.count == 4
    assert [p.token[i] for i in range(4)] == [1, 2, 3, 4]
    raw = [math.exp(0.0), math.exp(0.0), math.exp(-1.0), math.exp(-5.0)]
    for i in range(4):
        assert abs(p.probability[i] - raw[i] / sum(raw)) < 1e-12
    rc, g = gfo.prepare(c, opts(gfo, t=0.0, k=4, r=2.0), history=[1])
    assert rc == 0 and g.count == 1 and g.token[0] == 1 and g.probability[0] == 1.0
    # malformed inputs fail closed
    assert gfo.prepare(cands(gfo, [(0, float("nan"))]), opts(gfo, k=1))[0] < 0
    assert gfo.prepare(cands(gfo, [(0, 1.0), (0, 2.0)]), opts(gfo, k=1))[0] < 0
    assert gfo.prepare(cands(gfo, [(0, 1.0)]), opts(gfo, k=2))[0] < 0


def test_integer_cdf_boundaries(gfo):
    half = TOTAL // 2
    q = law_from(gfo, [(4, 1), (7, half - 1), (9, half)])
    sel = lambda w: gfo.lib().gfo_draft_select(C.byref(q), C.c_uint32(w))
    assert sel(0) == 4 and sel(1) == 7 and sel(half - 1) == 7 and sel(half) == 9
    assert sel(0xFFFFFFFF) == 9
    delta = law_from(gfo, [(91, TOTAL)])
    assert gfo.lib().gfo_draft_select(C.byref(delta), C.c_uint32(0xFFFFFFFF)) == 91


def test_injected_draws_enumerate_exact_marginal(gfo):
    p = prepared_from(gfo, [(0, 0.25), (1, 0.5), (2, 0.25)])
    quarter = TOTAL // 4
    q = law_from(gfo, [(0, 2 * quarter), (1, quarter), (2, quarter)])
    counts = [0, 0, 0]
    for pb in range(8):
        word = (2 * pb + 1) * TOTAL // 16
        proposal = gfo.lib().gfo_draft_select(C.byref(q), C.c_uint32(word))
        for ab in range(8):
            for rb in range(8):
                rc, out = spec(gfo, p, q, proposal, (ab + 0.5) / 8, (rb + 0.5) / 8)
                assert rc == 0
                counts[out.token] += 1
    assert counts == [128, 256, 128]
    rc, out = spec(gfo, p, q, 0, float(np.nextafter(0.5, 0.0)), 0.0)
    assert rc == 0 and out.accepted == 1
    rc, out = spec(gfo, p, q, 0, 0.5, 0.0)
    assert rc == 0 and out.accepted == 0 and out.token == 1


def test_exact_analytic_marginals(gfo):
    unit = TOTAL // 8
    cases = [
        ([(0, 0.25), (1, 0.5), (2, 0.25)], [(0, 4 * unit), (1, unit), (2, 3 * unit)]),
        ([(0, 0.25), (1, 0.5), (2, 0.25)], [(1, 4 * unit), (3, 4 * unit)]),
        ([(0, 0.5), (1, 0.5)], [(2, 4 * unit), (3, 4 * unit)]),
        ([(0, 0.25), (1, 0.75)], [(0, 2 * unit), (1, 6 * unit)]),
    ]
    for target, draft in cases:
        p, q = prepared_from(gfo, target), law_from(gfo, draft)
        marginal = {}
        for tok, mass in draft:
            qx = mass / TOTAL
            rc, out = spec(gfo, p, q, tok, 0.0, 0.0)
            if rc != 0:
                continue
            a = out.acceptance_probability
            marginal[tok] = marginal.get(tok, 0.0) + qx * a
            if a < 1.0:
                # residual law: weights max(p-q,0) normalised
                res = {t: max(pr - dict(draft).get(t, 0) / TOTAL, 0.0) for t, pr in target}
                z = sum(res.values())
                assert abs(z - out.residual_total) < 1e-15
                for t, w in res.items():
                    marginal[t] = marginal.get(t, 0.0) + qx * (1 - a) * w / z
        for t, pr in target:
            assert abs(marginal.get(t, 0.0) - pr) < 1e-12, (target, draft, marginal)


def test_near_equal_residual_and_full_support(gfo):
    half = TOTAL // 2
    eps = 1.0 / TOTAL
    q = law_from(gfo, [(0, half), (1, half)])
    p = prepared_from(gfo, [(0, 0.5 + eps), (1, 0.5 - eps)])
    rc, out = spec(gfo, p, q, 1, float(np.nextafter(1.0, 0.0)), 0.75)
    assert rc == 0 and out.residual_count == 1 and out.residual_total == eps
    assert out.accepted == 0 and out.token == 0
    full_p = prepared_from(gfo, [(i, 1.0 / 256) for i in range(256)])
    full_q = law_from(gfo, [(i, TOTAL // 256) for i in range(256)])
    rc, out = spec(gfo, full_p, full_q, 255, 0.999, 0.5)
    assert rc == 0 and out.acceptance_probability == 1.0 and out.residual_count == 0
    # zero-mass proposal, draw outside [0,1) fail closed
    assert spec(gfo, p, q, 5, 0.1, 0.1)[0] < 0
    assert spec(gfo, p, q, 1, 1.0, 0.1)[0] < 0


def uniform_table(vocabulary):
    """The reference's 32 000-token proposal law: endpoint(i) = i * 2^32 / vocabulary, integer division."""
    return (np.arange(vocabulary + 1, dtype=np.uint64) * np.uint64(1 << 32)) // np.uint64(vocabulary)


def sparse_target(gfo):
    """p = {0: 0.125, 999: 0.375, 40000: 0.5} as logits (token 40000 lies outside the 32 000-token draft
    vocabulary); top-k 3, no nucleus, T = 1."""
    pairs = [(0, math.log(0.125)), (999, math.log(0.375)), (40000, math.log(0.5))]
    return cands(gfo, pairs), opts(gfo, 1.0, 3, 1.0, 0.0)


def test_gathered_full_table_recovers_the_target_marginal(gfo):
    """tests/engine/lossless_sampling_tests.cpp:375-432: over every proposal of a 32 000-token law with sparse
    lookups of q on p's support, sum_x q(x) [a(x) 1{x = t} + (1 - a(x)) r_x(t)] = p(t) — the acceptance is
    lossless — and the residual is never renormalised over the vocabulary intersection."""
    vocabulary = 32000
    cdf = uniform_table(vocabulary)
    row, o = sparse_target(gfo)
    rc, p = gfo.prepare(row, o)
    assert rc == 0 and p.count == 3
    tokens = [p.token[i] for i in range(3)]
    prob = {p.token[i]: p.probability[i] for i in range(3)}
    assert abs(prob[0] - 0.125) < 1e-7 and abs(prob[999] - 0.375) < 1e-7 and abs(prob[40000] - 0.5) < 1e-7
    total = float(1 << 32)
    mass = lambda t: float(int(cdf[t + 1]) - int(cdf[t])) if t < vocabulary else 0.0
    marginal = {t: 0.0 for t in tokens}
    for x in range(vocabulary):
        rc, got = gfo.spec_accept_full(row, row, cdf, x, o, 0.0, 0.99, 0.5)
        assert rc == 0, (x, rc)
        qx = mass(x) / total
        # the residual this proposal leaves: max(p - q, 0) over p's support in p's order, q not renormalised
        residual = [max(prob[t] - mass(t) / total, 0.0) for t in tokens]
        assert got.residual_count == sum(1 for r in residual if r > 0.0)
        assert abs(got.residual_total - sum(residual)) <= 4e-16
        if x in prob:
            assert abs(got.acceptance_probability - min(1.0, prob[x] / qx)) <= 1e-15
        else:
            assert got.acceptance_probability == 0.0
            assert not got.accepted and got.token == tokens[-1]   # u_residual 0.99 lands in the last entry
        for i, t in enumerate(tokens):
            inside = qx * got.acceptance_probability if t == x else 0.0
            marginal[t] += inside + qx * (1.0 - got.acceptance_probability) * residual[i] / got.residual_total
        if x == 17:
            assert abs(got.residual_total - (1.0 - (mass(0) + mass(999)) / total)) <= 1e-15
            # the correction can select a target token that the draft vocabulary does not have
            rc, first = gfo.spec_accept_full(row, row, cdf, x, o, 0.0, 0.0, 0.5)
            assert rc == 0 and tokens[0] == 40000 and not first.accepted and first.token == 40000
    for t in tokens:
        assert abs(marginal[t] - prob[t]) <= 1e-11, (t, marginal[t], prob[t])


def test_prepare_matches_compiled_reference_bit_exact(gfo, ref):
    if ref is None:
        pytest.skip("oracle/_ref not built")
    rng = np.random.default_rng(10)
    checked = 0
    for trial in range(300):
        n = int(rng.integers(64, 130))
        toks = rng.choice(262144, n, replace=False).astype(np.uint32)
        logit = rng.normal(0, rng.choice([0.5, 2.0, 6.0]), n).astype(np.float32)
        c = np.zeros(n, gfo.token_logit)
        c["token"], c["logit"] = toks, logit
        o = opts(gfo, t=float(rng.choice([0.0, 0.7, 1.0, 1.3])), k=int(rng.choice([1, 40, 64])),
                 p=float(rng.choice([0.5, 0.9, 0.95, 1.0])), m=float(rng.choice([0.0, 0.05])),
                 r=float(rng.choice([1.0, 1.1])))
        hist = toks[: int(rng.integers(0, 5))]
        rc_a, a = gfo.prepare(c, o, hist)
        rc_b, b = gfo.prepare(c, o, hist, which=ref)
        assert (rc_a == 0) == (rc_b == 0)
        if rc_a:
            continue
        checked += 1
        assert a.count == b.count and a.total_sampling_weight == b.total_sampling_weight
        for i in range(a.count):
            assert a.token[i] == b.token[i]
            assert a.probability[i] == b.probability[i]
            assert a.sampling_weight[i] == b.sampling_weight[i]
    assert checked > 200


def test_spec_accept_matches_compiled_reference(gfo, ref):
    if ref is None:
        pytest.skip("oracle/_ref not built")
    rng = np.random.default_rng(11)
    accepted = rejected = 0
    for trial in range(400):
        vocab = 4096
        p_logits = rng.normal(0, 3, (2, vocab)).astype(np.float32)
        q_logits = (p_logits[0] + rng.normal(0, 1.5, vocab)).astype(np.float32)
        o = opts(gfo, t=1.0, k=64, p=0.95)
        rc, law = gfo.draft_law_compact(q_logits, o)
        assert rc == 0
        word, ua, ur, un = gfo.step_draws(123, trial)
        proposal = gfo.lib().gfo_draft_select(C.byref(law), C.c_uint32(word))
        r0 = gfo.select_candidates(p_logits[0], 64)
        r1 = gfo.select_candidates(p_logits[1], 64)
        rc_a, a = gfo.spec_accept(r0, r1, law, proposal, o, ua, ur, un)
        rc_b, b = gfo.spec_accept(r0, r1, law, proposal, o, ua, ur, un, which=ref)
        assert rc_a == 0 and rc_b == 0
        assert (a.accepted, a.token, a.next_root) == (b.accepted, b.token, b.next_root)
        assert a.acceptance_probability == b.acceptance_probability
        assert a.residual_total == b.residual_total and a.residual_count == b.residual_count
        accepted += a.accepted
        rejected += 1 - a.accepted
    assert accepted > 50 and rejected > 50


def test_philox_known_answers_and_draws(gfo):
    # Random123 kat_vectors, philox4x32-10
    assert gfo.philox([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert gfo.philox([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert gfo.philox([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]) == \
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]
    seen = set()
    for step in range(2000):
        w, a, r, n = gfo.step_draws(7, step)
        assert 0 <= a < 1 and 0 <= r < 1 and 0 <= n < 1
        seen.add(w)
    assert len(seen) > 1990
    a0 = gfo.philox([5, 0, 0, 0], [7, 0])
    w, a, _, _ = gfo.step_draws(7, 5)
    assert w == a0[0] and a == (((a0[1] << 32) | a0[2]) >> 11) * 2.0 ** -53


def test_exp_f32_accuracy_and_monotonicity(gfo):
    xs = np.concatenate([-np.random.default_rng(12).uniform(0, 86, 20000), [0.0, -1e-8, -85.99]])
    xs = np.sort(xs.astype(np.float32))
    got = np.array([gfo.lib().gfo_exp_f32(C.c_float(float(x))) for x in xs], np.float32)
    want = np.exp(xs.astype(np.float64))
    ulp = np.spacing(want.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got - want) / ulp) < 1.5
    assert np.all(np.diff(got) >= 0)
    assert gfo.lib().gfo_exp_f32(C.c_float(0.0)) == 1.0
    assert gfo.lib().gfo_exp_f32(C.c_float(-90.0)) == 0.0
    assert gfo.lib().gfo_exp_f32(C.c_float(-np.inf)) == 0.0


def test_compact_law_invariants_and_softmax(gfo):
    vocab = 262144
    # 48 candidates in different 512-tiles, cutoff ties extend the support
    # (tests/engine/gemma3_draft_tests.cpp:332-362, data only)
    logits = np.full(vocab, -100.0, np.float32)
    toks = [37 + i * 4099 for i in range(48)]
    for i, t in enumerate(toks):
        logits[t] = 4.0 - i * 0.07 if i < 38 else 1.34
    o = opts(gfo, t=1.0, k=40, p=0.87, m=0.05)
    rc, law = gfo.draft_law_compact(logits, o)
    assert rc == 0 and law.cdf[law.count] == TOTAL and law.cdf[0] == 0
    ids = [law.ids[i] for i in range(law.count)]
    assert ids == sorted(ids)
    masses = {law.ids[i]: law.cdf[i + 1] - law.cdf[i] for i in range(law.count)}
    srt = sorted(((float(logits[t]), t) for t in toks), key=lambda v: (-v[0], v[1]))
    cutoff = srt[39][0]
    srt = [v for v in srt if v[0] >= cutoff]
    w = [math.exp(v[0] - srt[0][0]) for v in srt]
    total, tail, keep = sum(w), 0.0, {}
    for i in range(len(srt) - 1, -1, -1):
        tail += w[i]
        if i == 0 or (tail / total > 1.0 - float(np.float32(0.87)) and w[i] >= float(np.float32(0.05))):
            keep[srt[i][1]] = w[i]
    z = sum(keep.values())
    for t in toks:
        assert abs(masses.get(t, 0) / TOTAL - keep.get(t, 0.0) / z) < 1e-6
        if t not in keep:
            assert masses.get(t, 0) == 0
    # tie overflow: 256 ties stay compact, 257 overflow to the full path
    for count, want_rc in ((256, 0), (257, 1), (64, 0)):
        logits = np.full(vocab, -100.0, np.float32)
        logits[:count] = 0.0
        rc, law = gfo.draft_law_compact(logits, opts(gfo, t=1.0, k=1, p=1.0))
        assert rc == want_rc
        if rc == 0:
            sel = gfo.lib().gfo_draft_select(C.byref(law), C.c_uint32(0xFFFFFFFF))
            assert sel == count - 1
            m = law.cdf[law.count] - law.cdf[law.count - 1]
            assert abs(m / TOTAL - 1.0 / count) < 1e-6
    bad = np.zeros(vocab, np.float32)
    bad[5] = np.nan
    assert gfo.draft_law_compact(bad, opts(gfo, t=1.0, k=4))[0] < 0


def test_full_law_uniform_and_nucleus(gfo):
    vocab = 262144
    logits = np.zeros(vocab, np.float32)
    rc, cdf = gfo.draft_law_full(logits, opts(gfo, t=1.0, k=1, p=1.0))
    assert rc == 0
    assert np.all(np.diff(cdf.astype(np.int64)) == 16384) and int(cdf[-1]) == TOTAL
    assert gfo.lib().gfo_draft_select_full(cdf.ctypes, vocab, C.c_uint32(0xFFFFFFFF)) == vocab - 1
    rc, cdf = gfo.draft_law_full(logits, opts(gfo, t=1.0, k=1, p=0.5))
    assert rc == 0
    d = np.diff(cdf.astype(np.int64))
    assert d[0] == 32768 and d[1] == 32768 and d[-1] == 0 and d[-2] == 0 and d.sum() == TOTAL


def test_full_law_reference_cases(gfo):
    """tests/engine/gemma3_draft_tests.cpp:304-307, 392-403 of the reference, on the oracle's table."""
    vocab = 262144
    logits = np.zeros(vocab, np.float32)
    tiny = np.float32(1.401298464324817e-45)  # denorm_min: nothing but the best entry survives
    rc, cdf = gfo.draft_law_full(logits, opts(gfo, t=1.0, k=1, p=float(tiny)))
    assert rc == 0 and int(cdf[0]) == 0 and int(cdf[1]) == TOTAL
    assert gfo.draft_select_full(cdf, 0) == 0 and gfo.draft_select_full(cdf, 0xFFFFFFFF) == 0
    for count in (256, 257, 64):
        logits = np.full(vocab, -100, np.float32)
        logits[:count] = 0
        rc, cdf = gfo.draft_law_full(logits, opts(gfo, t=1.0, k=1, p=1.0))
        assert rc == 0
        assert gfo.draft_select_full(cdf, 0xFFFFFFFF) == count - 1
        assert int(cdf[count + 1]) - int(cdf[count]) == 0
        assert abs((int(cdf[count]) - int(cdf[count - 1])) / TOTAL - 1.0 / count) < 1e-6


def test_full_law_greedy_is_a_step_at_the_lowest_argmax(gfo):
    rng = np.random.default_rng(5)
    logits = rng.normal(0, 2, 1024).astype(np.float32)
    logits[[300, 17, 900]] = 9.5
    rc, cdf = gfo.draft_law_full(logits, opts(gfo, t=0.0, k=1, p=1.0))
    assert rc == 0
    assert np.all(cdf[:18] == 0) and np.all(cdf[18:] == TOTAL)
    for word in (0, 12345, 0xFFFFFFFF):
        assert gfo.draft_select_full(cdf, word) == 17


def test_full_law_agrees_with_the_compact_law(gfo):
    """Two independently written paths of the same law: the same support, masses within 1e-6
    (the f32 sums associate differently, so the tables need not be bit-equal)."""
    rng = np.random.default_rng(6)
    for k, p, m in ((64, 0.9, 0.0), (8, 1.0, 0.05), (40, 0.87, 0.05), (1, 1.0, 0.0)):
        logits = rng.normal(0, 2, 4096).astype(np.float32)
        o = opts(gfo, t=0.8, k=k, p=p, m=m)
        rc, law = gfo.draft_law_compact(logits, o)
        assert rc == 0
        rc, cdf = gfo.draft_law_full(logits, o)
        assert rc == 0
        mass = np.diff(cdf.astype(np.int64))
        support = np.nonzero(mass)[0]
        ids = np.array(law.ids[:law.count])
        cm = np.diff(np.array(law.cdf[:law.count + 1], dtype=np.int64))
        assert list(support) == list(ids[cm > 0])
        assert np.max(np.abs(mass[ids] - cm)) / TOTAL < 1e-6


def reverse_map(draft_to_target, target_vocab):
    t2d = np.full(target_vocab, -1, np.int32)
    for d, t in enumerate(draft_to_target):
        if t >= 0:
            assert t2d[t] < 0   # injective
            t2d[t] = d
    return t2d


def test_mapped_law_reference_case(gfo):
    """tests/engine/gemma3_draft_tests.cpp:404-425: a compact receipt lives in draft-id order; masses are looked up
    by target id through the map, an excluded control token gets no mass, and a NaN in an excluded raw logit
    still refuses."""
    vocab = 262144
    d2t = np.arange(vocab, dtype=np.int32)
    d2t[12], d2t[50000] = d2t[50000], d2t[12]
    d2t[0] = -1
    t2d = reverse_map(d2t, vocab)
    logits = np.full(vocab, -100, np.float32)
    logits[0], logits[12], logits[511] = 100, 0, 0
    opt = gfo.SamplerOptions(1.0, 1, 1.0, 0.0, 1.0)
    rc, law = gfo.draft_law_compact_mapped(logits, opt, d2t)
    half = 1 << 31
    assert rc == 0 and law.count == 2 and [law.ids[0], law.ids[1]] == [12, 511]
    assert [law.cdf[i] for i in range(3)] == [0, half, 2 * half]
    lib = gfo.lib()
    lib.gfo_law_mass_mapped.restype = C.c_uint64
    def mass(token):
        begin = C.c_uint64(0)
        m = lib.gfo_law_mass_mapped(C.byref(law), t2d.ctypes.data_as(C.c_void_p), C.c_uint32(token), C.byref(begin))
        return m, begin.value
    left = lib.gfo_draft_select(C.byref(law), C.c_uint32(0))
    assert left == 12 and d2t[left] == 50000 and mass(50000) == (half, 0)
    assert mass(0)[0] == 0 and mass(12)[0] == 0 and mass(511) == (half, half)
    right = lib.gfo_draft_select(C.byref(law), C.c_uint32(0xFFFFFFFF))
    assert right == 511 and d2t[right] == 511
    logits[0] = np.nan
    assert gfo.draft_law_compact_mapped(logits, opt, d2t)[0] == -10


def test_full_mapped_law_suppresses_unmapped_tokens_and_agrees_with_the_compact_one(gfo):
    """The full-vocabulary law behind a vocabulary map: the reference's mapped case (an excluded control token
    with the best logit gets no mass; a NaN in an excluded raw logit still refuses), the compact mapped law as a
    second path to the same masses, the double-precision rule over the mapped tokens only, and greedy drafting
    landing on the best MAPPED token."""
    from law_brute import law as brute_law
    vocab = 4096
    rng = np.random.default_rng(12)
    d2t = rng.permutation(vocab).astype(np.int32)
    d2t[rng.choice(vocab, 300, replace=False)] = -1
    logits = rng.normal(0, 2, vocab).astype(np.float32)
    logits[np.nonzero(d2t < 0)[0][:3]] = 50.0          # unmapped tokens with the best logits by far
    for t, k, p, m in ((0.8, 40, 0.9, 0.0), (1.0, 64, 1.0, 0.05), (1.2, 200, 0.95, 0.0), (0.7, 256, 1.0, 0.0)):
        o = opts(gfo, t=t, k=k, p=p, m=m)
        rc, cdf = gfo.draft_law_full_mapped(logits, o, d2t)
        assert rc == 0
        mass = np.diff(cdf.astype(np.int64))
        assert mass.sum() == TOTAL and not mass[d2t < 0].any()
        mapped = np.nonzero(d2t >= 0)[0]
        want, margin = brute_law(logits[mapped], t, k, p, m)       # the rule over the tokens that exist
        assert margin > 1e-5
        for i, w in want.items():
            assert abs(mass[mapped[i]] / TOTAL - w) <= 1e-6
        assert np.count_nonzero(mass) <= len(want)
        if k <= 64:
            rc, law = gfo.draft_law_compact_mapped(logits, o, d2t)
            assert rc == 0
            ids = np.array(law.ids[:law.count])
            cm = np.diff(np.array(law.cdf[:law.count + 1], dtype=np.int64))
            assert list(np.nonzero(mass)[0]) == list(ids[cm > 0])
            assert np.max(np.abs(mass[ids] - cm)) / TOTAL < 1e-6
    rc, cdf = gfo.draft_law_full_mapped(logits, opts(gfo, t=0.0, k=1, p=1.0, m=0.0), d2t)
    best_mapped = mapped[np.argmax(logits[mapped])]
    assert rc == 0 and gfo.draft_select_full(cdf, 12345) == best_mapped and d2t[best_mapped] >= 0
    broken = logits.copy()
    broken[np.nonzero(d2t < 0)[0][0]] = np.nan
    assert gfo.draft_law_full_mapped(broken, opts(gfo, k=100), d2t)[0] == -10
    assert gfo.draft_law_full_mapped(logits, opts(gfo, k=100), np.full(vocab, -1, np.int32))[0] != 0   # nothing left to propose
