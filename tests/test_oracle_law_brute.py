"""The oracle's compact and full proposal laws against a double-precision restatement of the rule
(tests/law_brute.py) on random cases at a 32768-token vocabulary: identical supports, masses within 1e-6.
Cases where a membership decision sits within 1e-5 of its edge are left out (single and double precision
may differ there) and counted."""
import numpy as np

from law_brute import law, random_case

VOCAB = 32768
TOTAL = float(1 << 32)
TINY = 2.0 ** -31      # a kept token below this mass may round to an empty integer bin


def check(masses, want, what, tiny=TINY):
    got = {t: m for t, m in masses.items() if m > 0}
    for token, mass in want.items():
        if mass > tiny:
            assert token in got, (what, "missing", token, mass)
    for token, mass in got.items():
        assert token in want, (what, "extra", token, mass)
        assert abs(mass - want[token]) <= 1e-6, (what, token, mass, want[token])
    assert abs(sum(got.values()) - 1.0) <= 1e-9


def test_compact_law_against_the_double_restatement(gfo):
    rng = np.random.default_rng(2024)
    checked = skipped = overflow = 0
    while checked < 220:
        logits, T, k, p, m = random_case(rng, VOCAB)
        want, margin = law(logits, T, k, p, m)
        if margin < 1e-5:
            skipped += 1
            continue
        rc, got = gfo.draft_law_compact(logits, gfo.SamplerOptions(T, k, p, m, 1.0))
        if rc == 1:            # more than 256 tied entries: the compact law hands over to the full one
            overflow += 1
            continue
        assert rc == 0
        masses = {got.ids[i]: (got.cdf[i + 1] - got.cdf[i]) / TOTAL for i in range(got.count)}
        check(masses, want, (T, k, p, m))
        checked += 1
    assert skipped < checked and overflow < 20


def test_full_law_against_the_double_restatement(gfo):
    rng = np.random.default_rng(77)
    checked = skipped = 0
    while checked < 200:
        logits, T, k, p, m = random_case(rng, VOCAB)
        k = int(rng.choice([k, 100, 200, 256]))         # also beyond the compact law's 64, up to the sampler's 256
        want, margin = law(logits, T, k, p, m)
        if margin < 1e-5:
            skipped += 1
            continue
        rc, cdf = gfo.draft_law_full(logits, gfo.SamplerOptions(T, k, p, m, 1.0))
        assert rc == 0
        bins = np.diff(cdf.astype(np.int64))
        masses = {int(t): bins[t] / TOTAL for t in np.nonzero(bins)[0]}
        # the full table adds float32 prefixes that reach 1: a mass below the tolerance may vanish in their rounding
        check(masses, want, (T, k, p, m), tiny=1e-6)
        checked += 1
    assert skipped < checked
