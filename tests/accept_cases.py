"""Acceptance cases restated as data from the reference's sampler tests
(tests/engine/lossless_sampling_tests.cpp), shared by the oracle's CPU test and the device's GPU test.

A case is a dict:
  rows      two candidate rows, each a list of (token, logit) in the order the selection emits them
            (best first, then the history tokens' own logits)
  history   two lists of distinct history tokens (row 0, row 1)
  law       compact proposal law as (token, mass) pairs in ascending token order, masses in units of 2^-32
  edit      optional function applied to the law record (numpy, hip.law_dtype layout) to break it
  proposal  the proposed token
  options   (temperature, top_k, top_p, min_p, repetition_penalty)
  draws     (u_accept, u_residual, u_next)
  want      optional (accepted, token) fixed by the reference's own expectation
  code      optional failure code the reference's rule implies (the kernel's and the oracle's numbering)
"""
import math

TOTAL = 1 << 32
U64_MAX = (1 << 64) - 1


def law_record(dtype, pairs, edit=None):
    import numpy as np
    law = np.zeros(1, dtype)
    law[0]["count"] = len(pairs)
    at = 0
    for i, (token, mass) in enumerate(pairs):
        law[0]["ids"][i] = token
        law[0]["cdf"][i] = at
        at += mass
    law[0]["cdf"][len(pairs)] = at
    if edit:
        edit(law[0])
    return law


def uniform4():
    return [(t, TOTAL // 4) for t in range(4)]


def transform_cases():
    """lossless_sampling_tests.cpp:215-245: temperature, top-k, top-p, min-p and the repetition penalty of the
    target sampler all act before the acceptance test; history {2, 0, 0} with a window of 2 is {0}."""
    logits = [(0, 1.0), (1, 0.7), (2, 0.3), (3, -2.0)]
    out = []
    for options in ((0.6, 4, 0.8, 0.05, 1.2), (1.3, 3, 1.0, 0.4, 0.7)):
        for proposal in range(4):
            for ua in (0.0, 0.2, 0.45, 0.7, 0.95):
                for ur in (0.05, 0.5, 0.93):
                    out.append(dict(rows=[logits + [(0, 1.0)], logits + [(0, 1.0)]], history=[[0], [0]], law=uniform4(),
                                    proposal=proposal, options=options, draws=(ua, ur, 0.3)))
    return out


def greedy_cases():
    """:328-345: a greedy target keeps its argmax whatever is proposed, and the acceptance draw plays no part."""
    out = []
    for proposal in (3, 7):
        for ua in (0.0, 0.5, 0.999999):
            out.append(dict(rows=[[(3, 1.0), (7, 0.0)]] * 2, history=[[], []], law=[(proposal, TOTAL)], proposal=proposal,
                            options=(0.0, 2, 1.0, 0.0, 1.0), draws=(ua, 0.5, 0.5), want=(int(proposal == 3), 3)))
    return out


def unit_bin_cases():
    """:550-578: 256 target tokens of equal weight against one-word q bins (acceptance 1, all 256 in the residual,
    total 1 - 256 / 2^32), and a 2^32-mass delta (acceptance 1, no residual)."""
    flat = [(t, 0.0) for t in range(256)]
    return [
        dict(rows=[flat, flat], history=[[], []], law=[(t, 1) for t in range(256)], proposal=0,
             options=(1.0, 256, 1.0, 0.0, 1.0), draws=(0.999, 0.5, 0.5), acceptance=1.0, residual_count=256,
             residual_total=1.0 - 256.0 / TOTAL),
        dict(rows=[[(0, 1.0)], [(0, 1.0)]], history=[[], []], law=[(0, TOTAL)], proposal=0,
             options=(1.0, 1, 1.0, 0.0, 1.0), draws=(0.999, 0.5, 0.5), acceptance=1.0, residual_count=0, want=(1, 0)),
    ]


def rollback_cases():
    """:508-548: 23 proposals of the law {0: 1/8, 1: 1/8, 2: 1/4, 7: 1/2} against a three-token target with top-p
    0.9, min-p 0.05, penalty 1.2 on history {1}, greedy and at T = 0.7; token 7 is outside the target's support."""
    law = [(0, TOTAL // 8), (1, TOTAL // 8), (2, TOTAL // 4), (7, TOTAL // 2)]
    logits = [(1, 1.0), (2, 0.8), (0, 0.0), (1, 1.0)]
    out = []
    for temperature in (0.0, 0.7):
        for step in range(23):
            proposal = (0, 1, 2, 7)[step % 4]
            ua, ur, un = (step * 0.61803398875) % 1.0, (step * 0.41421356237) % 1.0, (step * 0.7320508) % 1.0
            out.append(dict(rows=[logits, logits], history=[[1], [1]], law=law, proposal=proposal,
                            options=(temperature, 3, 0.9, 0.05, 1.2), draws=(ua, ur, un)))
    return out


def fault_cases():
    """:170-213 and :458-506, for what reaches the kernel: a proposal law whose masses are not what a law's are,
    a proposal outside q's support, target rows that are not a candidate list, draws outside [0, 1).  Codes:
    20 draws, 22 proposal mass, 23 gathered masses exceed 2^32, 4 non-finite logit, 5 a duplicate with another
    logit, 6 fewer candidates than top-k, 1 options, 2 candidate count."""
    half = [(0, TOTAL // 2), (1, TOTAL // 2)]
    rows = [[(0, 0.0), (1, 0.0)]] * 2
    base = dict(rows=rows, history=[[], []], law=half, proposal=0, options=(0.8, 2, 1.0, 0.0, 1.0), draws=(0.1, 0.1, 0.1))
    out = []

    def with_(code, **kw):
        case = dict(base)
        case.update(kw)
        case["code"] = code
        out.append(case)

    def count_zero(law): law["count"] = 0
    def mass_zero(law): law["cdf"][1] = law["cdf"][0]
    def mass_wraps(law): law["cdf"][0] = 5; law["cdf"][1] = 3            # a "negative" mass: a huge unsigned one
    def begin_beyond(law): law["cdf"][0] = TOTAL; law["cdf"][1] = TOTAL + 7
    def other_huge(law): law["cdf"][2] = U64_MAX                            # token 1's mass
    def other_total(law): law["cdf"][1] = 1; law["cdf"][2] = TOTAL + 1      # token 1 alone has all of 2^32

    with_(22, edit=count_zero)
    with_(22, edit=mass_zero)
    with_(22, edit=mass_wraps)
    with_(22, edit=begin_beyond)
    with_(23, edit=other_huge)
    with_(23, edit=other_total)
    with_(22, proposal=9)                                   # zero-probability proposal
    with_(22, proposal=17)
    for bad in (-1.0, 1.0, float("nan"), float("inf")):
        with_(20, draws=(bad, 0.1, 0.1))
        with_(20, draws=(0.1, bad, 0.1))
        with_(20, draws=(0.1, 0.1, bad))
    with_(4, rows=[[(0, float("nan")), (1, 0.0)]] * 2)
    with_(4, rows=[[(0, 0.0), (1, float("inf"))]] * 2)
    with_(5, rows=[[(0, 0.0), (1, 0.0), (0, 0.5)]] * 2)
    with_(6, rows=[[(0, 0.0), (0, 0.0)]] * 2)               # one distinct candidate for top-k 2
    with_(1, options=(0.8, 0, 1.0, 0.0, 1.0))
    with_(1, options=(0.8, 2, 0.0, 0.0, 1.0))
    with_(1, options=(float("nan"), 2, 1.0, 0.0, 1.0))
    with_(1, options=(0.8, 2, 1.0, 0.0, 0.0))
    with_(2, rows=[[], []])
    return out


def check_exact_marginal(prob, law, accept):
    """sum_x q(x) [a(x) 1{x = t} + (1 - a(x)) r_x(t)] = p(t) for every t of p's support, with accept(x) ->
    (acceptance probability, residual total, residual count) taken from the implementation under test."""
    q = {t: m / TOTAL for t, m in law}
    marginal = {t: 0.0 for t in prob}
    for x, qx in q.items():
        if qx == 0.0:
            continue
        a, total, count = accept(x)
        residual = {t: max(p - q.get(t, 0.0), 0.0) for t, p in prob.items()}
        assert count == sum(1 for r in residual.values() if r > 0.0)
        assert math.isclose(total, sum(residual.values()), rel_tol=0, abs_tol=1e-15)
        for t in prob:
            marginal[t] += (qx * a if t == x else 0.0) + (qx * (1.0 - a) * residual[t] / total if a < 1.0 else 0.0)
    for t, p in prob.items():
        assert abs(marginal[t] - p) <= 1e-12, (t, marginal[t], p)
