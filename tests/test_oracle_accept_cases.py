"""The oracle's acceptance on the reference's sampler cases restated as data (tests/accept_cases.py): the
reference's own expectations, its failure rules, and the exact-marginal identity that makes the scheme lossless."""
import ctypes as C
import math

import numpy as np
import pytest

import accept_cases as cases


def run(gfo, case):
    rows = [np.array(r, gfo.token_logit) if r else np.zeros(0, gfo.token_logit) for r in case["rows"]]
    hist = [np.array(h, np.uint32) for h in case["history"]]
    law_np = cases.law_record(np.dtype([("count", np.uint32), ("pad", np.uint32), ("ids", np.uint32, (256,)),
                                        ("cdf", np.uint64, (257,))]), case["law"], case.get("edit"))
    law = gfo.DraftLaw.from_buffer_copy(law_np.tobytes())
    ua, ur, un = case["draws"]
    return gfo.spec_accept_history(rows[0], hist[0], rows[1], hist[1], law, case["proposal"], gfo.SamplerOptions(*case["options"]),
                                   ua, ur, un)


@pytest.mark.parametrize("family", ["transforms", "greedy", "unit_bins", "rollback"])
def test_reference_cases_decide_as_the_reference_expects(gfo, family):
    todo = {"transforms": cases.transform_cases, "greedy": cases.greedy_cases, "unit_bins": cases.unit_bin_cases,
            "rollback": cases.rollback_cases}[family]()
    accepted = 0
    for case in todo:
        rc, got = run(gfo, case)
        assert rc == 0, (case["proposal"], case["options"], rc)
        if "want" in case:
            assert (got.accepted, got.token) == case["want"]
        if "acceptance" in case:
            assert got.acceptance_probability == case["acceptance"] and got.residual_count == case["residual_count"]
        if "residual_total" in case:
            assert math.isclose(got.residual_total, case["residual_total"], rel_tol=0, abs_tol=1e-15)
        accepted += got.accepted
    if family in ("transforms", "rollback"):
        assert 0 < accepted < len(todo)


@pytest.mark.parametrize("options", [(0.6, 4, 0.8, 0.05, 1.2), (1.3, 3, 1.0, 0.4, 0.7)])
def test_target_transforms_keep_the_marginal_exact(gfo, options):
    """lossless_sampling_tests.cpp:215-233 (check_exact_marginal): whatever the target sampler's transforms make
    of the logits, accepting with min(1, p/q) and correcting with max(p - q, 0) returns exactly that law."""
    logits = [(0, 1.0), (1, 0.7), (2, 0.3), (3, -2.0), (0, 1.0)]
    rc, p = gfo.prepare(np.array(logits, gfo.token_logit), gfo.SamplerOptions(*options), history=[0])
    assert rc == 0
    prob = {p.token[i]: p.probability[i] for i in range(p.count)}
    assert abs(sum(prob.values()) - 1.0) < 1e-15 and 1 <= len(prob) < 4     # the filters removed something

    def accept(x):
        case = dict(rows=[logits, logits], history=[[0], [0]], law=cases.uniform4(), proposal=x, options=options,
                    draws=(0.0, 0.0, 0.0))
        rc, got = run(gfo, case)
        assert rc == 0
        return got.acceptance_probability, got.residual_total, got.residual_count

    cases.check_exact_marginal(prob, cases.uniform4(), accept)


def test_malformed_laws_rows_and_draws_fail_closed(gfo):
    for case in cases.fault_cases():
        rc, got = run(gfo, case)
        assert rc == -case["code"], (case.get("edit"), case["proposal"], case["draws"], case["options"], rc)
