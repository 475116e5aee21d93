"""The acceptance kernel on the reference's sampler cases restated as data (tests/accept_cases.py): every
decision, probability and failure code equals the oracle's (tests/test_oracle_accept_cases.py holds the oracle to
the reference's own expectations), and the 32 000-token proposal table of
tests/engine/lossless_sampling_tests.cpp:375-432 gathered on the device."""
import numpy as np
import pytest

import accept_cases as cases
from test_oracle_accept_cases import run as oracle_run

pytestmark = pytest.mark.gpu

STATUS_LAW_INVALID = 16


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def device_run(hip, case, cdf=None):
    import torch
    cands = np.zeros(2, hip.candidates_dtype)
    for r, row in enumerate(case["rows"]):
        cands[r]["count"] = len(row)
        for i, (token, logit) in enumerate(row):
            cands[r]["values"]["token"][i] = token
            cands[r]["values"]["logit"][i] = logit
    hist = np.zeros((2, 64), np.uint32)
    counts = np.zeros(2, np.uint32)
    for r, h in enumerate(case["history"]):
        hist[r, :len(h)] = h
        counts[r] = len(h)
    law = cases.law_record(hip.law_dtype, case["law"], case.get("edit"))
    draws = np.zeros(1, hip.draws_dtype)
    draws[0]["u_accept"], draws[0]["u_residual"], draws[0]["u_next"] = case["draws"]
    up = lambda a: torch.from_numpy(a.view(np.uint8).reshape(-1)).cuda()
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    proposal = torch.tensor([case["proposal"]], dtype=torch.int64, device="cuda").to(torch.int32)
    options = hip.SamplerOptions(*case["options"])
    if cdf is not None:
        out = hip.spec_accept_law(up(cands), up(law), cdf, proposal, options, draws=up(draws), status=status)
    else:
        out = hip.spec_accept_history(up(cands), up(law), up(hist), up(counts), proposal, options, draws=up(draws), status=status)
    return out.cpu().numpy().view(hip.result_dtype)[0], int(status[0])


def same(got, want):
    assert (int(got["accepted"]), int(got["token"]), int(got["next_root"])) == (want.accepted, want.token, want.next_root)
    assert float(got["acceptance_probability"]) == want.acceptance_probability
    assert float(got["residual_total"]) == want.residual_total
    assert int(got["residual_count"]) == want.residual_count


@pytest.mark.parametrize("family", ["transforms", "greedy", "unit_bins", "rollback"])
def test_reference_cases_equal_the_oracle(hip, gfo, family):
    todo = {"transforms": cases.transform_cases, "greedy": cases.greedy_cases, "unit_bins": cases.unit_bin_cases,
            "rollback": cases.rollback_cases}[family]()
    for case in todo:
        rc, want = oracle_run(gfo, case)
        got, status = device_run(hip, case)
        assert rc == 0 and int(got["status"]) == 0 and status == 0, (case["proposal"], case["options"])
        same(got, want)
        if "want" in case:
            assert (int(got["accepted"]), int(got["token"])) == case["want"]


def test_fault_cases_fail_closed_with_the_oracles_codes(hip, gfo):
    for case in cases.fault_cases():
        got, status = device_run(hip, case)
        assert int(got["status"]) == case["code"], (case["proposal"], case["draws"], case["options"], int(got["status"]))
        assert status & STATUS_LAW_INVALID
        assert int(got["accepted"]) == 0 and int(got["token"]) == 0xFFFFFFFF and int(got["next_root"]) == 0xFFFFFFFF


def test_sparse_target_against_a_32000_token_table(hip, gfo):
    """Every 7th proposal of the uniform 32 000-token law (and the tokens of the target's support, one of which
    the table does not have) gathered from the full table on the device, against the oracle."""
    import math
    import torch
    vocabulary = 32000
    cdf = (np.arange(vocabulary + 1, dtype=np.uint64) * np.uint64(1 << 32)) // np.uint64(vocabulary)
    cdf_dev = torch.from_numpy(cdf.view(np.int64)).cuda()
    row = [(40000, math.log(0.5)), (999, math.log(0.375)), (0, math.log(0.125))]
    o = (1.0, 3, 1.0, 0.0, 1.0)
    full = lambda law: law.__setitem__("count", 0xFFFFFFFF)
    for x in sorted(set(range(0, vocabulary, 7)) | {0, 17, 999, vocabulary - 1}):
        for ur in (0.0, 0.99):
            case = dict(rows=[row, row], history=[[], []], law=[], edit=full, proposal=x, options=o, draws=(0.3, ur, 0.5))
            got, status = device_run(hip, case, cdf_dev)
            rc, want = gfo.spec_accept_full(np.array(row, gfo.token_logit), np.array(row, gfo.token_logit), cdf, x,
                                            gfo.SamplerOptions(*o), 0.3, ur, 0.5)
            assert rc == 0 and int(got["status"]) == 0 and status == 0, x
            same(got, want)
    # a proposal the table does not have has no mass: refused
    case = dict(rows=[row, row], history=[[], []], law=[], edit=full, proposal=40000, options=o, draws=(0.3, 0.5, 0.5))
    got, status = device_run(hip, case, cdf_dev)
    assert int(got["status"]) == 22 and status & STATUS_LAW_INVALID
