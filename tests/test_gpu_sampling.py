"""GPU parity of head selection, the proposal law and lossless acceptance.

Bars: candidate lists, argmax ids, integer CDF bins, proposals and accept / residual /
next-root decisions bit-exact against the CPU oracle given the same logits and draws.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOTAL = 1 << 32
VOCAB = 262144


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def opts(mod, t=1.0, k=64, p=0.95, m=0.0, r=1.0):
    return mod.SamplerOptions(t, k, p, m, r)


def test_step_draws_match_oracle_schedule(hip, gfo):
    for seed, step in ((0, 0), (7, 5), (2 ** 40 + 3, 2 ** 33 + 9)):
        d = hip.step_draws(seed, step)
        w, a, r, n = gfo.step_draws(seed, step)
        assert (int(d["word"]), float(d["u_accept"]), float(d["u_residual"]), float(d["u_next"])) == (w, a, r, n)


def test_selection_reference_tie_and_history_case(hip):
    logits = np.full((1, 1025), -2.0, np.float32)
    logits[0, 1000] = logits[0, 1001] = 101.0
    logits[0, 1010] = 100.0
    logits[0, 7] = -99.75
    hist = np.zeros((1, 64), np.uint32)
    hist[0, 0] = 7
    res, status = hip.select_candidates(dev(logits), 3, dev(hist), dev(np.array([1], np.uint32)))
    c = hip.candidates_to_numpy(res)[0]
    assert c["count"] == 4 and int(status[0]) == 0
    assert list(c["values"]["token"][:4]) == [1000, 1001, 1010, 7]
    assert list(c["values"]["logit"][:4]) == [101.0, 101.0, 100.0, -99.75]
    tok, lg = hip.argmax(dev(logits))
    assert int(tok[0]) == 1000 and float(lg[0]) == 101.0


@pytest.mark.parametrize("retain", [1, 64, 257, 320])
def test_selection_matches_oracle_on_full_vocabulary(hip, gfo, retain):
    rng = np.random.default_rng(retain)
    logits = rng.normal(0, 3, (2, VOCAB)).astype(np.float32)
    logits[0, rng.integers(0, VOCAB, 4000)] = logits[0, 12345]      # many exact ties
    logits[1, :500] = logits[1].max() + 1.0                          # a tie plateau at the top
    res, status = hip.select_candidates(dev(logits), retain)
    c = hip.candidates_to_numpy(res)
    for row in range(2):
        want = gfo.select_candidates(logits[row], retain)
        assert c[row]["count"] == retain
        assert np.array_equal(c[row]["values"]["token"][:retain], want["token"])
        assert np.array_equal(c[row]["values"]["logit"][:retain].view(np.uint32), want["logit"].view(np.uint32))
    tok, _ = hip.argmax(dev(logits))
    assert [int(t) for t in tok] == [gfo.lib().gfo_argmax(logits[r].ctypes, VOCAB) for r in range(2)]


@pytest.mark.parametrize("vocab,retain,shape", [
    (VOCAB, 64, "uniform"),          # every logit ties: the collected list overflows, the whole-row select decides
    (VOCAB, 64, "plateau1500"),      # 1500 logits tie at the top: the list is sorted as a whole
    (VOCAB, 257, "plateau1500"),
    (200003, 64, "normal"),          # a ragged last segment and a ragged last tile
    (200003, 100, "clustered"),      # the best logits sit in a few segments: the bound is loose
    (131072, 256, "normal"),         # exactly twice as many segments as kept entries
    (65536, 128, "normal"),
    (65536, 129, "normal"),          # one entry too many for the bound: sorted tiles serve the call
])
def test_selection_paths_of_large_vocabularies(hip, gfo, vocab, retain, shape):
    rng = np.random.default_rng(vocab + retain)
    logits = rng.normal(0, 3, (2, vocab)).astype(np.float32)
    if shape == "uniform":
        logits[0, :] = 1.25
        logits[1, :] = -0.0
        logits[1, ::2] = 0.0          # both zeros order as one value, ties go to the lower id
    elif shape == "plateau1500":
        logits[0, rng.choice(vocab, 1500, replace=False)] = 40.0
        logits[1, 1000:2500] = 40.0
    elif shape == "clustered":
        logits[0, 5000:5600] += 30.0
        logits[1, vocab - 700:] += 30.0
    res, status = hip.select_candidates(dev(logits), retain)
    c = hip.candidates_to_numpy(res)
    assert int(status[0]) == 0 and int(status[1]) == 0
    for row in range(2):
        want = gfo.select_candidates(logits[row], retain)
        assert c[row]["count"] == retain
        assert np.array_equal(c[row]["values"]["token"][:retain], want["token"])
        assert np.array_equal(c[row]["values"]["logit"][:retain].view(np.uint32), want["logit"].view(np.uint32))


def test_selection_of_a_large_vocabulary_with_histories_and_row_counts(hip, gfo):
    """Rows that keep different numbers of entries and append their own history tokens' logits, twice in a
    row on one workspace-sized call each (the counters of the first call must not leak into the second)."""
    rng = np.random.default_rng(77)
    for trial in range(2):
        logits = rng.normal(0, 2, (2, VOCAB)).astype(np.float32)
        hist = np.zeros((2, 64), np.uint32)
        counts = np.array([5, 64], np.uint32)
        hist[0, :5] = rng.integers(0, VOCAB, 5)
        hist[1] = rng.integers(0, VOCAB, 64)
        res, status = hip.select_candidates(dev(logits), 64 + trial, history=dev(hist), history_count=dev(counts))
        c = hip.candidates_to_numpy(res)
        for row in range(2):
            want = gfo.select_candidates(logits[row], 64 + trial, hist[row, :counts[row]])
            n = 64 + trial + int(counts[row])
            assert c[row]["count"] == n and int(status[row]) == 0
            assert np.array_equal(c[row]["values"]["token"][:n], want["token"])
            assert np.array_equal(c[row]["values"]["logit"][:n].view(np.uint32), want["logit"].view(np.uint32))


def test_selection_flags_non_finite_logits(hip):
    logits = np.zeros((2, 4096), np.float32)
    logits[1, 77] = np.inf
    _, status = hip.select_candidates(dev(logits), 8)
    assert int(status[0]) == 0 and int(status[1]) & 2
    logits = np.zeros((2, VOCAB), np.float32)
    logits[0, VOCAB - 1] = np.nan
    _, status = hip.select_candidates(dev(logits), 8)
    assert int(status[0]) & 2 and int(status[1]) == 0


def law_np(hip, law):
    return law.cpu().numpy().view(hip.law_dtype)[0]


def check_law(hip, gfo, logits, o_gpu, o_cpu, word):
    import torch
    draws = np.zeros(1, hip.draws_dtype)
    draws["word"] = word
    draws["u_accept"], draws["u_residual"], draws["u_next"] = 0.5, 0.5, 0.5
    law, proposal, status = hip.draft_law(dev(logits), o_gpu, draws=dev(draws.view(np.uint8)))
    rc, want = gfo.draft_law_compact(logits, o_cpu)
    if rc != 0:
        assert int(status[0]) & 16
        return None
    got = law_np(hip, law)
    assert int(status[0]) == 0
    assert got["count"] == want.count
    assert list(got["ids"][:want.count]) == [want.ids[i] for i in range(want.count)]
    assert list(got["cdf"][:want.count + 1]) == [want.cdf[i] for i in range(want.count + 1)]
    assert int(proposal[0]) & 0xFFFFFFFF == gfo.lib().gfo_draft_select(C.byref(want), C.c_uint32(word))
    return got


def test_draft_law_bit_exact_against_oracle(hip, gfo):
    rng = np.random.default_rng(5)
    for trial in range(12):
        logits = rng.normal(0, 2, VOCAB).astype(np.float32)
        k = int(rng.choice([1, 8, 40, 64]))
        t = float(rng.choice([0.7, 1.0, 1.3]))
        p = float(rng.choice([0.5, 0.9, 0.95, 1.0]))
        m = float(rng.choice([0.0, 0.05]))
        got = check_law(hip, gfo, logits, opts(hip, t, k, p, m), opts(gfo, t, k, p, m),
                        int(rng.integers(0, 2 ** 32)))
        assert got is not None and int(got["cdf"][got["count"]]) == TOTAL


def test_draft_law_reference_fixtures(hip, gfo):
    # tests/engine/gemma3_draft_tests.cpp:332-362 (48 candidates in different tiles, cutoff ties)
    logits = np.full(VOCAB, -100.0, np.float32)
    for i in range(48):
        logits[37 + i * 4099] = 4.0 - i * 0.07 if i < 38 else 1.34
    got = check_law(hip, gfo, logits, opts(hip, 1.0, 40, 0.87, 0.05), opts(gfo, 1.0, 40, 0.87, 0.05), 123456789)
    assert got is not None
    # :366-375 cutoff ties: 256 stay compact, 257 overflow, 64 compact
    for count in (256, 257, 64):
        logits = np.full(VOCAB, -100.0, np.float32)
        logits[:count] = 0.0
        got = check_law(hip, gfo, logits, opts(hip, 1.0, 1, 1.0, 0.0), opts(gfo, 1.0, 1, 1.0, 0.0), 0xFFFFFFFF)
        if count == 257:
            assert got is None
        else:
            mass = int(got["cdf"][count]) - int(got["cdf"][count - 1])
            assert abs(mass / TOTAL - 1.0 / count) < 1e-6
    bad = np.zeros(VOCAB, np.float32)
    bad[5] = np.nan
    _, _, status = hip.draft_law(dev(bad), opts(hip, 1.0, 4, 1.0, 0.0))
    assert int(status[0]) & 16


def cdf_margin(weights, draw):
    """Relative distance of `draw` (in [0, total)) from the nearest bin edge of the running sum of `weights`:
    how far a draw is from selecting a neighbouring token."""
    edges = np.cumsum(np.asarray(weights, np.float64))
    return float(np.min(np.abs(edges[:-1] - draw)) / edges[-1]) if edges.size > 1 else 1.0


def decision_margins(gfo, prepared, law, want, ua, ur, un):
    """(margin of the accept decision, margin of the token draw that follows it) for one step."""
    total = float(1 << 32)
    if want.accepted:
        nxt = prepared[1]
        weights = [nxt.sampling_weight[i] for i in range(nxt.count)]
        return abs(ua - want.acceptance_probability), cdf_margin(weights, un * nxt.total_sampling_weight)
    tgt = prepared[0]
    mass = {law.ids[i]: (law.cdf[i + 1] - law.cdf[i]) / total for i in range(law.count)}
    norm = sum(tgt.sampling_weight[i] for i in range(tgt.count))
    residual = [tgt.sampling_weight[i] / norm - mass.get(tgt.token[i], 0.0) for i in range(tgt.count)]
    residual = [d for d in residual if d > 0.0]
    assert len(residual) == want.residual_count
    return abs(ua - want.acceptance_probability), cdf_margin(residual, ur * sum(residual))


def run_steps(hip, gfo, p_logits, q_logits, steps, seed, o_gpu, o_cpu, margins=None):
    """steps of draft-law + accept on the GPU against the oracle; returns (accepted, rejected).  With a
    `margins` list, the smallest accept and draw margins of the run are appended to it."""
    import torch
    sets = p_logits.shape[0]
    cands, laws_cpu, cands_cpu = [], [], []
    for s in range(sets):
        res, status = hip.select_candidates(dev(p_logits[s]), o_gpu.top_k)
        assert int(status.abs().sum()) == 0
        cands.append(res)
        rc, law = gfo.draft_law_compact(q_logits[s], o_cpu)
        assert rc == 0
        laws_cpu.append(law)
        c = hip.candidates_to_numpy(res)
        for row in range(2):   # the GPU's selection equals the oracle's on the same logits
            want = gfo.select_candidates(p_logits[s, row], o_gpu.top_k)
            assert np.array_equal(c[row]["values"]["token"][:want.size], want["token"])
        cands_cpu.append([gfo.select_candidates(p_logits[s, r], o_gpu.top_k) for r in range(2)])
    prepared = [[gfo.prepare(cands_cpu[s][r], o_cpu)[1] for r in range(2)] for s in range(sets)]
    least_accept = least_draw = 1.0
    q_dev = [dev(q_logits[s]) for s in range(sets)]
    results = torch.zeros(steps * hip.result_dtype.itemsize, dtype=torch.uint8, device="cuda")
    law = torch.zeros(hip.law_dtype.itemsize, dtype=torch.uint8, device="cuda")
    proposal = torch.zeros(1, dtype=torch.int32, device="cuda")
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    lib = hip.lib()
    lib.guffin_hip_draft_law_workspace_bytes.restype = C.c_uint64
    ws = torch.zeros(lib.guffin_hip_draft_law_workspace_bytes(VOCAB), dtype=torch.uint8, device="cuda")
    size = hip.result_dtype.itemsize
    for step in range(steps):
        s = step % sets
        hip.draft_law(q_dev[s], o_gpu, seed=seed, step=step, law=law, proposal=proposal, status=status, workspace=ws)
        hip.spec_accept(cands[s], law, proposal, o_gpu, seed=seed, step=step,
                        result=results[step * size:(step + 1) * size], status=status)
    got = results.cpu().numpy().view(hip.result_dtype)
    assert int(status[0]) == 0
    accepted = rejected = 0
    for step in range(steps):
        s = step % sets
        word, ua, ur, un = gfo.step_draws(seed, step)
        prop = gfo.lib().gfo_draft_select(C.byref(laws_cpu[s]), C.c_uint32(word))
        rc, want = gfo.spec_accept(cands_cpu[s][0], cands_cpu[s][1], laws_cpu[s], prop, o_cpu, ua, ur, un)
        assert rc == 0 and got[step]["status"] == 0, (step, rc, got[step]["status"])
        assert got[step]["proposal"] == prop
        assert (got[step]["accepted"], got[step]["token"], got[step]["next_root"]) == \
            (want.accepted, want.token, want.next_root), step
        assert got[step]["residual_count"] == want.residual_count
        # the laws' doubles agree to a few ulp (device exp vs libm exp); decisions are exact
        assert abs(got[step]["acceptance_probability"] - want.acceptance_probability) <= 1e-14
        accepted += want.accepted
        rejected += 1 - want.accepted
        if margins is not None:
            m_accept, m_draw = decision_margins(gfo, prepared[s], laws_cpu[s], want, ua, ur, un)
            least_accept, least_draw = min(least_accept, m_accept), min(least_draw, m_draw)
    if margins is not None:
        margins += [least_accept, least_draw]
    return accepted, rejected


def test_ten_thousand_seeded_steps_bit_exact(hip, gfo):
    """Config 3: T=1, top-k 64, top-p 0.95, drafter logits N(0,4) independent of the target."""
    rng = np.random.default_rng(2024)
    sets = 8
    p_logits = rng.normal(0, 3, (sets, 2, VOCAB)).astype(np.float32)
    q_logits = rng.normal(0, 2, (sets, VOCAB)).astype(np.float32)
    margins = []
    a, r = run_steps(hip, gfo, p_logits, q_logits, 10000, 0, opts(hip), opts(gfo), margins)
    assert a + r == 10000
    # "bit-exact decisions" must not rest on a near-tie: the device and the oracle agree on the laws' doubles
    # to about 1e-15, and no draw of this run comes within 1e-9 of the edge it is compared with
    print("10000 steps: %d accepted, %d rejected; least |u_accept - a| = %.3e, least draw-to-edge distance = %.3e"
          % (a, r, margins[0], margins[1]))
    assert margins[0] > 1e-9 and margins[1] > 1e-9, margins


def test_correlated_drafter_mixes_accepts_and_rejections(hip, gfo):
    rng = np.random.default_rng(99)
    sets = 8
    p_logits = rng.normal(0, 3, (sets, 2, VOCAB)).astype(np.float32)
    q_logits = (p_logits[:, 0] + rng.normal(0, 1.0, (sets, VOCAB))).astype(np.float32)
    margins = []
    a, r = run_steps(hip, gfo, p_logits, q_logits, 3000, 17, opts(hip), opts(gfo), margins)
    assert a > 300 and r > 300, (a, r)
    # here the acceptance probability is strictly between 0 and 1 on most steps: the accept decisions,
    # the residual draws and the next-root draws all stay clear of their edges
    print("3000 correlated steps: %d accepted, %d rejected; least |u_accept - a| = %.3e, least draw-to-edge distance = %.3e"
          % (a, r, margins[0], margins[1]))
    assert margins[0] > 1e-9 and margins[1] > 1e-9, margins
    a2, r2 = run_steps(hip, gfo, p_logits, q_logits, 500, 18, opts(hip, 0.8, 40, 0.9, 0.05), opts(gfo, 0.8, 40, 0.9, 0.05))
    assert a2 + r2 == 500


def test_spec_accept_fails_closed(hip, gfo):
    import torch
    rng = np.random.default_rng(3)
    p = rng.normal(0, 3, (2, 4096)).astype(np.float32)
    res, _ = hip.select_candidates(dev(p), 64)
    law, proposal, status = hip.draft_law(dev(rng.normal(0, 2, 4096).astype(np.float32)), opts(hip))
    bad_prop = torch.full((1,), 5000, dtype=torch.int32, device="cuda")   # not in q's support
    out = hip.spec_accept(res, law, bad_prop, opts(hip), status=status).cpu().numpy().view(hip.result_dtype)[0]
    assert out["status"] == 22 and int(status[0]) & 16


def test_device_accept_replays_reference_golden_vectors(hip):
    """tests/golden/accept.npz was written from the compiled reference sampling.cpp
    (prepare_speculative_distribution + sample_speculative_token): the device kernel must take the
    same decisions on the same candidate rows, proposal laws and injected draws."""
    import os
    import torch
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "accept.npz"))
    o = hip.SamplerOptions(1.0, 64, 0.95, 0.0, 1.0)
    n = g["proposal"].size
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    accepted = 0
    for i in range(n):
        cands = np.zeros(2, hip.candidates_dtype)
        for r in range(2):
            cands[r]["count"] = 64
            cands[r]["values"]["token"][:64] = g["row_tokens"][i, r]
            cands[r]["values"]["logit"][:64] = g["row_logits"][i, r]
        law = np.zeros(1, hip.law_dtype)
        cnt = int(g["law_count"][i])
        law[0]["count"] = cnt
        law[0]["ids"][:cnt] = g["law_ids"][i, :cnt]
        law[0]["cdf"][:cnt + 1] = g["law_cdf"][i, :cnt + 1]
        draws = np.zeros(1, hip.draws_dtype)
        draws[0]["u_accept"], draws[0]["u_residual"], draws[0]["u_next"] = g["draws"][i]
        out = hip.spec_accept(torch.from_numpy(cands.view(np.uint8)).cuda(), torch.from_numpy(law.view(np.uint8)).cuda(),
                              torch.tensor([int(g["proposal"][i])], dtype=torch.int32, device="cuda"), o,
                              draws=torch.from_numpy(draws.view(np.uint8)).cuda(), status=status)
        got = out.cpu().numpy().view(hip.result_dtype)[0]
        assert got["status"] == 0, i
        assert (int(got["accepted"]), int(got["token"]), int(got["next_root"])) == \
            (int(g["accepted"][i]), int(g["token"][i]), int(g["next_root"][i])), i
        assert abs(float(got["acceptance_probability"]) - float(g["acceptance"][i])) <= 1e-13
        assert int(got["residual_count"]) == int(g["residual_count"][i])
        accepted += int(got["accepted"])
    assert int(status[0]) == 0 and 0 < accepted < n


def test_accept_applies_the_repetition_penalty_to_each_rows_history(hip, gfo):
    """src/engine/sampling.cpp:430-446: history tokens are penalised before the sort, so the candidate
    rows carry top_k + |history| entries plus the history tokens' own logits; decisions equal the oracle's."""
    import torch
    rng = np.random.default_rng(77)
    vocab, k = 8192, 40
    o_gpu, o_cpu = hip.SamplerOptions(0.9, k, 0.95, 0.0, 1.7), gfo.SamplerOptions(0.9, k, 0.95, 0.0, 1.7)
    accepted = rejected = 0
    for trial in range(40):
        p_logits = rng.normal(0, 3, (2, vocab)).astype(np.float32)
        q_logits = (p_logits[0] + rng.normal(0, 1.0, vocab)).astype(np.float32)
        top = np.argsort(-p_logits[0])[:8]                      # penalise some of the very best tokens
        hist0 = np.concatenate([top[:5], rng.integers(0, vocab, 20)]).astype(np.uint32)
        hist1 = np.concatenate([hist0, top[5:6]]).astype(np.uint32)
        hist = np.zeros((2, 64), np.uint32)
        hist[0, :hist0.size], hist[1, :hist1.size] = hist0, hist1
        counts = np.array([hist0.size, hist1.size], np.uint32)
        retain = k + hist1.size
        res, status = hip.select_candidates(dev(p_logits), retain, history=dev(hist), history_count=dev(counts))
        assert int(status.abs().sum()) == 0
        law, proposal, st = hip.draft_law(dev(q_logits), hip.SamplerOptions(0.9, k, 0.95, 0.0, 1.0), seed=3, step=trial)
        out = hip.spec_accept_history(res, law, dev(hist), dev(counts), proposal, o_gpu, seed=3, step=trial, status=st)
        got = out.cpu().numpy().view(hip.result_dtype)[0]
        rc, law_cpu = gfo.draft_law_compact(q_logits, gfo.SamplerOptions(0.9, k, 0.95, 0.0, 1.0))
        word, ua, ur, un = gfo.step_draws(3, trial)
        prop = gfo.lib().gfo_draft_select(C.byref(law_cpu), C.c_uint32(word))
        rows = [gfo.select_candidates(p_logits[0], retain, hist0), gfo.select_candidates(p_logits[1], retain, hist1)]
        rc, want = gfo.spec_accept_history(rows[0], hist0, rows[1], hist1, law_cpu, prop, o_cpu, ua, ur, un)
        assert int(st[0]) == 0 and rc == 0 and got["status"] == 0 and got["proposal"] == prop
        assert (got["accepted"], got["token"], got["next_root"]) == (want.accepted, want.token, want.next_root), trial
        # the penalty matters: without it the decision inputs differ for at least the penalised best token
        accepted += want.accepted
        rejected += 1 - want.accepted
    assert accepted > 0 and rejected > 0


def test_draft_side_repetition_penalty(hip, gfo):
    """src/engine/gemma3_draft.mm:186-204: the drafter penalises the history's tokens before its law is built
    (score < 0 ? score * r : score / r, then the temperature).  The scores equal the same float32 arithmetic in
    numpy bit for bit, and the law built from them equals the oracle's law on those scores."""
    import torch
    rng = np.random.default_rng(123)
    vocab = 16384
    logits = rng.normal(0, 3, vocab).astype(np.float32)
    best = np.argsort(-logits)[:6]
    history = np.concatenate([best[:4], rng.integers(0, vocab, 40), np.argsort(logits)[:2]]).astype(np.uint32)
    r = np.float32(1.6)
    want = logits.copy()
    hit = np.zeros(vocab, bool)
    hit[history] = True
    want[hit & (logits < 0)] = logits[hit & (logits < 0)] * r
    want[hit & (logits >= 0)] = logits[hit & (logits >= 0)] / r
    scores = hip.draft_process(dev(logits), dev(history), float(r))
    assert np.array_equal(scores.cpu().numpy().view(np.uint32), want.view(np.uint32))
    o_gpu, o_cpu = opts(hip, t=0.8, k=40), opts(gfo, t=0.8, k=40)
    for step in range(4):
        word = gfo.step_draws(11, step)[0]
        check_law(hip, gfo, want, o_gpu, o_cpu, word)
        law, proposal, st = hip.draft_law(scores, o_gpu, seed=11, step=step)
        rc, law_cpu = gfo.draft_law_compact(want, o_cpu)
        assert rc == 0 and int(st[0]) == 0
        assert int(proposal[0]) == gfo.lib().gfo_draft_select(C.byref(law_cpu), C.c_uint32(word))
    plain = gfo.draft_law_compact(logits, o_cpu)[1]
    assert bytes(plain) != bytes(law_cpu)   # the penalty moved the law
    with pytest.raises(hip.GuffinError):
        hip.draft_process(dev(logits), dev(np.zeros(65, np.uint32)), 1.5)


def _reverse_map(draft_to_target, target_vocab):
    t2d = np.full(target_vocab, -1, np.int32)
    ok = draft_to_target >= 0
    t2d[draft_to_target[ok]] = np.nonzero(ok)[0].astype(np.int32)
    return t2d


def test_mapped_law_reference_case_on_the_device(hip, gfo):
    """tests/engine/gemma3_draft_tests.cpp:404-425 on the device path: law in draft ids {12, 511} with half the
    mass each, proposals 50000 / 511 in target ids, and a NaN in an excluded raw logit still refuses."""
    vocab = 262144
    d2t = np.arange(vocab, dtype=np.int32)
    d2t[12], d2t[50000] = d2t[50000], d2t[12]
    d2t[0] = -1
    logits = np.full(vocab, -100, np.float32)
    logits[0], logits[12], logits[511] = 100, 0, 0
    o = hip.SamplerOptions(1.0, 1, 1.0, 0.0, 1.0)
    half = 1 << 31
    for word, draft_want, target_want in ((0, 12, 50000), (0xFFFFFFFF, 511, 511)):
        draws = np.zeros(1, hip.draws_dtype)
        draws["word"] = word
        draws["u_accept"], draws["u_residual"], draws["u_next"] = 0.5, 0.5, 0.5
        law, draft, target, status = hip.draft_law_mapped(dev(logits), dev(d2t), o, draws=dev(draws.view(np.uint8)))
        got = law_np(hip, law)
        assert int(status[0]) == 0 and got["count"] == 2
        assert list(got["ids"][:2]) == [12, 511] and list(got["cdf"][:3]) == [0, half, 2 * half]
        assert int(draft[0]) == draft_want and int(target[0]) == target_want
    logits[0] = np.nan
    status = hip.draft_law_mapped(dev(logits), dev(d2t), o)[3]
    assert int(status[0]) & 2


def test_mapped_law_and_accept_against_the_oracle(hip, gfo):
    """A drafter vocabulary that is a shuffled, partly unmapped view of the target's: the law (draft ids), the
    proposal in both id spaces and every accept / residual decision equal the oracle's with the same maps."""
    import torch
    rng = np.random.default_rng(321)
    vocab, k = 8192, 24
    perm = rng.permutation(vocab).astype(np.int32)
    d2t = perm.copy()
    d2t[rng.choice(vocab, 700, replace=False)] = -1            # draft tokens the target does not have
    t2d = _reverse_map(d2t, vocab)
    o_gpu, o_cpu = hip.SamplerOptions(0.9, k, 0.95, 0.0, 1.3), gfo.SamplerOptions(0.9, k, 0.95, 0.0, 1.3)
    accepted = rejected = unmapped_best = 0
    for trial in range(30):
        p_logits = rng.normal(0, 3, (2, vocab)).astype(np.float32)
        # the drafter sees the target's row 0 through the map, plus noise
        q_logits = np.where(d2t >= 0, p_logits[0][np.maximum(d2t, 0)], 0).astype(np.float32) + rng.normal(0, 1, vocab).astype(np.float32)
        unmapped_best += int(d2t[int(np.argmax(q_logits))] < 0)
        hist_draft = rng.integers(0, vocab, 12).astype(np.uint32)           # draft-side history, draft ids
        law, draft, target, st = hip.draft_law_mapped(dev(q_logits), dev(d2t), o_gpu, history=dev(hist_draft), seed=5, step=trial)
        r = np.float32(1.3)
        scores = q_logits.copy()
        hit = np.zeros(vocab, bool)
        hit[hist_draft] = True
        scores[hit] = np.where(scores[hit] < 0, scores[hit] * r, scores[hit] / r)
        rc, law_cpu = gfo.draft_law_compact_mapped(scores, o_cpu, d2t)
        word, ua, ur, un = gfo.step_draws(5, trial)
        d_want = gfo.lib().gfo_draft_select(C.byref(law_cpu), C.c_uint32(word))
        got = law_np(hip, law)
        assert rc == 0 and int(st[0]) == 0 and got["count"] == law_cpu.count
        assert list(got["ids"][:law_cpu.count]) == [law_cpu.ids[i] for i in range(law_cpu.count)]
        assert list(got["cdf"][:law_cpu.count + 1]) == [law_cpu.cdf[i] for i in range(law_cpu.count + 1)]
        assert all(d2t[i] >= 0 for i in got["ids"][:law_cpu.count])
        assert int(draft[0]) == d_want and int(target[0]) == d2t[d_want]
        res, status = hip.select_candidates(dev(p_logits), k)
        out = hip.spec_accept_mapped(res, law, dev(t2d), target, o_gpu, seed=5, step=trial, status=st)
        g = out.cpu().numpy().view(hip.result_dtype)[0]
        rows = [gfo.select_candidates(p_logits[i], k) for i in range(2)]
        rc, want = gfo.spec_accept_mapped(rows[0], (), rows[1], (), law_cpu, t2d, int(d2t[d_want]), o_cpu, ua, ur, un)
        assert rc == 0 and g["status"] == 0 and int(st[0]) == 0
        assert (g["accepted"], g["token"], g["next_root"]) == (want.accepted, want.token, want.next_root), trial
        assert abs(g["acceptance_probability"] - want.acceptance_probability) <= 1e-14
        accepted += want.accepted
        rejected += 1 - want.accepted
    assert accepted > 0 and rejected > 0
