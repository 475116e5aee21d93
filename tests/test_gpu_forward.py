"""GPU parity of the block graph and of one whole H1 cycle against the CPU oracle.

Bars: hidden rows and logits within 1e-3 of the oracle relative to the row's RMS (the oracle
runs the CPU operators in their sequential fp32 order; fp16 K/V bits may differ on rare
rounding ties, tolerated at 2^-10 as the reference's own stack test does,
tests/engine/gemma3_target_runtime_tests.cpp:310-327); proposal, accept / reject decision,
emitted token and next root bit-exact against the oracle evaluated on the GPU's own logits
with the same Philox draws.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rel_rms(got, want):
    want = want.astype(np.float64)
    scale = np.sqrt((want ** 2).mean(axis=-1, keepdims=True)) + 1e-30
    return float(np.max(np.abs(got.astype(np.float64) - want) / scale))


def check_private_rows(got, want, frac=0.97):
    import torch
    g = got.view(torch.int16).cpu().numpy().view(np.uint16)
    same = np.mean(g == want)
    assert same >= frac, same
    d = np.abs(g.view(np.float16).astype(np.float32) - want.view(np.float16).astype(np.float32))
    scale = np.abs(want.view(np.float16).astype(np.float32)).max()
    assert d.max() <= 2.0 ** -9 * scale + 1e-6


@pytest.mark.parametrize("kind,rows,position", [("drafter", 1, 700), ("drafter", 2, 5), ("target", 2, 1500), ("target", 1, 0)])
def test_forward_rows_matches_oracle(hip, gfo, kind, rows, position):
    import torch
    from dataclasses import replace
    from guffin_amd import model
    if kind == "drafter":
        shape = replace(model.GEMMA3_270M, layers=7, vocab=4096, ring_global=1024)
    else:
        shape = replace(model.GEMMA3_12B, layers=6, vocab=2048, ring_global=2048)
    host = model.HostModel(shape, seed=3, position=position)
    devm = model.DeviceModel.from_host(host)
    tokens = np.array([17, 1999][:rows], np.uint32)
    want, wk, wv = gfo.forward(host, tokens, position, threads=8)
    hidden, sums, pk, pv, status = devm.forward(dev(tokens), position)
    assert int(status.item()) == 0
    assert rel_rms(hidden.cpu().numpy(), want) <= 1e-3
    check_private_rows(pk, wk)
    check_private_rows(pv, wv)
    h = hidden.cpu().numpy().astype(np.float64)
    ref_sums = np.concatenate([h.reshape(rows, -1, 16).sum(-1), h.reshape(rows, -1, 32).sum(-1)], axis=1)
    assert np.allclose(sums.cpu().numpy(), ref_sums, rtol=0, atol=1e-4 * np.abs(h).max() * 4)


def test_drafter_greedy_token_at_full_size_equals_the_oracles_argmax(hip, gfo):
    """The drafter's decode as the benchmark times it (18 blocks, a 4096-token cache, the 262144 x 640 Q8_0
    head, argmax): the greedy token from the device's logits is the argmax of the ORACLE's logits, and the
    oracle's best two logits are further apart than the two sides' logits differ."""
    import torch
    from guffin_amd import model
    shape, position = model.GEMMA3_270M, 4096
    host = model.HostModel(shape, seed=21, position=position, untied_head=True)   # a tied random head would elect the input token
    devm = model.DeviceModel.from_host(host)
    token = np.array([4242], np.uint32)
    want_hidden, _, _ = gfo.forward(host, token, position, threads=8)
    want = gfo.gemv(shape.embed_dtype, host.head, want_hidden, shape.vocab, threads=8)[0]
    hidden, sums, _, _, status = devm.forward(dev(token), position)
    logits = hip.gemv_packed(int(shape.embed_dtype), devm.head_tiles, hidden, sums, shape.vocab)
    got_token, got_logit = hip.argmax(logits)
    assert int(status.item()) == 0
    best, second = np.argsort(-want, kind="stable")[:2]
    margin = float(want[best] - want[second])
    differ = float(np.max(np.abs(logits.cpu().numpy()[0] - want)))
    print("drafter argmax %d, top-2 margin %.4g (logit std %.3g), device and oracle logits differ by at most %.3g"
          % (best, margin, float(want.std()), differ))
    assert margin > 4 * differ          # the election does not rest on the sides' rounding
    assert int(got_token[0]) == int(best) == int(np.argmax(want))


def run_h1(hip, gfo, t_shape, d_shape, t_pos, d_pos, steps, seed, threads=8):
    """`steps` cycles from one root with the benchmark's sampler options.  The two random models are
    unrelated, so the drafter reaches the target through a vocabulary map that lines its 64 best tokens
    up with the target's (built from the first pass's logits): proposals then fall inside the target's
    support and the run sees acceptances and rejections.  Returns the decisions among the rest."""
    import torch
    from guffin_amd import model
    # heads of their own: a random tied head puts nearly all mass on the input token
    t_host = model.HostModel(t_shape, seed=11, position=t_pos, untied_head=True)
    d_host = model.HostModel(d_shape, seed=12, position=d_pos, untied_head=True)
    target = model.DeviceModel.from_host(t_host)
    drafter = model.DeviceModel.from_host(d_host)
    root = 123
    probe = model.H1Plan(target, drafter, t_pos, d_pos, seed=seed, publish=False)
    probe.root.fill_(root)
    probe.step(0)
    torch.cuda.synchronize()
    assert int(probe.status.item()) == 0
    q0, p0 = probe.buffers()["q_logits"].cpu().numpy(), probe.buffers()["p_logits"].cpu().numpy()[0]
    del probe
    # these random models' logits have a spread in the thousands: the output norms are rescaled (on the
    # host and on the device alike) so that both laws spread over many tokens; the ranking, and with it the
    # map below, is unchanged by the positive factor
    for host, devm, logits in ((t_host, target, p0), (d_host, drafter, q0)):
        factor = np.float32(1.5 / logits.std())
        host.out_norm *= factor
        devm.out_norm.copy_(torch.from_numpy(host.out_norm))
    d2t, t2d = gfo.correlating_map(q0, p0, root)
    plan = model.H1Plan(target, drafter, t_pos, d_pos, seed=seed, publish=False, draft_to_target=d2t, target_to_draft=t2d)
    opt_cpu = gfo.SamplerOptions(1.0, 64, 0.95, 0.0, 1.0)
    none = np.zeros(0, np.uint32)
    plan.root.fill_(root)
    decisions, supports = [], []
    for step in range(steps):
        plan.step(step)
        torch.cuda.synchronize()
        bufs = plan.buffers()
        res = plan.read_result()
        assert int(plan.status.item()) == 0 and res["status"] == 0
        # the oracle's decision for this cycle, evaluated on the GPU's logits through the same map
        rc, law = gfo.draft_law_compact_mapped(bufs["q_logits"].cpu().numpy(), opt_cpu, d2t)
        assert rc == 0
        word, ua, ur, un = gfo.step_draws(seed, step)
        draft = gfo.lib().gfo_draft_select(C.byref(law), C.c_uint32(word))
        proposal = int(d2t[draft])
        p_logits = bufs["p_logits"].cpu().numpy()
        r0, r1 = gfo.select_candidates(p_logits[0], 64), gfo.select_candidates(p_logits[1], 64)
        rc, want = gfo.spec_accept_mapped(r0, none, r1, none, law, t2d, proposal, opt_cpu, ua, ur, un)
        assert rc == 0
        assert res["proposal"] == proposal
        assert (res["accepted"], res["token"], res["next_root"]) == (want.accepted, want.token, want.next_root)
        assert abs(res["acceptance_probability"] - want.acceptance_probability) <= 1e-13
        decisions.append(int(res["accepted"]))
        supports.append((int(law.count), int(gfo.prepare(r0, opt_cpu)[1].count)))
        if step == 0:
            # numerical parity of both forwards and both heads against the CPU path
            dh, _, _ = gfo.forward(d_host, [root], d_pos, threads=threads)
            assert rel_rms(bufs["drafter_hidden"].cpu().numpy()[None, :], dh) <= 1e-3
            ql = gfo.gemv(d_shape.embed_dtype, d_host.head, dh, d_shape.vocab, threads=threads)
            assert rel_rms(bufs["q_logits"].cpu().numpy()[None, :], ql) <= 1e-3
            toks = bufs["tokens"].cpu().numpy().view(np.uint32)[:2]   # the verify pair: root, proposal
            assert toks[0] == root and toks[1] == proposal
            th, wk, wv = gfo.forward(t_host, toks, t_pos, threads=threads)
            assert rel_rms(bufs["target_hidden"].cpu().numpy(), th) <= 1e-3
            pl = gfo.gemv(t_shape.embed_dtype, t_host.head, th, t_shape.vocab, threads=threads)
            assert rel_rms(bufs["p_logits"].cpu().numpy(), pl) <= 1e-3
            check_private_rows(plan.t_pk, wk)
            check_private_rows(plan.t_pv, wv)
    # both laws spread over many tokens, and the run took both branches of the acceptance test
    assert min(q for q, p in supports) > 8 and min(p for q, p in supports) > 8, supports
    assert 0 < sum(decisions) < steps, decisions
    return decisions, plan, target, drafter, t_host


def test_h1_cycle_small_models(hip, gfo):
    from dataclasses import replace
    from guffin_amd import model
    t_shape = replace(model.GEMMA3_12B, layers=3, vocab=16384, ring_global=2048)
    d_shape = replace(model.GEMMA3_270M, layers=4, vocab=16384, ring_global=2048)
    run_h1(hip, gfo, t_shape, d_shape, 1300, 1300, steps=12, seed=5)


def test_h1_cycle_with_the_full_vocabulary_law(hip, gfo):
    """A step whose sampler options rule out the compact law (top_k > 64, then greedy drafting):
    proposal and decision equal the oracle's on the step's own logits, q gathered from the table."""
    import torch
    from dataclasses import replace
    from guffin_amd import model
    t_shape = replace(model.GEMMA3_12B, layers=2, vocab=8192, ring_global=2048)
    d_shape = replace(model.GEMMA3_270M, layers=2, vocab=8192, ring_global=2048)
    target = model.DeviceModel.from_host(model.HostModel(t_shape, seed=31, position=900))
    drafter = model.DeviceModel.from_host(model.HostModel(d_shape, seed=32, position=900))
    for temperature, top_k in ((1.0, 128), (0.0, 1)):
        plan = model.H1Plan(target, drafter, 900, 900, temperature=temperature, top_k=top_k, seed=4, publish=False,
                            full_law=True)
        opt_cpu = gfo.SamplerOptions(temperature, top_k, 0.95, 0.0, 1.0)
        plan.root.fill_(55)
        for step in range(6):
            plan.step(step)
            torch.cuda.synchronize()
            bufs, res = plan.buffers(), plan.read_result()
            assert int(plan.status.item()) == 0
            rc, cdf = gfo.draft_law_full(bufs["q_logits"].cpu().numpy(), opt_cpu)
            assert rc == 0
            assert np.array_equal(bufs["full_cdf"].cpu().numpy().view(np.uint64), cdf)
            word, ua, ur, un = gfo.step_draws(4, step)
            proposal = gfo.draft_select_full(cdf, word)
            p_logits = bufs["p_logits"].cpu().numpy()
            rows = [gfo.select_candidates(p_logits[r], top_k) for r in range(2)]
            rc, want = gfo.spec_accept_full(rows[0], rows[1], cdf, proposal, opt_cpu, ua, ur, un)
            assert res["proposal"] == proposal
            if rc != 0:
                assert res["status"] == -rc
                continue
            assert res["status"] == 0
            assert (res["accepted"], res["token"], res["next_root"]) == (want.accepted, want.token, want.next_root)
    # the compact options with the fallback encoded take the same decisions as without it
    a = model.H1Plan(target, drafter, 900, 900, seed=4, publish=False, full_law=True)
    b = model.H1Plan(target, drafter, 900, 900, seed=4, publish=False)
    for plan in (a, b):
        plan.root.fill_(55)
        plan.step(3)
    torch.cuda.synchronize()
    assert a.read_result().tobytes() == b.read_result().tobytes()


def test_h1_cycle_with_sampler_history(hip, gfo):
    """The verify pass's sampler sees the generated tokens so far, and row 1 also the proposal
    (src/engine/sampling.cpp:430-446): decisions equal the oracle's with both rows' histories, for a
    short history and for a full window where the oldest token leaves row 1's history."""
    import torch
    from dataclasses import replace
    from guffin_amd import model
    t_shape = replace(model.GEMMA3_12B, layers=2, vocab=8192, ring_global=2048)
    d_shape = replace(model.GEMMA3_270M, layers=2, vocab=8192, ring_global=2048)
    t_host, d_host = model.HostModel(t_shape, seed=41, position=600), model.HostModel(d_shape, seed=42, position=600)
    # these random models' logits reach 9e4 (target) and 1e3 (drafter): bring them to a sampler's range
    t_host.out_norm *= np.float32(1e-4)
    d_host.out_norm *= np.float32(1e-2)
    target, drafter = model.DeviceModel.from_host(t_host), model.DeviceModel.from_host(d_host)
    # where the target's mass sits for this root, so that the penalty moves decisions
    probe = model.H1Plan(target, drafter, 600, 600, seed=9, publish=False)
    probe.root.fill_(77)
    probe.step(0)
    torch.cuda.synchronize()
    best = np.argsort(-probe.buffers()["p_logits"].cpu().numpy()[0])[:6].astype(np.uint32)
    rng = np.random.default_rng(5)
    differs = 0
    for count in (9, 64):
        history = np.concatenate([rng.integers(0, 8192, count - best.size).astype(np.uint32), best])
        history[1] = history[0]   # a token seen twice is listed, penalised and counted once
        plan = model.H1Plan(target, drafter, 600, 600, temperature=1.0, top_k=32, seed=9, publish=False,
                            history=history.tolist(), repetition_penalty=1.9)
        opt_cpu = gfo.SamplerOptions(1.0, 32, 0.95, 0.0, 1.9)
        plan.root.fill_(77)
        for step in range(8):
            plan.step(step)
            torch.cuda.synchronize()
            bufs, res = plan.buffers(), plan.read_result()
            assert int(plan.status.item()) == 0 and res["status"] == 0
            # the drafter penalises the same history before it builds its law (gemma3_draft.mm:186-204)
            q_scores = bufs["q_logits"].cpu().numpy().copy()
            hit = np.zeros(q_scores.size, bool)
            hit[history] = True
            r = np.float32(1.9)
            q_scores[hit] = np.where(q_scores[hit] < 0, q_scores[hit] * r, q_scores[hit] / r)
            rc, law = gfo.draft_law_compact(q_scores, opt_cpu)
            assert rc == 0
            word, ua, ur, un = gfo.step_draws(9, step)
            proposal = gfo.lib().gfo_draft_select(C.byref(law), C.c_uint32(word))
            assert res["proposal"] == proposal
            hist1 = np.concatenate([history, [proposal]]).astype(np.uint32)[-64:]
            # each row retains top_k + its own count of distinct history tokens (base_candidate_count,
            # src/engine/sampling.cpp:352-378) and then lists those tokens' logits, first occurrence first
            uniq0, uniq1 = [np.array(list(dict.fromkeys(h.tolist())), np.uint32) for h in (history, hist1)]
            p_logits = bufs["p_logits"].cpu().numpy()
            r0 = gfo.select_candidates(p_logits[0], 32 + uniq0.size, uniq0)
            r1 = gfo.select_candidates(p_logits[1], 32 + uniq1.size, uniq1)
            got = hip.candidates_to_numpy(bufs["candidates"])
            for row, want_row in enumerate((r0, r1)):
                assert got[row]["count"] == want_row.size
                assert np.array_equal(got[row]["values"]["token"][:want_row.size], want_row["token"])
                assert np.array_equal(got[row]["values"]["logit"][:want_row.size].view(np.uint32),
                                      want_row["logit"].view(np.uint32))
            rc, want = gfo.spec_accept_history(r0, history, r1, hist1, law, proposal, opt_cpu, ua, ur, un)
            assert rc == 0
            assert (res["accepted"], res["token"], res["next_root"]) == (want.accepted, want.token, want.next_root)
            assert abs(res["acceptance_probability"] - want.acceptance_probability) <= 1e-13
            rc, plain = gfo.spec_accept(gfo.select_candidates(p_logits[0], 32), gfo.select_candidates(p_logits[1], 32),
                                        law, proposal, opt_cpu, ua, ur, un)
            differs += int(rc != 0 or plain.acceptance_probability != want.acceptance_probability
                           or plain.token != want.token)
    assert differs > 0   # the history is not a no-op on these steps


def test_h1_commit_publishes_verified_rows(hip, gfo):
    import torch
    from dataclasses import replace
    from guffin_amd import model
    t_shape = replace(model.GEMMA3_12B, layers=6, vocab=4096, ring_global=2048)
    d_shape = replace(model.GEMMA3_270M, layers=6, vocab=4096, ring_global=2048)
    t_pos = 1030
    target = model.DeviceModel.from_host(model.HostModel(t_shape, seed=21, position=t_pos))
    drafter = model.DeviceModel.from_host(model.HostModel(d_shape, seed=22, position=t_pos))
    before = [(k.clone(), v.clone()) for k, v in zip(target.ring_k, target.ring_v)]
    plan = model.H1Plan(target, drafter, t_pos, t_pos, seed=9, publish=True)
    plan.root.fill_(77)
    plan.step(0)
    torch.cuda.synchronize()
    res = plan.read_result()
    publish = 1 + int(res["accepted"])
    for l in range(t_shape.layers):
        cap = t_shape.ring_local if t_shape.is_local(l) else t_shape.ring_global
        for row in range(2):
            slot = (t_pos + row) & (cap - 1)
            if row < publish:
                assert torch.equal(target.ring_k[l][slot], plan.t_pk[l, row])
                assert torch.equal(target.ring_v[l][slot], plan.t_pv[l, row])
            else:
                assert torch.equal(target.ring_k[l][slot], before[l][0][slot])
        untouched = [s for s in range(cap) if s not in ((t_pos) & (cap - 1), (t_pos + 1) & (cap - 1))][:50]
        assert torch.equal(target.ring_k[l][untouched], before[l][0][untouched])
    cap = d_shape.ring_local
    assert torch.equal(drafter.ring_k[0][t_pos & (cap - 1)], plan.d_pk[0, 0])


def test_h1_cycle_full_size_models(hip, gfo):
    """Config 4 shapes: the 48-block 12B target at an 8192-token context with the 18-block drafter."""
    from guffin_amd import model
    decisions, plan, *_ = run_h1(hip, gfo, model.GEMMA3_12B, model.GEMMA3_270M, 8190, 4096, steps=10, seed=1, threads=16)
    print("full-size decisions:", decisions)


def test_h1_cycle_with_a_vocabulary_map(hip, gfo):
    """The drafter's vocabulary is a shuffled, partly unmapped view of the target's (the reference's TLI map,
    src/engine/gemma3_draft.mm:648-675): the root reaches the drafter in its own id, the law lives in draft ids
    without unmapped tokens, the proposal enters the verify pass in the target's id, and the decision equals the
    oracle's with the same maps on the step's own logits."""
    import torch
    from dataclasses import replace
    from guffin_amd import model
    vocab = 8192
    t_shape = replace(model.GEMMA3_12B, layers=2, vocab=vocab, ring_global=2048)
    d_shape = replace(model.GEMMA3_270M, layers=2, vocab=vocab, ring_global=2048)
    t_host, d_host = model.HostModel(t_shape, seed=51, position=300), model.HostModel(d_shape, seed=52, position=300)
    t_host.out_norm *= np.float32(1e-4)   # bring these random models' logits to a sampler's range
    d_host.out_norm *= np.float32(1e-2)
    target, drafter = model.DeviceModel.from_host(t_host), model.DeviceModel.from_host(d_host)
    rng = np.random.default_rng(8)
    d2t = rng.permutation(vocab).astype(np.int32)
    root = 77
    unmapped = rng.choice(vocab, 500, replace=False)
    unmapped = unmapped[d2t[unmapped] != root]        # the root stays known to the drafter
    d2t[unmapped] = -1
    t2d = np.full(vocab, -1, np.int32)
    t2d[d2t[d2t >= 0]] = np.nonzero(d2t >= 0)[0].astype(np.int32)
    history = np.array([5, 6, root], np.uint32)
    plan = model.H1Plan(target, drafter, 300, 300, temperature=1.0, top_k=32, seed=3, publish=False,
                        history=history.tolist(), repetition_penalty=1.5, draft_to_target=d2t, target_to_draft=t2d)
    opt_cpu = gfo.SamplerOptions(1.0, 32, 0.95, 0.0, 1.5)
    plan.root.fill_(root)
    for step in range(6):
        plan.step(step)
        torch.cuda.synchronize()
        bufs, res = plan.buffers(), plan.read_result()
        assert int(plan.status.item()) == 0 and res["status"] == 0
        toks = bufs["tokens"].cpu().numpy().view(np.uint32)
        assert toks[8] == t2d[root]                                        # the drafter's input row, in its ids
        if step == 0:   # the drafter really ran on that id
            dh, _, _ = gfo.forward(d_host, [int(t2d[root])], 300, threads=8)
            assert rel_rms(bufs["drafter_hidden"].cpu().numpy()[None, :], dh) <= 1e-3
        scores = bufs["q_logits"].cpu().numpy().copy()
        hist_draft = t2d[history]
        r = np.float32(1.5)
        for dtok in hist_draft[hist_draft >= 0]:
            scores[dtok] = scores[dtok] * r if scores[dtok] < 0 else scores[dtok] / r
        rc, law = gfo.draft_law_compact_mapped(scores, opt_cpu, d2t)
        assert rc == 0
        word, ua, ur, un = gfo.step_draws(3, step)
        draft = gfo.lib().gfo_draft_select(C.byref(law), C.c_uint32(word))
        assert toks[2] == draft and toks[1] == d2t[draft] and res["proposal"] == d2t[draft]
        hist1 = np.concatenate([history, [d2t[draft]]]).astype(np.uint32)
        retain = 32 + history.size + 1
        p_logits = bufs["p_logits"].cpu().numpy()
        r0 = gfo.select_candidates(p_logits[0], retain, history)
        r1 = gfo.select_candidates(p_logits[1], retain, hist1)
        rc, want = gfo.spec_accept_mapped(r0, history, r1, hist1, law, t2d, int(d2t[draft]), opt_cpu, ua, ur, un)
        assert rc == 0
        assert (res["accepted"], res["token"], res["next_root"]) == (want.accepted, want.token, want.next_root)
    # the same map with a law that needs the full table (top_k beyond the compact law's 64)
    wide = model.H1Plan(target, drafter, 300, 300, temperature=1.0, top_k=100, seed=4, publish=False, full_law=True,
                        draft_to_target=d2t, target_to_draft=t2d)
    wide_cpu = gfo.SamplerOptions(1.0, 100, 0.95, 0.0, 1.0)
    wide.root.fill_(root)
    for step in range(4):
        wide.step(step)
        torch.cuda.synchronize()
        bufs, res = wide.buffers(), wide.read_result()
        assert int(wide.status.item()) == 0 and res["status"] == 0
        rc, cdf = gfo.draft_law_full_mapped(bufs["q_logits"].cpu().numpy(), wide_cpu, d2t)
        assert rc == 0 and np.array_equal(bufs["full_cdf"].cpu().numpy().view(np.uint64), cdf)
        word, ua, ur, un = gfo.step_draws(4, step)
        draft = gfo.draft_select_full(cdf, word)
        toks = bufs["tokens"].cpu().numpy().view(np.uint32)
        assert toks[2] == draft and toks[1] == d2t[draft] and res["proposal"] == d2t[draft]
        p_logits = bufs["p_logits"].cpu().numpy()
        rc, want = gfo.spec_accept_full_mapped(gfo.select_candidates(p_logits[0], 100), gfo.select_candidates(p_logits[1], 100),
                                               cdf, t2d, int(d2t[draft]), wide_cpu, ua, ur, un)
        assert rc == 0
        assert (res["accepted"], res["token"], res["next_root"]) == (want.accepted, want.token, want.next_root)
    # a root the drafter does not have raises the bad-token bit instead of reading outside its table
    orphan = int(np.nonzero(t2d < 0)[0][0])
    plan.root.fill_(orphan)
    plan.step(9)
    torch.cuda.synchronize()
    assert int(plan.status.item()) & 1
