"""Consecutive H1 cycles through the session lifecycle (positions, pending drafter token, poisoning)
against the CPU oracle run teacher-forced on the same tokens with its own mirrored caches.
Reference behaviour: src/engine/gemma3_draft.mm:1430-1486 (pending token),
include/local_gguf_engine/engine/gemma2_metal_plan.hpp:208-215 (transaction states)."""
import ctypes as C
from dataclasses import replace

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def rel_rms(got, want):
    want = want.astype(np.float64)
    scale = np.sqrt((want ** 2).mean(axis=-1, keepdims=True)) + 1e-30
    return float(np.max(np.abs(got.astype(np.float64) - want) / scale))


def small_models(vocab, t_pos, d_pos):
    from guffin_amd import model
    t_shape = replace(model.GEMMA3_12B, layers=3, vocab=vocab, ring_global=2048)
    d_shape = replace(model.GEMMA3_270M, layers=3, vocab=vocab, ring_global=2048)
    t_host = model.HostModel(t_shape, seed=41, position=t_pos)
    d_host = model.HostModel(d_shape, seed=42, position=d_pos)
    return t_host, d_host, model.DeviceModel.from_host(t_host), model.DeviceModel.from_host(d_host)


def test_session_generates_over_many_cycles(hip, gfo):
    import torch
    from guffin_amd import model
    t_pos, d_pos, cycles, seed = 1000, 1000, 24, 7
    t_host, d_host, target, drafter = small_models(256, t_pos, d_pos)
    # random weights with a tied head make both laws peak on the root token; a high temperature
    # flattens them enough for acceptances and rejections to alternate
    sess = model.Session(target, drafter, 123, t_pos, d_pos, cycles, temperature=256.0, top_p=1.0, seed=seed)
    opt = gfo.SamplerOptions(256.0, 64, 1.0, 0.0, 1.0)
    root, pending, confirmed = 123, None, []
    accepts = rejects = 0
    for cycle in range(cycles):
        sess.submit()
        with pytest.raises(hip.GuffinError):
            sess.submit()                      # one cycle in flight at a time
        emitted = sess.complete()
        bufs, res = sess.buffers(), sess.read_result()
        # the oracle's decision on the cycle's own logits
        rc, law = gfo.draft_law_compact(bufs["q_logits"].cpu().numpy(), opt)
        assert rc == 0
        word, ua, ur, un = gfo.step_draws(seed, cycle)
        proposal = gfo.lib().gfo_draft_select(C.byref(law), C.c_uint32(word))
        p_logits = bufs["p_logits"].cpu().numpy()
        rows = [gfo.select_candidates(p_logits[r], 64) for r in range(2)]
        rc, want = gfo.spec_accept(rows[0], rows[1], law, proposal, opt, ua, ur, un)
        assert rc == 0 and res["status"] == 0 and res["proposal"] == proposal
        assert (res["accepted"], res["token"], res["next_root"]) == (want.accepted, want.token, want.next_root)
        assert emitted == ([proposal, want.next_root] if want.accepted else [want.token])
        # both passes against the oracle, teacher-forced, on the oracle's own mirrored caches
        d_tokens = [pending, root] if pending is not None else [root]
        dh, dk, dv = gfo.forward(d_host, d_tokens, d_pos)
        assert rel_rms(bufs["drafter_hidden_rows"].cpu().numpy(), dh) <= 1e-3, cycle
        th, tk, tv = gfo.forward(t_host, [root, proposal], t_pos)
        assert rel_rms(bufs["target_hidden"].cpu().numpy(), th) <= 1e-3, cycle
        d_host.commit(dk, dv, d_pos, len(d_tokens))
        t_host.commit(tk, tv, t_pos, 1 + want.accepted)
        d_pos += len(d_tokens)
        t_pos += 1 + want.accepted
        pending = proposal if want.accepted else None
        root = want.next_root
        confirmed += emitted
        accepts += want.accepted
        rejects += 1 - want.accepted
        assert (sess.s.desc.target_position, sess.s.desc.drafter_position) == (t_pos, d_pos)
        assert (sess.s.root, bool(sess.s.has_pending)) == (root, pending is not None)
    assert accepts >= 3 and rejects >= 3, (accepts, rejects)   # both branches of the pending token ran
    assert len(confirmed) == cycles + accepts and sess.s.cycles == cycles and sess.s.accepted == accepts
    # what the device published equals the oracle's caches (fp16 rows, rare rounding ties aside)
    for l in (0, t_host.shape.layers - 1):
        cap = t_host.shape.ring_local if t_host.shape.is_local(l) else t_host.shape.ring_global
        slots = np.arange(1000, t_pos) & (cap - 1)
        got = target.ring_k[l].cpu().numpy()[slots].astype(np.float32)
        want_k = t_host.ring_k[l][slots].astype(np.float32)
        assert np.max(np.abs(got - want_k)) <= 2.0 ** -8 * np.abs(want_k).max() + 1e-6


def test_session_poisons_on_a_device_fault_and_refuses_further_cycles(hip, gfo):
    import torch
    from guffin_amd import model
    t_host, d_host, target, drafter = small_models(256, 600, 600)
    sess = model.Session(target, drafter, 5, 600, 600, 4, top_p=1.0, seed=3)
    sess.submit()
    assert sess.complete()
    # a root outside the vocabulary raises the device status word: the cycle is refused for good
    sess.s.root = 100000
    sess.submit()
    with pytest.raises(hip.GuffinError):
        sess.complete()
    assert sess.s.state == 5
    with pytest.raises(hip.GuffinError):
        sess.submit()


def test_session_requires_ring_tables_and_order(hip):
    from guffin_amd import model
    t_host, d_host, target, drafter = small_models(256, 100, 100)
    sess = model.Session(target, drafter, 5, 100, 100, 2, top_p=1.0)
    with pytest.raises(hip.GuffinError):
        sess.complete()                        # nothing in flight
    sess.s.desc.target_ring_k = None
    with pytest.raises(hip.GuffinError):
        hip.check(hip.lib().guffin_hip_session_start(C.byref(sess.s), 5, 100, 100))
