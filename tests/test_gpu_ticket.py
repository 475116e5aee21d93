"""The verify pass as a transaction on the device (guffin_hip_ticket_*).

What the pass computes is the block graph, head and selection that tests/test_gpu_forward.py and
tests/test_gpu_sampling.py hold against the oracle; here the ticket's results must be those same
bytes, and the ring rows must go through the reference's protocol exactly
(src/engine/target_verifier_runtime.cpp:535-673): a provisional commit publishes the selected
private rows and keeps what they overwrote, finalize keeps a prefix and restores the rest, and no
other ring row ever changes.  Local rings wrap in these cases (position 1023 of 1024 slots).
"""
from dataclasses import replace

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

POSITION = 1023


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


@pytest.fixture()
def target(hip):
    from guffin_amd import model
    shape = replace(model.GEMMA3_12B, layers=6, vocab=2048, ring_global=2048)
    host = model.HostModel(shape, seed=3, position=POSITION)
    return model.DeviceModel.from_host(host)


def rings(target):
    return [(k.clone(), v.clone()) for k, v in zip(target.ring_k, target.ring_v)]


def assert_rings(target, want):
    import torch
    for l, (k, v) in enumerate(want):
        assert torch.equal(target.ring_k[l], k), "layer %d keys" % l
        assert torch.equal(target.ring_v[l], v), "layer %d values" % l


def run_pass(hip, target, ticket, tokens, position):
    import torch
    from guffin_amd import model
    ticket.encode(tokens, position)
    assert ticket.state == model.TXN_ENCODED
    ticket.submit()
    assert ticket.state == model.TXN_SUBMITTED
    assert ticket.complete() == 0
    assert ticket.state == model.TXN_COMPLETED
    # the same pass through the plain entry points
    tok = torch.tensor(tokens, dtype=torch.int32, device="cuda")
    hidden, sums, pk, pv, status = target.forward(tok, position)
    logits = hip.gemv_packed(int(target.shape.embed_dtype), target.head_tiles, hidden, sums, target.shape.vocab)
    cands, _ = hip.select_candidates(logits, 64)
    want = hip.candidates_to_numpy(cands)
    got = ticket.read_candidates()
    rows = len(tokens)
    for r in range(rows):
        n = int(want[r]["count"])
        assert n == 64 and int(got[r]["count"]) == n and int(got[r]["status"]) == 0
        assert np.array_equal(got[r]["values"][:n], want[r]["values"][:n])
    kvw = target.shape.kv_width
    assert torch.equal(ticket.priv_k.view(-1)[:pk.numel()].view(-1, rows, kvw), pk)
    assert torch.equal(ticket.priv_v.view(-1)[:pv.numel()].view(-1, rows, kvw), pv)
    return pk, pv


def publish(want, target, pk, pv, position, path):
    for l in range(target.shape.layers):
        cap = want[l][0].shape[0]
        for i, node in enumerate(path):
            want[l][0][(position + i) & (cap - 1)] = pk[l, node]
            want[l][1][(position + i) & (cap - 1)] = pv[l, node]


def test_provisional_commit_then_keep_one_row(hip, target):
    from guffin_amd import model
    ticket = model.VerifyTicket(target, POSITION + 4)
    before = rings(target)
    pk, pv = run_pass(hip, target, ticket, [17, 1999], POSITION)
    assert_rings(target, before)                       # a completed pass has not touched the caches
    ticket.provisional_commit([0, 1])
    assert ticket.state == model.TXN_PROVISIONAL and ticket.desc.provisional_count == 2
    both = rings_copy(before)
    publish(both, target, pk, pv, POSITION, [0, 1])
    assert_rings(target, both)                         # local rings: slot 1023, then slot 0
    ticket.finalize(1)
    assert ticket.state == model.TXN_IDLE
    one = rings_copy(before)
    publish(one, target, pk, pv, POSITION, [0])
    assert_rings(target, one)                          # the rejected row's slot holds its old bytes again
    # the next pass starts behind the kept row and can be dropped whole
    pk2, pv2 = run_pass(hip, target, ticket, [5, 6], POSITION + 1)
    ticket.provisional_commit([0])
    kept = rings_copy(one)
    publish(kept, target, pk2, pv2, POSITION + 1, [0])
    assert_rings(target, kept)
    ticket.discard()
    assert ticket.state == model.TXN_IDLE
    assert_rings(target, one)


def rings_copy(src):
    return [(k.clone(), v.clone()) for k, v in src]


def test_single_row_pass_and_release(hip, target):
    from guffin_amd import model
    ticket = model.VerifyTicket(target, POSITION + 4)
    before = rings(target)
    pk, pv = run_pass(hip, target, ticket, [42], POSITION)
    with pytest.raises(hip.GuffinError) as err:
        ticket.provisional_commit([0, 1])               # row 1 was not in this pass
    assert err.value.code == -1 and ticket.state == model.TXN_COMPLETED
    ticket.provisional_commit([0])
    ticket.release()                                    # what the reference's destructor does: roll back
    assert ticket.state == model.TXN_IDLE
    assert_rings(target, before)
    with pytest.raises(hip.GuffinError) as err:
        ticket.submit()                                 # nothing encoded
    assert err.value.code == -6


def test_a_raised_status_word_drops_the_transaction(hip, target):
    from guffin_amd import model
    ticket = model.VerifyTicket(target, POSITION + 4)
    before = rings(target)
    ticket.encode([17, target.shape.vocab + 5], POSITION)   # a token outside the vocabulary
    ticket.submit()
    with pytest.raises(hip.GuffinError) as err:
        ticket.complete()
    assert err.value.code == -7
    assert ticket.state == model.TXN_IDLE                   # private rows only: the caches are as before
    assert_rings(target, before)
    pk, pv = run_pass(hip, target, ticket, [17, 1999], POSITION)   # and the ticket is usable again
    ticket.discard()
    assert ticket.state == model.TXN_IDLE
