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


@pytest.mark.parametrize("accepted", [0, 1])
def test_commit_and_finalize_leave_the_rings_as_commit_rows_does(hip, target, accepted):
    """The H1 step publishes after the decision (commit_rows with the accept word); a host that keeps the
    reference's protocol publishes both rows and finalizes 1 + accepted of them.  Both must leave every ring,
    local (1024 slots, wrapping here) and global (2048 slots), with the same bytes."""
    import ctypes as C
    import torch
    from guffin_amd import model
    ticket = model.VerifyTicket(target, POSITION + 4)
    before = rings(target)
    pk, pv = run_pass(hip, target, ticket, [17, 1999], POSITION)
    # commit_rows on copies of the rings
    copies = rings_copy(before)
    k_table = torch.tensor([k.data_ptr() for k, _ in copies], dtype=torch.int64, device="cuda")
    v_table = torch.tensor([v.data_ptr() for _, v in copies], dtype=torch.int64, device="cuda")
    word = torch.tensor([accepted], dtype=torch.int32, device="cuda")
    hip.check(hip.lib().guffin_hip_commit_rows(
        hip._stream(), C.byref(target.desc), C.c_void_p(pk.data_ptr()),
        C.c_void_p(pv.data_ptr()), C.c_void_p(k_table.data_ptr()), C.c_void_p(v_table.data_ptr()),
        C.c_void_p(word.data_ptr()), C.c_uint32(POSITION), C.c_uint32(2)))
    torch.cuda.synchronize()
    ticket.provisional_commit([0, 1])
    ticket.finalize(1 + accepted)
    assert ticket.state == model.TXN_IDLE
    assert_rings(target, copies)
    changed = sum(int((k != b[0]).any(dim=-1).sum()) for (k, _), b in zip(copies, before))
    assert changed == (1 + accepted) * target.shape.layers   # one slot per published row and layer (random rows differ)


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


def oracle_candidates(gfo, host, tokens, position, row, retain=64):
    """Top `retain` candidates of chain row `row` from the oracle's forward pass and head."""
    hidden, pk, pv = gfo.forward(host, np.array(tokens, np.uint32), position, threads=8)
    logits = gfo.gemv(host.shape.embed_dtype, host.head, hidden[row:row + 1], host.shape.vocab, threads=8)[0]
    return gfo.select_candidates(logits, retain), pk[:, row], pv[:, row]


def same_tokens_close_logits(got, want, scale, rel=1e-3):
    """The device and the oracle sum in different orders: candidates agree as sets of tokens down to the
    point where two logits are closer than the sides differ, and in value within 1e-3 of the logit scale."""
    n = want.size
    g = {int(t): float(l) for t, l in zip(got["values"]["token"][:n], got["values"]["logit"][:n])}
    w = {int(t): float(l) for t, l in zip(want["token"], want["logit"])}
    tol = rel * scale
    for token, logit in w.items():
        if token in g:
            assert abs(g[token] - logit) <= tol
        else:
            assert logit <= float(want["logit"][-1]) + 2 * tol, "a clear member of the oracle's top is missing"
    assert len(set(g) & set(w)) >= n - 2


def test_three_row_tree_against_the_oracle_and_every_path(hip, gfo):
    """Rows [root, A, B] with A and B both children of the root (two proposals for the same position):
    row 1 equals row 1 of the chain [root, A] and row 2 equals row 1 of the chain [root, B], in the oracle's
    arithmetic and on the device's own chain pass; a provisional commit publishes any root-to-node path."""
    import torch
    from guffin_amd import model
    shape = replace(model.GEMMA3_12B, layers=6, vocab=2048, ring_global=2048)
    host = model.HostModel(shape, seed=5, position=POSITION, untied_head=True)
    target = model.DeviceModel.from_host(host)
    ticket = model.VerifyTicket(target, POSITION + 4)
    root, a, b = 17, 1999, 42
    before = rings(target)
    ticket.encode_tree([root, a, b], [None, 0, 0], POSITION)
    ticket.submit()
    assert ticket.complete() == 0 and ticket.state == model.TXN_COMPLETED
    assert_rings(target, before)
    got = ticket.read_candidates()
    kvw = shape.kv_width
    priv_k = ticket.priv_k.view(-1)[:shape.layers * 3 * kvw].view(shape.layers, 3, kvw)
    priv_v = ticket.priv_v.view(-1)[:shape.layers * 3 * kvw].view(shape.layers, 3, kvw)
    # (1) the oracle, chain by chain
    for row, (chain, chain_row) in enumerate([((root, a), 0), ((root, a), 1), ((root, b), 1)]):
        want, wk, wv = oracle_candidates(gfo, host, chain, POSITION, chain_row)
        assert int(got[row]["count"]) == 64 and int(got[row]["status"]) == 0
        same_tokens_close_logits(got[row], want, float(np.abs(want["logit"]).max()))
        k = priv_k[:, row].view(torch.int16).cpu().numpy().view(np.uint16)
        v = priv_v[:, row].view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.mean(k == wk) >= 0.95 and np.mean(v == wv) >= 0.95
    # (2) the device's own two-row chain passes (fused attention) give the same rows up to summation order
    for row, chain in ((1, (root, a)), (2, (root, b))):
        hidden, sums, pk, pv, status = target.forward(torch.tensor(chain, dtype=torch.int32, device="cuda"), POSITION)
        logits = hip.gemv_packed(int(shape.embed_dtype), target.head_tiles, hidden, sums, shape.vocab)
        want = hip.candidates_to_numpy(hip.select_candidates(logits, 64)[0])[1]
        assert np.array_equal(got[row]["values"]["token"][:8], want["values"]["token"][:8])
        assert np.allclose(got[row]["values"]["logit"][:64], want["values"]["logit"][:64], rtol=0, atol=1e-3 * float(np.abs(want["values"]["logit"][:64]).max()))
        assert np.mean((priv_k[:, row] == pk[:, 1]).cpu().numpy()) >= 0.97
    # (3) paths: [0, 2] publishes the root and B; keeping one row restores B's slot; [0, 1, 2] is no path
    with pytest.raises(hip.GuffinError):
        ticket.provisional_commit([0, 1, 2])
    ticket.provisional_commit([0, 2])
    want = rings_copy(before)
    publish(want, target, priv_k, priv_v, POSITION, [0, 2])
    assert_rings(target, want)
    ticket.finalize(1)
    kept = rings_copy(before)
    publish(kept, target, priv_k, priv_v, POSITION, [0])
    assert_rings(target, kept)
    # a four-row tree with a grandchild: [root, A, A's child, B]
    ticket.encode_tree([a, b, 7, root], [None, 0, 1, 0], POSITION + 1)
    ticket.submit()
    assert ticket.complete() == 0
    got = ticket.read_candidates()
    host.commit(np.stack([priv_k[:, 0].view(torch.int16).cpu().numpy().view(np.uint16)] * 1, axis=1),
                np.stack([priv_v[:, 0].view(torch.int16).cpu().numpy().view(np.uint16)] * 1, axis=1), POSITION, 1)
    # the ring row below this tree is the device's own (published above), so the sides start a little apart
    for row, (chain, chain_row) in ((1, ((a, b), 1)), (3, ((a, root), 1))):
        want, _, _ = oracle_candidates(gfo, host, chain, POSITION + 1, chain_row)
        same_tokens_close_logits(got[row], want, float(np.abs(want["logit"]).max()), rel=2e-3)
    ticket.provisional_commit([0, 1, 2])
    ticket.discard()
    assert_rings(target, kept)
