"""The drafter's lifecycle (guffin_hip_draft_plan_*) on the cases of the reference's transaction_lifecycle
test (tests/engine/gemma3_draft_tests.cpp:206-277): aborted and truncated suffixes leave the caches as they
were, a committed prefix followed by a different next root gives the logits and caches of a plain replay,
bit for bit, and that replay agrees with the oracle run token by token over mirrored host caches."""
from dataclasses import replace

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT, NEXT_ROOT, CORRECTION = 55, 719, 111


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def stream(n):
    return [int((i * 37 + 11) % 4000) for i in range(n)]


def reference_stream(n):
    """tests/engine/gemma3_draft_tests.cpp:188-190"""
    return [3 + (i * 499) % 255997 if i else 2 for i in range(n)]


class World:
    """A drafter to run the lifecycle on: `scaled` is a three-block model with 64-row local rings (prompt 62, the
    oracle replays it); `reference` is the reference's own case, its closed-form fixture at the full 270M geometry
    with a 510-token prompt against 512-row rings (tests/drafter_fixture.py holds that model to its closed form)."""

    def __init__(self, kind):
        from guffin_amd import model
        self.kind = kind
        if kind == "scaled":
            self.shape = replace(model.GEMMA3_270M, layers=3, global_period=3, vocab=4096, sliding_window=64, ring_local=64,
                                 ring_global=256)
            self.host = model.HostModel(self.shape, seed=31, position=0, untied_head=True)
            self.prompt, self.stream = 62, stream
        else:
            import drafter_fixture as fx
            self.host = fx.host_model(model, ring_global=1024)
            self.shape = self.host.shape
            self.prompt, self.stream = 510, reference_stream
        self.device = model.DeviceModel.from_host(self.host)

    def __iter__(self):     # (shape, host, device), as the tests unpack it
        return iter((self.shape, self.host, self.device))


_worlds = {}


def world_of(kind):
    if kind not in _worlds:
        _worlds[kind] = World(kind)
    return _worlds[kind]


@pytest.fixture(scope="module", params=["scaled", "reference"])
def world(hip, request):
    return world_of(request.param)


@pytest.fixture(scope="module")
def scaled_world(hip):
    """The sampled-proposal test needs logits that spread: the closed-form fixture's take 53 values, so that every
    cut-off ties thousands of tokens."""
    return world_of("scaled")


def greedy(hip):
    return hip.SamplerOptions(0.0, 40, 0.95, 0.05, 1.0)


def snapshot(plan, shape):
    """Every materialized row each layer still holds, in position order."""
    rows = []
    for layer in range(shape.layers):
        cap = shape.ring_local if shape.is_local(layer) else shape.ring_global
        first = max(0, plan.materialized_position - cap)
        rows.append((first,) + plan.read_cache(layer, first, plan.materialized_position - first))
    return rows


def same_caches(a, b):
    return all(fa == fb and np.array_equal(ka, kb) and np.array_equal(va, vb) for (fa, ka, va), (fb, kb, vb) in zip(a, b))


def refuses(hip, call, code):
    with pytest.raises(hip.GuffinError) as info:
        call()
    assert info.value.code == code, info.value


def oracle_replay(gfo, host, tokens):
    """The oracle over host caches it fills itself, one token at a time: (logits after the last token, caches)."""
    import copy
    mirror = copy.copy(host)
    mirror.ring_k = [np.zeros_like(r) for r in host.ring_k]
    mirror.ring_v = [np.zeros_like(r) for r in host.ring_v]
    hidden = None
    for position, token in enumerate(tokens):
        hidden, pk, pv = gfo.forward(mirror, np.array([token], np.uint32), position, threads=8)
        mirror.commit(pk, pv, position, 1)
    logits = gfo.gemv(host.shape.embed_dtype, host.head, hidden, host.shape.vocab, threads=8)[0]
    return logits, mirror


def test_transactions_leave_no_trace_and_commits_replay(hip, gfo, world):
    from guffin_amd import model
    shape, host, device = world
    PROMPT = world.prompt
    plan = model.DraftPlan(device)
    prompt = world.stream(PROMPT)
    plan.append(prompt)
    before = snapshot(plan, shape)
    words = [0] * 23

    plan.begin_transaction()
    plan.append([ROOT])
    plan.propose(words[:3], greedy(hip))
    plan.abort_transaction()
    assert plan.position == PROMPT and same_caches(snapshot(plan, shape), before), "abort moved the prefix"

    for accepted in range(4):
        plan.begin_transaction()
        plan.append([ROOT])
        proposed = plan.propose(words[:3], greedy(hip))
        assert plan.position == PROMPT + 4 and plan.materialized_position == PROMPT + 3, "the last draft is pending, not run"
        plan.commit_prefix(PROMPT + 1 + accepted)
        if accepted == 3:
            pending_cache, old = snapshot(plan, shape), plan.materialized_position
            plan.begin_transaction()
            plan.append([NEXT_ROOT])
            plan.propose(words[:1], greedy(hip))
            plan.abort_transaction()
            assert plan.position == PROMPT + 4 and plan.materialized_position == old
            assert same_caches(snapshot(plan, shape), pending_cache), "abort lost the committed pending token"
        plan.append([NEXT_ROOT])
        actual, committed = plan.read_logits(), snapshot(plan, shape)
        replay = prompt + [ROOT] + proposed[:accepted] + [NEXT_ROOT]
        plan.reset()
        plan.append(replay)
        expected = plan.read_logits()
        assert np.array_equal(actual.view(np.uint32), expected.view(np.uint32)), "commit + next root differs from a replay"
        assert same_caches(snapshot(plan, shape), committed)
        if accepted in (0, 3) and world.kind == "scaled":     # the replay itself against the oracle over its own mirrored caches
            want, mirror = oracle_replay(gfo, host, replay)
            assert np.sqrt(np.mean((expected - want) ** 2)) <= 1e-3 * np.sqrt(np.mean(want ** 2))
            assert int(np.argmax(expected)) == int(np.argmax(want))
            for layer, (first, k, v) in enumerate(snapshot(plan, shape)):
                cap = mirror.ring_k[layer].shape[0]
                slots = (np.arange(first, len(replay)) & (cap - 1))
                assert np.mean(k == mirror.ring_k[layer][slots].view(np.uint16)) >= 0.95
                assert np.mean(v == mirror.ring_v[layer][slots].view(np.uint16)) >= 0.95
        plan.reset()
        plan.append(prompt)

    # truncate an encoded speculative suffix before appending a correction
    plan.begin_transaction()
    plan.append([ROOT])
    drafted = plan.propose(words[:3], greedy(hip))
    plan.truncate(PROMPT + 2)
    plan.append([CORRECTION])
    plan.commit_prefix(PROMPT + 3)
    assert not plan.can_truncate(PROMPT + 2)
    refuses(hip, lambda: plan.truncate(PROMPT + 2), -6)
    logits, corrected = plan.read_logits(), snapshot(plan, shape)
    plan.reset()
    plan.append(prompt + [ROOT, drafted[0], CORRECTION])
    assert np.array_equal(logits.view(np.uint32), plan.read_logits().view(np.uint32)), "truncate + correction differs from a replay"
    assert same_caches(snapshot(plan, shape), corrected)


def test_horizons_capacity_and_pending_restoration(hip, world):
    from guffin_amd import model
    shape, host, device = world
    plan = model.DraftPlan(device)
    plan.append([ROOT])
    for horizon in (1, 2, 3, 5, 23):
        plan.begin_transaction()
        drafted = plan.propose([7] * horizon, greedy(hip))
        assert len(drafted) == horizon and plan.position == horizon + 1, "a requested horizon was narrowed"
        plan.abort_transaction()
        assert plan.position == 1
    plan.begin_transaction()
    refuses(hip, plan.begin_transaction, -6)                          # nested transaction
    refuses(hip, lambda: plan.append(stream(33)), -4)                 # more rows than a transaction can take back
    assert plan.position == 1, "a refused append changed the state"
    plan.abort_transaction()
    refuses(hip, lambda: plan.append(stream(shape.ring_global)), -4)  # context overflow
    refuses(hip, lambda: plan.append([shape.vocab]), -1)              # token outside the vocabulary
    refuses(hip, lambda: plan.propose([0], greedy(hip)), -6)          # proposals live inside a transaction
    assert plan.position == 1 and not plan.poisoned

    plan.reset()
    plan.append([ROOT])
    plan.restore_pending_token(CORRECTION)
    assert plan.position == 2 and plan.materialized_position == 1, "a restored pending token was run eagerly"
    refuses(hip, lambda: plan.restore_pending_token(CORRECTION), -6)
    plan.begin_transaction()
    refuses(hip, lambda: plan.restore_pending_token(ROOT), -6)
    plan.append([NEXT_ROOT])
    plan.abort_transaction()
    assert plan.position == 2 and plan.materialized_position == 1, "abort changed the pending frontier"
    plan.append([NEXT_ROOT])
    logits = plan.read_logits()
    plan.reset()
    plan.append([ROOT, CORRECTION, NEXT_ROOT])
    assert np.array_equal(logits.view(np.uint32), plan.read_logits().view(np.uint32)), "a restored pending token changed later logits"


def test_sampled_proposals_follow_the_law_of_each_step(hip, gfo, scaled_world):
    """With temperature and a repetition penalty, draft i is the oracle's selection from the law of the
    logits the plan holds after draft i-1, with the history grown by the drafts so far."""
    import ctypes as C
    from guffin_amd import model
    shape, host, device = scaled_world
    plan = model.DraftPlan(device)
    plan.append(stream(10))
    history = [3, 4, 3]
    rng = np.random.default_rng(4)
    words = [int(w) for w in rng.integers(0, 2 ** 32, 4)]
    options = hip.SamplerOptions(0.9, 40, 0.95, 0.02, 1.3)
    plan.begin_transaction()
    drafted = plan.propose(words, options, history)
    plan.abort_transaction()
    # replay the chain token by token through append / read_logits and build each law on the CPU
    window = list(history)
    for i, word in enumerate(words):
        plan.begin_transaction()
        if i:
            plan.append(drafted[:i])
        logits = plan.read_logits()
        plan.abort_transaction()
        scores = logits.copy()
        hit = np.zeros(scores.size, bool)
        hit[window] = True
        scores[hit] = np.where(scores[hit] < 0, scores[hit] * np.float32(1.3), scores[hit] / np.float32(1.3))
        rc, law = gfo.draft_law_compact(scores, gfo.SamplerOptions(0.9, 40, 0.95, 0.02, 1.0))
        assert rc == 0
        assert drafted[i] == gfo.lib().gfo_draft_select(C.byref(law), C.c_uint32(word))
        window = (window + [drafted[i]])[-64:]


def test_a_pass_that_gives_up_a_wait_is_run_again_per_operator(hip, scaled_world):
    """The resident pass bounds every wait; when one gives up (forced here from the host: a spin limit of 0), the
    drafter plan takes GUFFIN_STATUS_SYNC down, switches the resident form off for the process and runs the pass
    again with one launch per operator: same logits and caches as a plan that ran per operator from the start."""
    from guffin_amd import model
    shape, host, device = scaled_world
    tokens = stream(9)
    hip.set_forward_mode(1)
    plain = model.DraftPlan(device)
    plain.append(tokens)
    want_logits, want_caches = plain.read_logits().copy(), snapshot(plain, shape)
    hip.set_forward_mode(0)
    assert hip.lib().guffin_hip_resident_enabled() == 1
    hip.set_spin_limit(0)
    try:
        print("draft plan with a spin limit of 0", flush=True)
        plan = model.DraftPlan(device)
        plan.append(tokens)                      # no exception: the pass was redone
        assert hip.lib().guffin_hip_resident_enabled() == 0
        assert np.array_equal(plan.read_logits(), want_logits)
        assert same_caches(snapshot(plan, shape), want_caches)
    finally:
        hip.set_spin_limit(1 << 20)
        hip.set_forward_mode(0)                  # an explicit choice enables the resident form again
    assert hip.lib().guffin_hip_resident_enabled() == 1


def test_truncate_and_abort_outside_a_transaction(hip, scaled_world):
    """gemma3_draft.mm:1283-1312: truncating to the current position is always admitted and changes nothing; an
    abort with no transaction open poisons the plan."""
    from guffin_amd import model
    shape, host, device = scaled_world
    plan = model.DraftPlan(device)
    plan.append(stream(5))
    before = snapshot(plan, shape)
    assert plan.can_truncate(5) and not plan.can_truncate(4) and not plan.can_truncate(6)
    plan.truncate(5)
    assert plan.position == 5 and same_caches(snapshot(plan, shape), before)
    refuses(hip, lambda: plan.truncate(4), -6)
    assert not plan.poisoned
    refuses(hip, plan.abort_transaction, -6)
    assert plan.poisoned
    refuses(hip, lambda: plan.append([ROOT]), -6)
    plan.reset()
    plan.append([ROOT])
    assert plan.position == 1 and not plan.poisoned


def test_logits_and_proposals_at_a_frontier_a_transaction_went_back_to(hip, scaled_world):
    """gemma3_draft.mm:984-992: inside a transaction the head projects from the kept final state of the row at the
    frontier, so after a truncate or a shorter commit logits can be read and proposals drafted without another
    token; each equals a plain replay of the kept tokens bit for bit."""
    from guffin_amd import model
    shape, host, device = scaled_world
    prompt = stream(20)
    words = [0] * 23
    replica = model.DeviceModel.from_host(host)         # the same weights over rings of its own, for the replays

    def replay_logits(tokens):
        fresh = model.DraftPlan(replica)
        fresh.append(tokens)
        return fresh.read_logits().copy(), fresh

    plan = model.DraftPlan(device)
    plan.append(prompt)
    plan.begin_transaction()
    plan.append([ROOT])
    drafted = plan.propose(words[:4], greedy(hip))
    assert plan.materialized_position == 24 and plan.position == 25
    plan.truncate(23)                                   # keeps ROOT and two drafts, all of them run
    assert plan.position == 23 and plan.materialized_position == 23 and not plan.poisoned
    want, fresh = replay_logits(prompt + [ROOT] + drafted[:2])
    assert np.array_equal(plan.read_logits().view(np.uint32), want.view(np.uint32))
    fresh.begin_transaction()
    again = plan.propose(words[:2], greedy(hip))        # drafts from the truncated frontier
    assert again == fresh.propose(words[:2], greedy(hip)) and again[0] == drafted[2]
    plan.truncate(21)                                   # back to ROOT alone
    want, _ = replay_logits(prompt + [ROOT])
    assert np.array_equal(plan.read_logits().view(np.uint32), want.view(np.uint32))
    plan.truncate(20)                                   # back to where the transaction began
    want, _ = replay_logits(prompt)
    assert np.array_equal(plan.read_logits().view(np.uint32), want.view(np.uint32))
    plan.append([ROOT])
    drafted = plan.propose(words[:3], greedy(hip))
    plan.commit_prefix(22)                              # a shorter commit: ROOT and the first draft
    assert not plan.transaction_active and plan.position == 22 and plan.materialized_position == 22
    want, _ = replay_logits(prompt + [ROOT, drafted[0]])
    assert np.array_equal(plan.read_logits().view(np.uint32), want.view(np.uint32))
    plan.begin_transaction()
    assert plan.propose(words[:1], greedy(hip)) == [drafted[1]]
    plan.abort_transaction()
    assert np.array_equal(plan.read_logits().view(np.uint32), want.view(np.uint32)) and not plan.poisoned


def test_a_frontier_with_no_pass_is_a_state_error_that_poisons_nothing(hip, scaled_world):
    from guffin_amd import model
    shape, host, device = scaled_world
    plan = model.DraftPlan(device)
    plan.begin_transaction()
    refuses(hip, lambda: plan.propose([0], greedy(hip)), -6)      # nothing materialized
    refuses(hip, plan.read_logits, -6)
    assert not plan.poisoned
    plan.append([ROOT])
    assert plan.propose([0, 0], greedy(hip)) and not plan.poisoned


def test_the_transaction_capacity_is_the_callers(hip, scaled_world):
    """The reference's constructor takes the transaction capacity (gemma3_draft.mm:648-657: at least the horizon
    + 2); here it also has to fit the smallest ring, 64 rows in this world."""
    from guffin_amd import model
    shape, host, device = scaled_world
    for rows in (24, 65, 1 << 20):
        with pytest.raises(ValueError):
            model.DraftPlan(device, transaction_rows=rows)
    plan = model.DraftPlan(device, transaction_rows=48)
    plan.append(stream(70))                              # beyond the local window: the transaction overwrites live ring rows
    before, logits = snapshot(plan, shape), plan.read_logits().copy()
    plan.begin_transaction()
    plan.append(stream(40))
    refuses(hip, lambda: plan.append(stream(9)), -4)     # 49 rows
    plan.append(stream(8))
    assert plan.position == 118
    plan.truncate(100)
    want = model.DraftPlan(model.DeviceModel.from_host(host))     # the same weights over rings of its own
    want.append(stream(70) + stream(40)[:30])
    assert np.array_equal(plan.read_logits().view(np.uint32), want.read_logits().view(np.uint32))
    assert same_caches(snapshot(plan, shape), snapshot(want, shape))
    plan.abort_transaction()
    assert plan.position == 70 and same_caches(snapshot(plan, shape), before)
    assert np.array_equal(plan.read_logits().view(np.uint32), logits.view(np.uint32))
