"""The target on the device against the reference's dyadic six-block fixture (tests/target_fixture.py), on the
sequences of the reference's own target tests (tests/engine/gemma3_target_runtime_tests.cpp):
  :353-386  twelve tokens one at a time, then the same twelve as one prefill and a continuation, across the wrap
            of the 8-row local rings: logits and cache rows against the independent evaluation, replays bit-equal
  :388-462  prompts of 127, 128, 129 and 257 tokens as one prefill and as chunks of 32: last-row logits and every
            cache row still held agree, rows beyond the prompt keep the NaN pattern the caches were filled with, and a
            decode step continues from either
  :719-790  a V projection scaled from 2^-11 to 2^11: the row's fp32 values are finite, their binary16 narrowing is not;
            the plain pass raises the status bit, the width-two transaction ends and leaves every cache bit
  :515-572  a two-row verify pass at position 7: rows bit-equal to one-row passes, close to the evaluation; both
            rows published and 0, 1 or 2 of them kept: every cache byte as a plain run leaves it, and a decode
            step after the rollback."""
import ctypes as C

import numpy as np
import pytest

import target_fixture as fx

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


@pytest.fixture(scope="module")
def fixture():
    return fx.Fixture()


def fresh(fixture, ring_global=32):
    from guffin_amd import model
    return model.DeviceModel.from_host(fixture.host_model(model, ring_global))


def logits_of(hip, device, hidden, sums):
    sh = device.shape
    return hip.gemv_packed(int(sh.embed_dtype), device.head_tiles, hidden, sums, sh.vocab).cpu().numpy()[:, :fx.VOCAB]


def commit(hip, device, pk, pv, position, rows):
    hip.check(hip.lib().guffin_hip_commit_rows(hip._stream(), C.byref(device.desc), C.c_void_p(pk.data_ptr()),
                                               C.c_void_p(pv.data_ptr()), C.c_void_p(device.ring_k_table.data_ptr()),
                                               C.c_void_p(device.ring_v_table.data_ptr()), None, C.c_uint32(position),
                                               C.c_uint32(rows)))


def decode(hip, device, token, position):
    """One ordinary step: a one-row pass, its row published; returns the logits."""
    import torch
    hidden, sums, pk, pv, status = device.forward(torch.tensor([token], dtype=torch.int32, device="cuda"), position)
    commit(hip, device, pk, pv, position, 1)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    return logits_of(hip, device, hidden, sums)[0]


def prefill(hip, device, tokens, position):
    import torch
    hidden, status = device.prefill(torch.tensor(list(tokens), dtype=torch.int32, device="cuda"), position)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    last = hidden[-1:].contiguous()
    return logits_of(hip, device, last, hip.group_sums(last))[0]


def reader(device):
    def read(layer, position):
        cap = device.ring_k[layer].shape[0]
        return (device.ring_k[layer][position & (cap - 1)].float().cpu().numpy().reshape(-1),
                device.ring_v[layer][position & (cap - 1)].float().cpu().numpy().reshape(-1))
    return read


def caches(device):
    return [(k.clone(), v.clone()) for k, v in zip(device.ring_k, device.ring_v)]


def same_caches(a, b):
    import torch
    return all(torch.equal(ka, kb) and torch.equal(va, vb) for (ka, va), (kb, vb) in zip(a, b))


def test_complete_synthetic_reference_and_wrapped_batch(hip, fixture):
    ref = fx.Reference(fixture)
    scalar = fresh(fixture)
    worst = 0.0
    for i in range(12):
        expected = ref.append(fx.TOKENS[i])
        print("target fixture: scalar token", i, flush=True)
        worst = max(worst, fx.assert_close(decode(hip, scalar, fx.TOKENS[i], i), expected, "scalar logits of token %d" % i))
        if i in (6, 7, 8, 11):
            fx.assert_cache(scalar, ref, i + 1, reader(scalar))
    print("device vs dense evaluation: worst logit error %.2f of the budget" % worst, flush=True)
    batch = fresh(fixture)
    fx.assert_close(prefill(hip, batch, fx.TOKENS[:12], 0), ref.logits[-1], "twelve-row batched logits")
    fx.assert_cache(batch, ref, 12, reader(batch))
    expected = ref.append(fx.TOKENS[12])
    last = prefill(hip, batch, fx.TOKENS[12:], 12)
    fx.assert_close(last, expected, "continuation after the wrapped batch")
    fx.assert_cache(batch, ref, 13, reader(batch))
    replay = fresh(fixture)
    prefill(hip, replay, fx.TOKENS[:12], 0)
    again = prefill(hip, replay, fx.TOKENS[12:], 12)
    assert np.array_equal(again.view(np.uint32), last.view(np.uint32)), "segmented replay changed the logits"
    assert same_caches(caches(replay), caches(batch))


def test_width_two_prefix_publication_and_rollback(hip, fixture):
    import torch
    from guffin_amd import model
    tokens = fx.TOKENS[:9]
    ref = fx.Reference(fixture)
    for token in tokens:
        ref.append(token)
    ordinary = fresh(fixture)
    prefill(hip, ordinary, tokens[:7], 0)
    ordinary_logits = [decode(hip, ordinary, tokens[7 + i], 7 + i) for i in range(2)]
    for retained in range(3):
        print("target fixture: width two, retained", retained, flush=True)
        plan = fresh(fixture)
        prefill(hip, plan, tokens[:7], 0)
        before = caches(plan)
        ticket = model.VerifyTicket(plan, 7 + 4)
        ticket.encode(list(tokens[7:9]), 7)
        ticket.submit()
        assert ticket.complete() == 0
        assert same_caches(caches(plan), before), "a completed pass touched the caches"
        # the pass's rows through the plain entry point: logits of both rows
        hidden, sums, pk, pv, status = plan.forward(torch.tensor(list(tokens[7:9]), dtype=torch.int32, device="cuda"), 7)
        logits = logits_of(hip, plan, hidden, sums)
        for row in range(2):
            assert np.array_equal(logits[row].view(np.uint32), ordinary_logits[row].view(np.uint32)), \
                "width-two target conditionals differ from ordinary logits"
            fx.assert_close(logits[row], ref.logits[7 + row], "verifier row %d" % row)
        kvw = plan.shape.kv_width
        assert torch.equal(ticket.priv_k.view(-1)[:pk.numel()].view(-1, 2, kvw), pk)
        ticket.provisional_commit([0, 1])
        ticket.finalize(retained)
        assert ticket.state == model.TXN_IDLE
        if retained == 0:
            assert same_caches(caches(plan), before), "full rejection did not restore every slot across the wrap"
        fx.assert_cache(plan, ref, 7 + retained, reader(plan))
        check = fresh(fixture)
        prefill(hip, check, tokens[:7], 0)
        for i in range(retained):
            decode(hip, check, tokens[7 + i], 7 + i)
        assert same_caches(caches(plan), caches(check)), "kept rows differ from a plain run's"
        if retained < 2:
            fx.assert_close(decode(hip, plan, tokens[7 + retained], 7 + retained), ref.logits[7 + retained],
                            "decode after the suffix was rolled back")


@pytest.mark.parametrize("count", [127, 128, 129, 257])
def test_bulk_prefill_cache_across_chunk_partitions(hip, fixture, count):
    import torch
    tokens = [(i * 19 + i // 7 + 2) % 32 for i in range(258)]
    batch, segmented = fresh(fixture, 512), fresh(fixture, 512)
    for plan in (batch, segmented):
        for k, v in zip(plan.ring_k, plan.ring_v):
            k.view(torch.int16).fill_(0x7e00)
            v.view(torch.int16).fill_(0x7e00)
    whole = prefill(hip, batch, tokens[:count], 0)
    first = 0
    while first < count:
        rows = min(32, count - first)
        last = prefill(hip, segmented, tokens[first:first + rows], first)
        first += rows
    fx.assert_close(whole, last, "chunk partition logits")

    def check(committed):
        for layer in range(fx.LAYERS):
            cap = batch.ring_k[layer].shape[0]
            held = range(max(0, committed - cap), committed)
            for a, b in ((batch.ring_k[layer], segmented.ring_k[layer]), (batch.ring_v[layer], segmented.ring_v[layer])):
                a, b = a.float().cpu().numpy().reshape(cap, -1), b.float().cpu().numpy().reshape(cap, -1)
                for position in held:
                    fx.assert_close(a[position & (cap - 1)], b[position & (cap - 1)], "committed row %d of block %d" % (position, layer),
                                    3e-4, 3e-4 + 2.0 ** -10)
            if committed < cap:
                for ring in (batch.ring_k[layer], batch.ring_v[layer], segmented.ring_k[layer], segmented.ring_v[layer]):
                    rest = ring.view(torch.int16).reshape(cap, -1)[committed:]
                    assert bool((rest == 0x7e00).all()), "a row beyond the prompt was written"

    check(count)
    fx.assert_close(decode(hip, batch, tokens[count], count), decode(hip, segmented, tokens[count], count),
                    "ordinary decode after the partitioned prompt")
    check(count + 1)


def test_f16_cache_overflow_preserves_transaction_boundaries(hip, fixture):
    import copy
    import torch
    from guffin_amd import model
    KV_NONFINITE = 8
    broken = copy.copy(fixture)
    broken.packed = dict(fixture.packed)
    embd = fixture.packed["token_embd.weight"].copy()
    embd[:210] = 0                                      # token 0 embeds to zero: a prefix with finite zero K/V
    broken.packed["token_embd.weight"] = embd
    v = fixture.packed["blk.0.attn_v.weight"].copy().reshape(-1, 210)
    v[:, 208], v[:, 209] = 0x00, 0x68                   # d = 2^11 instead of 2^-11
    broken.packed["blk.0.attn_v.weight"] = v.reshape(-1)
    host = broken.host_model(model)

    def plan_with_prefix():
        plan = model.DeviceModel.from_host(host)
        prefill(hip, plan, [0], 0)
        for k, vv in zip(plan.ring_k, plan.ring_v):
            assert float(k[0].float().abs().max()) == 0.0 and float(vv[0].float().abs().max()) == 0.0
        return plan

    plan = plan_with_prefix()
    hidden, sums, pk, pv, status = plan.forward(torch.tensor([2], dtype=torch.int32, device="cuda"), 1)
    torch.cuda.synchronize()
    assert int(status.item()) & KV_NONFINITE, "a non-finite narrowed V row went unreported"
    assert not bool(torch.isfinite(pv[0].float()).all())

    plan = plan_with_prefix()
    before = caches(plan)
    ticket = model.VerifyTicket(plan, 8)
    ticket.encode([2, 7], 1)
    ticket.submit()
    with pytest.raises(hip.GuffinError) as err:
        ticket.complete()
    assert err.value.code == -7                          # numerical fault: the transaction is dropped
    assert ticket.state == model.TXN_IDLE
    assert same_caches(caches(plan), before), "the overflowing pass changed a cache bit"
