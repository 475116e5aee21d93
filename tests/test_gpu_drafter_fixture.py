"""The drafter on the device against the reference's closed-form fixture (tests/drafter_fixture.py, after
tests/engine/gemma3_draft_tests.cpp:31-186, `synthetic_forward`): full 270M geometry through the lifecycle
entry points — a three-token prefix, one decode step, logits over all 262144 tokens and the cache rows of all
18 blocks within the reference's tolerances of the independent scalar evaluation, and a token-by-token replay
bit-equal to the first run."""
import numpy as np
import pytest

import drafter_fixture as fx

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    yield module
    module.set_forward_mode(0)


@pytest.mark.parametrize("mode", [0, 1])     # the resident pass (the default for this model), then one launch per operator
def test_synthetic_forward_equals_the_closed_form(hip, mode):
    from guffin_amd import model
    hip.set_forward_mode(mode)
    device = model.DeviceModel.from_host(fx.host_model(model))
    plan = model.DraftPlan(device)
    ref = fx.Reference()
    plan.append(list(fx.TOKENS[:3]))
    for token in fx.TOKENS[:3]:
        ref.step(token)
    worst = fx.assert_logits_close(plan.read_logits(), ref.logits(), "prefix logits")
    print("device vs closed form after the prefix: max abs logit error %.3g" % worst, flush=True)
    plan.append([fx.TOKENS[3]])
    ref.step(fx.TOKENS[3])
    actual = plan.read_logits()
    worst = fx.assert_logits_close(actual, ref.logits(), "decode logits")
    print("device vs closed form after the decode step: max abs logit error %.3g" % worst, flush=True)
    for layer in range(fx.LAYERS):
        k, v = (a.view(np.float16).astype(np.float32) for a in plan.read_cache(layer, 0, 4))   # fp16 rows as stored
        fx.assert_cache_close(k, np.stack(ref.keys[layer]), "K of block %d" % layer)
        fx.assert_cache_close(v, np.stack(ref.values[layer]), "V of block %d" % layer)
    plan.reset()
    for token in fx.TOKENS:
        plan.append([token])
    assert np.array_equal(plan.read_logits().view(np.uint32), actual.view(np.uint32)), "scalar and batched replay differ"
    hip.set_forward_mode(0)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("position,capacity", [(768, 1024), (32767, 32768)])
def test_context_endpoint_with_a_zero_prefix(hip, mode, position, capacity):
    """tests/engine/gemma3_draft_tests.cpp:471-496: one token behind `position` zero cache rows (768: a session-sized
    context; 32767: the last row of the model's context), logits and that row's K/V against the closed form; one
    row further is refused before anything runs."""
    import torch
    from guffin_amd import model
    hip.set_forward_mode(mode)
    device = model.DeviceModel.from_host(fx.host_model(model, ring_global=capacity))
    ref = fx.Reference()
    ref.position = position
    ref.keys = [[None] * position for _ in range(fx.LAYERS)]
    ref.values = [[None] * position for _ in range(fx.LAYERS)]
    token = 111 if position == 768 else 119
    ref.step(token, zero_prefix=True)
    hidden, sums, pk, pv, status = device.forward(torch.tensor([token], dtype=torch.int32, device="cuda"), position)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    logits = hip.gemv_packed(int(device.shape.embed_dtype), device.head_tiles, hidden, sums, fx.VOCAB).cpu().numpy()[0]
    worst = fx.assert_logits_close(logits, ref.logits(), "logits behind %d zero rows" % position)
    print("zero prefix of %d rows, mode %d: max abs logit error %.3g" % (position, mode, worst), flush=True)
    for layer in range(fx.LAYERS):
        fx.assert_cache_close(pk[layer, 0].float().cpu().numpy(), ref.keys[layer][-1], "endpoint K of block %d" % layer)
        fx.assert_cache_close(pv[layer, 0].float().cpu().numpy(), ref.values[layer][-1], "endpoint V of block %d" % layer)
    if position + 1 == capacity:
        with pytest.raises(hip.GuffinError) as err:
            device.forward(torch.tensor([token], dtype=torch.int32, device="cuda"), position + 1)
        assert err.value.code == -4                       # capacity: nothing was enqueued
    hip.set_forward_mode(0)
