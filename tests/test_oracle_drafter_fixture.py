"""The oracle's whole drafter pass on the reference's closed-form fixture (tests/drafter_fixture.py, after
tests/engine/gemma3_draft_tests.cpp:31-186): full 270M geometry, four tokens one at a time, logits and cache
rows against the independent scalar evaluation with the reference's tolerances."""
import numpy as np

import drafter_fixture as fx


def test_oracle_forward_equals_the_closed_form(gfo):
    from guffin_amd import model
    host = fx.host_model(model)
    ref = fx.Reference()
    for position, token in enumerate(fx.TOKENS):
        hidden, pk, pv = gfo.forward(host, np.array([token], np.uint32), position, threads=8)
        host.commit(pk, pv, position, 1)
        ref.step(token)
        if position >= 2:      # the reference compares after the three-token prefill and after the decode step
            distinct = gfo.gemv(host.shape.embed_dtype, host.embed[:53 * (fx.WIDTH // 32) * 34], hidden, 53, threads=1)[0]
            worst = fx.assert_logits_close(distinct, ref.logits()[:53], "oracle logits at %d" % position)
            print("oracle vs closed form, position %d: max abs logit error %.3g" % (position, worst))
    for layer in range(fx.LAYERS):
        k = host.ring_k[layer][:4].astype(np.float32)
        v = host.ring_v[layer][:4].astype(np.float32)
        fx.assert_cache_close(k, np.stack(ref.keys[layer]), "K of block %d" % layer)
        fx.assert_cache_close(v, np.stack(ref.values[layer]), "V of block %d" % layer)


def test_the_fixture_is_not_degenerate():
    """The closed form must exercise every operator: attention over more than one token with unequal weights,
    a non-trivial rotation, logits that spread."""
    ref = fx.Reference()
    for token in fx.TOKENS:
        ref.step(token)
    logits = ref.logits()[:53]
    assert logits.std() > 1.0 and len(np.unique(logits)) == 53
    assert all(np.abs(np.stack(ref.keys[l])[3] - np.stack(ref.keys[l])[0]).max() > 0.1 for l in range(fx.LAYERS))


def test_context_endpoint_with_a_zero_prefix(gfo):
    """tests/engine/gemma3_draft_tests.cpp:483-496: one token at the last position of a 32768-token context whose
    earlier cache rows are zero, against the closed form for that case (global layers attend over all 32767 zero
    rows, local ones over 511)."""
    from guffin_amd import model
    last = 32768 - 1
    host = fx.host_model(model, ring_global=32768)
    ref = fx.Reference()
    ref.position = last
    ref.keys = [[None] * last for _ in range(fx.LAYERS)]      # placeholders: the closed form never reads them
    ref.values = [[None] * last for _ in range(fx.LAYERS)]
    ref.step(119, zero_prefix=True)
    hidden, pk, pv = gfo.forward(host, np.array([119], np.uint32), last, threads=8)
    distinct = gfo.gemv(host.shape.embed_dtype, host.embed[:53 * (fx.WIDTH // 32) * 34], hidden, 53, threads=1)[0]
    fx.assert_logits_close(distinct, ref.logits()[:53], "logits at the context endpoint")
    for layer in range(fx.LAYERS):
        fx.assert_cache_close(pk[layer, 0].view(np.float16).astype(np.float32), ref.keys[layer][-1], "endpoint K of block %d" % layer)
        fx.assert_cache_close(pv[layer, 0].view(np.float16).astype(np.float32), ref.values[layer][-1], "endpoint V of block %d" % layer)
