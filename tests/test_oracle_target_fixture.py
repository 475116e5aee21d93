"""The oracle's target pass on the reference's dyadic six-block fixture (tests/target_fixture.py, after
tests/engine/gemma3_target_runtime_tests.cpp:353-386): thirteen tokens one at a time across the wrap of the
8-row local rings, logits and cache rows against the independent evaluation from dense values, with the
reference's tolerances; and the packed blocks against the dense copy, exactly."""
import numpy as np

import target_fixture as fx


def test_packed_blocks_decode_to_the_dense_values_exactly(gfo):
    f = fx.Fixture()
    for name, packed in f.packed.items():
        six = name.endswith(("attn_v.weight", "ffn_down.weight", "token_embd.weight"))
        got = gfo.dequant(2 if six else 1, packed)
        assert np.array_equal(got, f.dense[name].reshape(-1)), name      # as values: a zero quant under a negative scale is -0


def test_oracle_forward_equals_the_dense_evaluation(gfo):
    from guffin_amd import model
    f = fx.Fixture()
    host = f.host_model(model)
    ref = fx.Reference(f)
    worst = 0.0
    for position, token in enumerate(fx.TOKENS):
        hidden, pk, pv = gfo.forward(host, np.array([token], np.uint32), position, threads=4)
        host.commit(pk, pv, position, 1)
        logits = gfo.gemv(host.shape.embed_dtype, host.embed, hidden, fx.PADDED_VOCAB, threads=1)[0][:fx.VOCAB]
        worst = max(worst, fx.assert_close(logits, ref.append(token), "logits of token %d" % position))
        if position + 1 in (7, 8, 9, 12, 13):
            def read(layer, p):
                cap = host.ring_k[layer].shape[0]
                return host.ring_k[layer][p & (cap - 1)].astype(np.float32), host.ring_v[layer][p & (cap - 1)].astype(np.float32)
            fx.assert_cache(host, ref, position + 1, read)
    print("oracle vs dense evaluation: worst logit error %.2f of the budget" % worst)
    assert np.std(ref.logits[-1]) > 0.05      # the fixture's logits spread
