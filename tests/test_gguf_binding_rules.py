"""guffin_gguf_bind_gemma3 on the cases of the reference's weight-binding tests
(tests/engine/gemma3_model_plan_tests.cpp:96-112, 141-157; rules src/engine/gemma_model.cpp:72-177): a valid
file binds every tensor by name; an unpaired head geometry, a context shorter than the window, a missing Q/K
norm, a matrix of another's shape and a missing tensor are refused with the reference's error class and detail."""
from dataclasses import replace

import numpy as np
import pytest

from gguf_image import write_gguf


def config_for(gguf, shape, target, **changes):
    c = gguf.Gemma3Config()
    c.block_count, c.embedding_length, c.feed_forward_length, c.vocab_size = shape.layers, shape.hidden, shape.ffn, shape.vocab
    c.attention_head_count, c.attention_head_count_kv = shape.q_heads, shape.kv_heads
    c.attention_key_length = c.attention_value_length = shape.head_dim
    c.sliding_window, c.context_length, c.attention_global_layer_period = shape.sliding_window, 8192, 6
    c.uses_qk_norm, c.uses_tied_output_weight, c.target_geometry = 1, 0, 1 if target else 0
    c.rms_norm_epsilon, c.attention_logit_softcap, c.final_logit_softcap = 1e-6, 0.0, 0.0
    c.rope_freq_base, c.local_rope_freq_base, c.rope_freq_scale = 1e6, 1e4, 0.125
    for k, v in changes.items():
        setattr(c, k, v)
    return c


@pytest.fixture(scope="module")
def world():
    from guffin_amd import gguf, model
    shape = replace(model.GEMMA3_12B, layers=2, vocab=512, hidden=256, ffn=512, q_heads=2, kv_heads=1)
    return gguf, model, shape, model.HostModel(shape, seed=2, position=0)


def refused(gguf, image, config, code, fragment):
    with pytest.raises(gguf.BindError) as info:
        gguf.Reader(image).bind_gemma3(config)
    assert info.value.code == code and fragment in info.value.detail, info.value


def test_a_valid_file_binds_every_tensor_by_name(world):
    gguf, model, shape, host = world
    reader = gguf.Reader(write_gguf(host))
    binding, blocks = reader.bind_gemma3(config_for(gguf, shape, target=True))
    assert reader.tensor_at(binding.token_embedding)["name"] == "token_embd.weight"
    assert reader.tensor_at(binding.output_norm)["name"] == "output_norm.weight"
    assert binding.tied_output == 1 and binding.output == binding.token_embedding
    for l in range(shape.layers):
        for i, m in enumerate(model.DeviceModel.GGUF_MATRICES):
            t = reader.tensor_at(blocks[l].matrix[i])
            assert t["name"] == "blk.%d.%s.weight" % (l, m) and t["dims"] == list(shape.proj_shapes()[i])
            assert blocks[l].type_id[i] == t["type_id"]
        for i, n in enumerate(model.DeviceModel.GGUF_NORMS):
            assert reader.tensor_at(blocks[l].norm[i])["name"] == "blk.%d.%s.weight" % (l, n)
    # an output matrix of its own is bound instead of the embedding, unless the model says the output is tied
    extra = [("output.weight", [shape.hidden, shape.vocab], 14, host.embed)]
    binding, _ = gguf.Reader(write_gguf(host, extra=extra)).bind_gemma3(config_for(gguf, shape, target=True))
    assert binding.tied_output == 0 and binding.output != binding.token_embedding
    refused(gguf, write_gguf(host, extra=extra), config_for(gguf, shape, True, uses_tied_output_weight=1), "invalid_tensor",
            "tied output must alias token_embd.weight")


def test_the_references_refusals(world):
    gguf, model, shape, host = world
    image = write_gguf(host)
    good = lambda **kw: config_for(gguf, shape, True, **kw)
    refused(gguf, image, good(attention_head_count=4), "invalid_tensor", "paired GQA")
    refused(gguf, image, good(context_length=4), "invalid_tensor", "local attention window")
    refused(gguf, write_gguf(host, drop=("blk.0.attn_k_norm.weight",)), good(), "missing_tensor", "attn_k_norm.weight")
    refused(gguf, write_gguf(host, drop=("blk.1.ffn_down.weight",)), good(), "missing_tensor", "blk.1.ffn_down.weight")
    refused(gguf, write_gguf(host, drop=("token_embd.weight",)), good(), "missing_tensor", "token_embd.weight")
    # attn_q written with attn_k's shape (the reference swaps the views)
    k_shape = list(shape.proj_shapes()[1])
    wrong = write_gguf(host, reshape={"blk.0.attn_q.weight": k_shape})
    refused(gguf, wrong, good(), "invalid_tensor", "blk.0.attn_q.weight: expected native Q4_K/Q6_K GGUF matrix [256, 512]")
    for bad in (dict(attention_logit_softcap=50.0), dict(final_logit_softcap=30.0), dict(attention_global_layer_period=3),
                dict(uses_qk_norm=0), dict(rms_norm_epsilon=0.0), dict(local_rope_freq_base=-1.0),
                dict(rope_freq_scale=float("nan")), dict(attention_value_length=128), dict(block_count=0)):
        refused(gguf, image, good(**bad), "invalid_tensor", "Gemma 3 execution configuration")
    # more blocks in the configuration than in the file: the lookup fails first; a file that has them is refused by the rule
    refused(gguf, image, good(block_count=65), "missing_tensor", "blk.2.attn_norm.weight")
    deep = replace(shape, layers=65)
    refused(gguf, write_gguf(model.HostModel(deep, seed=2, position=0)), config_for(gguf, deep, True), "invalid_tensor",
            "at most 64 layers")


def test_tensor_formats_and_widths(world):
    gguf, model, shape, host = world
    good = config_for(gguf, shape, True)
    refused(gguf, write_gguf(host, retype={"blk.1.attn_norm.weight": 1}), good, "invalid_tensor",
            "blk.1.attn_norm.weight: expected F32 norm with width 256")
    refused(gguf, write_gguf(host, reshape={"blk.0.attn_q_norm.weight": [128]}), good, "invalid_tensor", "expected F32 norm with width 256")
    refused(gguf, write_gguf(host, retype={"token_embd.weight": 12}, reshape=None), good, "invalid_tensor",
            "token_embd.weight: expected native Q6_K")
    # the drafter's formats are admitted only without the target's geometry, and never mixed inside a block
    d_shape = replace(model.GEMMA3_270M, layers=2, vocab=512)
    d_host = model.HostModel(d_shape, seed=3, position=0)
    d_image = write_gguf(d_host)
    gguf.Reader(d_image).bind_gemma3(config_for(gguf, d_shape, target=False))
    refused(gguf, d_image, config_for(gguf, d_shape, target=True), "invalid_tensor", "paired GQA")
    wide = replace(d_shape, hidden=512, ffn=1024, layer_dtypes=((0,) * 7, (1, 0, 0, 0, 0, 0, 0)))   # block 1: a Q4_K attn_q among Q8_0
    refused(gguf, write_gguf(model.HostModel(wide, seed=3, position=0)), config_for(gguf, wide, target=False), "invalid_tensor",
            "mixes 32-weight and 256-weight formats")


def test_which_refusal_wins_when_two_things_are_wrong(world):
    """bind_gemma_model_weights looks every tensor up before validate_gemma3_model_weights sees anything
    (src/engine/gemma_model.cpp:72-103): a missing tensor wins over any invalid one and over the configuration,
    blocks are looked up before token_embd / output_norm and inside a block in the order of the reference's
    initialisers (:38-68: attn_norm, post_attention_norm, q, k, v, o, q_norm, k_norm, ffn_norm, post_ffw_norm,
    gate, up, down).  Validation then runs token_embd, output, output_norm, and per block attn_norm,
    post_attention_norm, q_norm, k_norm, q, k, v, o, ffn_norm, post_ffw_norm, gate, up, down (:149-175)."""
    gguf, model, shape, host = world
    good = lambda **kw: config_for(gguf, shape, True, **kw)
    # missing beats invalid, wherever each sits
    refused(gguf, write_gguf(host, drop=("blk.1.ffn_down.weight",), retype={"token_embd.weight": 12}), good(),
            "missing_tensor", "blk.1.ffn_down.weight")
    refused(gguf, write_gguf(host, drop=("output_norm.weight",), reshape={"blk.0.attn_q_norm.weight": [128]}), good(),
            "missing_tensor", "output_norm.weight")
    # missing beats a configuration that would be refused
    refused(gguf, write_gguf(host, drop=("blk.0.attn_v.weight",)), good(attention_logit_softcap=50.0),
            "missing_tensor", "blk.0.attn_v.weight")
    refused(gguf, write_gguf(host, drop=("token_embd.weight",)), good(context_length=4), "missing_tensor", "token_embd.weight")
    # two missing tensors: blocks before the model's own tensors, block 0 before block 1, initialiser order inside a block
    refused(gguf, write_gguf(host, drop=("token_embd.weight", "blk.1.ffn_up.weight")), good(), "missing_tensor", "blk.1.ffn_up.weight")
    refused(gguf, write_gguf(host, drop=("blk.1.attn_norm.weight", "blk.0.ffn_down.weight")), good(), "missing_tensor", "blk.0.ffn_down.weight")
    refused(gguf, write_gguf(host, drop=("blk.0.attn_q_norm.weight", "blk.0.attn_output.weight")), good(),
            "missing_tensor", "blk.0.attn_output.weight")
    refused(gguf, write_gguf(host, drop=("blk.0.attn_q_norm.weight", "blk.0.ffn_norm.weight")), good(),
            "missing_tensor", "blk.0.attn_q_norm.weight")
    refused(gguf, write_gguf(host, drop=("blk.0.post_attention_norm.weight", "blk.0.attn_q.weight")), good(),
            "missing_tensor", "blk.0.post_attention_norm.weight")
    # without Q/K norms in the configuration their names are not looked up: the configuration is what is refused
    refused(gguf, write_gguf(host, drop=("blk.0.attn_q_norm.weight",)), good(uses_qk_norm=0), "invalid_tensor",
            "Gemma 3 execution configuration")
    # the configuration beats any invalid tensor; among invalid tensors the validation order decides
    refused(gguf, write_gguf(host, retype={"token_embd.weight": 12}), good(rms_norm_epsilon=0.0), "invalid_tensor",
            "Gemma 3 execution configuration")
    refused(gguf, write_gguf(host, retype={"token_embd.weight": 12, "blk.0.attn_norm.weight": 1}), good(), "invalid_tensor",
            "token_embd.weight: expected native Q6_K")
    k_shape = list(shape.proj_shapes()[1])
    refused(gguf, write_gguf(host, reshape={"blk.0.attn_q.weight": k_shape, "blk.0.attn_k_norm.weight": [128]}), good(),
            "invalid_tensor", "blk.0.attn_k_norm.weight: expected F32 norm")
    refused(gguf, write_gguf(host, reshape={"blk.0.attn_q.weight": k_shape}, retype={"blk.0.ffn_norm.weight": 1}), good(),
            "invalid_tensor", "blk.0.attn_q.weight: expected native")
    refused(gguf, write_gguf(host, retype={"blk.0.post_ffw_norm.weight": 1, "blk.1.attn_norm.weight": 1}), good(),
            "invalid_tensor", "blk.0.post_ffw_norm.weight")
    refused(gguf, write_gguf(host, retype={"output_norm.weight": 1, "blk.0.attn_norm.weight": 1}), good(), "invalid_tensor",
            "output_norm.weight: expected F32 norm")


def test_the_width_refusal_keeps_the_references_wording(world):
    gguf, model, shape, host = world
    wide = config_for(gguf, shape, False, attention_head_count=1 << 25, attention_head_count_kv=1 << 25,
                      attention_key_length=256, attention_value_length=256)
    refused(gguf, write_gguf(host), wide, "invalid_tensor", "Gemma 3 attention width exceeds Metal indexing range")
