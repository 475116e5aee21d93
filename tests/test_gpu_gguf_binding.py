"""A Gemma-3-shaped model written as a GGUF file image, read back by the library's reader and bound
to the device: the forward pass equals the one of the same weights bound directly, bit for bit.
Tensor and metadata names follow the reference (src/engine/gemma_model.cpp:36-116,
src/engine/model.cpp:330-390)."""
import struct
from dataclasses import replace

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GGUF_TYPE = {0: 8, 1: 12, 2: 14}      # library dtype (Q8_0, Q4_K, Q6_K) -> GGUF tensor type id


def gguf_string(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(host, alignment=64):
    """Serialises a HostModel the way a converter lays a Gemma 3 file out."""
    sh = host.shape
    md = [("general.architecture", 8, "gemma3"), ("general.alignment", 4, alignment),
          ("gemma3.context_length", 4, 8192), ("gemma3.embedding_length", 4, sh.hidden),
          ("gemma3.block_count", 4, sh.layers), ("gemma3.feed_forward_length", 4, sh.ffn),
          ("gemma3.attention.head_count", 4, sh.q_heads), ("gemma3.attention.head_count_kv", 4, sh.kv_heads),
          ("gemma3.attention.key_length", 4, sh.head_dim), ("gemma3.attention.value_length", 4, sh.head_dim),
          ("gemma3.attention.sliding_window", 4, sh.sliding_window),
          ("gemma3.attention.layer_norm_rms_epsilon", 6, sh.eps), ("gemma3.rope.freq_base", 6, sh.global_base),
          ("gemma3.rope.scaling.type", 8, "linear"), ("gemma3.rope.scaling.factor", 6, 1.0 / sh.global_scale),
          ("tokenizer.ggml.tokens", 9, ["<s>", "</s>"])]
    tensors = [("token_embd.weight", [sh.hidden, sh.vocab], GGUF_TYPE[sh.embed_dtype], host.embed),
               ("output_norm.weight", [sh.hidden], 0, host.out_norm)]
    names = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")
    norms = ("attn_norm", "attn_q_norm", "attn_k_norm", "post_attention_norm", "ffn_norm", "post_ffw_norm")
    for l in range(sh.layers):
        for i, (n, (K, N)) in enumerate(zip(names, sh.proj_shapes())):
            tensors.append(("blk.%d.%s.weight" % (l, n), [K, N], GGUF_TYPE[sh.dtypes_of(l)[i]], host.w[l][i]))
        for i, n in enumerate(norms):
            tensors.append(("blk.%d.%s.weight" % (l, n), [host.norm[l][i].size], 0, host.norm[l][i]))
    out = bytearray(b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(md)))
    for key, t, v in md:
        out += gguf_string(key) + struct.pack("<I", t)
        if t == 8:
            out += gguf_string(v)
        elif t == 4:
            out += struct.pack("<I", v)
        elif t == 6:
            out += struct.pack("<f", v)
        else:
            out += struct.pack("<IQ", 8, len(v)) + b"".join(gguf_string(x) for x in v)
    offset, payloads = 0, []
    for name, dims, type_id, array in tensors:
        raw = np.ascontiguousarray(array).view(np.uint8).tobytes()
        out += gguf_string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", type_id, offset)
        payloads.append((offset, raw))
        offset = (offset + len(raw) + alignment - 1) // alignment * alignment
    out += b"\0" * (-len(out) % alignment)
    start = len(out)
    for off, raw in payloads:
        out += b"\0" * (start + off - len(out)) + raw
    return np.frombuffer(bytes(out), np.uint8)


@pytest.mark.parametrize("kind", ["target", "drafter"])
def test_model_bound_from_a_gguf_image_runs_like_the_direct_binding(kind):
    import torch
    from guffin_amd import gguf, hip, model
    hip.init(0)
    base = model.GEMMA3_12B if kind == "target" else model.GEMMA3_270M
    shape = replace(base, layers=7, vocab=2048, ring_global=1024, ring_local=base.ring_local)
    host = model.HostModel(shape, seed=5, position=0)
    image = write_gguf(host)
    reader = gguf.Reader(image)
    assert reader.info.alignment == 64 and reader.metadata()["general.architecture"] == "gemma3"
    assert len(reader.tensors()) == 2 + 13 * shape.layers
    bound = model.DeviceModel.from_gguf(reader, ring_local=shape.ring_local, ring_global=shape.ring_global)
    direct = model.DeviceModel.from_host(host)
    assert replace(bound.shape, eps=shape.eps) == shape and abs(bound.shape.eps - shape.eps) < 1e-12
    tokens = torch.tensor([17, 1999], dtype=torch.int32, device="cuda")
    got = bound.forward(tokens, 0)
    want = direct.forward(tokens, 0)
    torch.cuda.synchronize()
    assert int(got[4].item()) == 0 and int(want[4].item()) == 0
    for g, w in zip(got[:4], want[:4]):
        assert torch.equal(g.view(torch.uint8), w.view(torch.uint8))


def test_blocks_of_mixed_formats_bind_matrix_by_matrix(gfo):
    """A Q4_K_M file keeps attn_v and ffn_down in Q6_K in some blocks and in Q4_K in others; each matrix is
    bound in its own format (src/engine/gemma_model.cpp:140-148) and the pass agrees with the oracle on the
    same canonical weights."""
    import torch
    from guffin_amd import gguf, hip, model
    hip.init(0)
    Q4, Q6 = model.Q4_K, model.Q6_K
    per_layer = ((Q4, Q4, Q6, Q4, Q4, Q4, Q6), (Q4, Q4, Q4, Q4, Q4, Q4, Q4), (Q4, Q4, Q6, Q4, Q4, Q4, Q4),
                 (Q4, Q4, Q4, Q4, Q4, Q4, Q6), (Q4, Q4, Q4, Q4, Q6, Q4, Q6), (Q4, Q4, Q6, Q4, Q4, Q4, Q6))
    shape = replace(model.GEMMA3_12B, layers=6, vocab=2048, ring_global=1024, layer_dtypes=per_layer)
    host = model.HostModel(shape, seed=8, position=0)
    bound = model.DeviceModel.from_gguf(gguf.Reader(write_gguf(host)), ring_local=shape.ring_local,
                                        ring_global=shape.ring_global)
    assert bound.shape.layer_dtypes == per_layer
    assert [[bound.layers[l].dtype[i] for i in range(7)] for l in range(6)] == [list(r) for r in per_layer]
    assert bound.shape.body_weight_bytes() == sum(host.w[l][i].size for l in range(6) for i in range(7))
    tokens = torch.tensor([17, 1999], dtype=torch.int32, device="cuda")
    got = bound.forward(tokens, 0)
    torch.cuda.synchronize()
    assert int(got[4].item()) == 0
    want, wk, wv = gfo.forward(host, [17, 1999], 0, threads=8)
    hidden = got[0].cpu().numpy().astype(np.float64)
    scale = np.sqrt((want.astype(np.float64) ** 2).mean(-1, keepdims=True))
    assert np.max(np.abs(hidden - want) / scale) <= 1e-3
    direct = model.DeviceModel.from_host(host).forward(tokens, 0)
    torch.cuda.synchronize()
    assert torch.equal(got[0].view(torch.uint8), direct[0].view(torch.uint8))


def test_binding_refuses_files_that_do_not_fit_the_model():
    from guffin_amd import gguf, hip, model
    hip.init(0)
    shape = replace(model.GEMMA3_270M, layers=2, vocab=512, ring_global=512)
    host = model.HostModel(shape, seed=6, position=0)
    host.norm[1][0] = host.norm[1][0][:-1].copy()          # a norm of the wrong width
    with pytest.raises(ValueError):
        model.DeviceModel.from_gguf(gguf.Reader(write_gguf(host)), ring_global=512)
